// Kernel parameter blocks shared by the host launcher and the device code.
#pragma once
#include <stdint.h>

namespace sba {

struct TensorRef {     // [batch,] head, token, head_dim; element strides; head_dim stride 1
  void* ptr;
  int64_t sb, sh, st;
};
struct VectorRef {     // [batch,] head, token
  void* ptr;
  int64_t sb, sh, st;
};

// Tile descriptor produced by the scheduler kernel.
struct Tile {
  int32_t seq_start;   // first token of the sequence in the packed token axis (0 in fixed-length mode)
  int32_t seq_len;
  int32_t origin;      // first query row (query tiles) or first key (key tiles), relative to the sequence
  int32_t seq_id;      // sequence index; selects the batch stride in fixed-length mode
  int64_t carry_base;  // first carry slot of the sequence within a head's plane (0 when no carries are laid out)
};

// Slots of the scheduler's `counts` array.
enum : int { kCountQ = 0, kCountK = 1, kCountStatus = 2, kCountCovered = 3 };
// Values of counts[kCountStatus].
enum : int { kSchedOk = 0, kSchedBadCu = 1, kSchedCarryOverflow = 2, kSchedChainTimeout = 3, kSchedChainXcd = 4 };

struct SchedParams {
  const void* cu;          // NULL: fixed-length mode
  int32_t cu_is_int64, cu_has_leading_zero;
  int32_t num_seqs;
  int32_t fixed_len;       // L in fixed-length mode
  int64_t total_tokens;    // T: rows of the packed token axis (L in fixed-length mode)
  int64_t carry_capacity;  // carry slots reserved per head
  int32_t attend_current;
  int32_t want_key_tiles;  // backward: also build the key-tile list
  int32_t want_carry_base; // also lay out the per-sequence carry offsets
  Tile* q_tiles;           // query tiles (kBlockQ rows), heaviest first
  Tile* k_tiles;           // key tiles (key_tile keys), heaviest first
  int32_t* counts;         // [kCountQ] query tiles, [kCountK] key tiles, [kCountStatus], [kCountCovered] = tokens
                           // covered by sequences (rows at or beyond it belong to no sequence and are zero-filled)
  int64_t* carry_base;     // per sequence: first carry slot of the sequence (per head)
  int32_t* head_queue;     // backward: per-head cursor into the key-tile list, reset to 0 here
  int32_t num_heads;
  int32_t key_tile;        // keys per key tile (a multiple of 32; what the dK/dV kernel that will run sweeps)
  uint32_t* zero_fill;     // optional: 16-byte aligned region cleared by the launch (the one-kernel backward's flags
  int64_t zero_bytes;      // and tags start every call at zero), a multiple of 16 bytes
};

struct FwdParams {
  TensorRef q, k, v, o;
  VectorRef rem;
  float* row_stat;
  int64_t stat_sb, stat_sh;    // row_stat strides (token stride 1)
  float* carry;                // optional [head][slot]: running product per (row, key tile)
  const int64_t* carry_base;
  int64_t carry_head_stride;
  const Tile* tiles;
  const int32_t* counts;
  int32_t num_heads, head_dim;
  float scale_log2;            // logit_scale * log2(e)
  int32_t attend_current;
  int32_t vec_ok;              // all row strides / base pointers allow 16-byte accesses and head_dim % 8 == 0
  int32_t add_rem;             // write o + rem * v
  int32_t max_tiles;           // query-tile slots the launch provides per head (>= counts[kCountQ])
  int64_t total_tokens;        // packed mode: rows of the token axis; rows no sequence covers are zero-filled
};

struct BwdParams {
  TensorRef q, k, v, d_o, dq, dk, dv;
  VectorRef d_rem;
  const Tile* q_tiles;
  const Tile* k_tiles;
  const int32_t* counts;
  const int64_t* carry_base;
  const float* carry;          // [head][slot]: the forward's running product per (row, 32-key sub-tile)
  float* prefix;               // [head][slot]: prefix sum of g over the keys below the sub-tile, per (row, sub-tile)
  int64_t carry_head_stride;   // carry slots reserved per head
  int32_t num_heads, head_dim;
  float scale_log2;
  float logit_scale;
  int32_t attend_current;
  int32_t vec_ok;
  // Fused remainder term (the forward wrote o + rem * v): d_rem_eff = d_rem + d_o . v per row, dv += rem * d_o.
  int32_t add_rem;
  const float* row_stat;       // log2(rem), fp32 [batch][head][token]
  int64_t stat_sb, stat_sh;
  int32_t wgs_per_head;        // persistent dK/dV workgroups per head
  int32_t* head_queue;         // per head: next key tile not yet taken (beyond the first wgs_per_head), zero at launch
  int64_t drem_sb;             // batch stride of drem_eff: the heads of THIS launch (row_stat's stride counts the caller's)
  float* drem_eff;             // workspace, (B, heads, T) fp32: the gradient of rem per row in fp32 (d_rem, plus
                               // d_o . v when add_rem), written by the dQ kernel and read by the dK/dV kernel
  int32_t max_tiles;           // query-tile slots the dQ launch provides per head
  int64_t total_tokens;        // packed mode: rows of the token axis; rows no sequence covers are zero-filled
  // One-kernel backward (sba_bwd_chain.hip): what the key tiles of a (head, sequence) hand to each other.
  float* chain_dq;             // [head][row][128] fp32: partial dQ of a row over the key tiles below the reader
  uint32_t* chain_c;           // [head][row] {fp32 C below the reader's tile, tag = index of the reader's tile}
  int32_t* chain_flags;        // [head][key tile slot][8]: per consumer wave, row blocks whose partial dQ is complete
  int32_t* chain_head_xcc;     // [head]: XCC id + 1 of the head's workgroups (0 = none yet)
  int32_t* status;             // the scheduler's status word; the kernel raises it when a wait runs out
  int64_t chain_rows;          // rows per head in chain_dq / chain_c
  int64_t chain_sb;            // fixed-length mode: rows per batch element (0 in packed mode)
  int32_t chain_tile_cap;      // key-tile slots per head in chain_flags
};

// One sequence's token range from cu_seqlens (cumulative sequence ends, optionally preceded by a 0).  Returns false
// when the entry is unusable: ends must be non-decreasing, within [0, total_tokens], and a leading entry must be 0.
// The reference reads the same two entries without any check (sb_varlen_fwd.py:283-288); here a bad entry voids the
// whole schedule instead of sending tiles outside the tensors.  Shared by the device scheduler and its host mirror.
__host__ __device__ inline bool seq_span(const void* cu, int is_int64, int leading_zero, int s, int64_t total_tokens,
                                         int32_t* start, int32_t* len) {
  const int idx = s + (leading_zero ? 1 : 0);
  const int64_t end = is_int64 ? ((const int64_t*)cu)[idx] : (int64_t)((const int32_t*)cu)[idx];
  const int64_t beg = idx == 0 ? 0 : (is_int64 ? ((const int64_t*)cu)[idx - 1] : (int64_t)((const int32_t*)cu)[idx - 1]);
  const bool ok = beg >= 0 && beg <= end && end <= total_tokens && !(leading_zero && s == 0 && beg != 0);
  *start = ok ? (int32_t)beg : 0;
  *len = ok ? (int32_t)(end - beg) : 0;
  return ok;
}

// Carry slots.  Carries are kept per (row, 32-key sub-tile): sub-tile U covers keys 32U .. 32U+31 of the
// sequence and is needed by the rows of query tiles U/4, U/4 + 1, ..., M-1 (M = query tiles of 128 rows the
// sequence rounds up to).  Slot of (sub-tile U, row i), i >= 128*(U/4):
//   carry_offset(U, M) + (i - 128*(U/4))
__host__ __device__ inline int64_t carry_offset(int64_t U, int64_t M) {
  const int64_t q = U >> 2, r = U & 3;
  const int64_t tri = 2 * q * (q - 1) + r * q;            // sum_{U' < U} floor(U'/4)
  return U * (M * 128) - 128 * tri;
}
__host__ __device__ inline int64_t carry_slots(int64_t M) { return 256 * M * (M + 1); }   // carry_offset(4M, M)

}  // namespace sba
