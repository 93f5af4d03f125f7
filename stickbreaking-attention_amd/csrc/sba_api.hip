// C ABI of libsba: argument validation, workspace layout and kernel launches.  See include/sba.h.
#include <hip/hip_runtime.h>

#include <atomic>

#include "../../include/sba.h"
#include "sba_params.hpp"

namespace sba {
hipError_t launch_sched(const SchedParams& p, hipStream_t stream);
hipError_t launch_fwd(const FwdParams& p, int dtype_is_f16, int max_tiles, hipStream_t stream);
hipError_t launch_fwd_carry_only(const FwdParams& p, int dtype_is_f16, int max_tiles, hipStream_t stream);
hipError_t launch_bwd_dq(const BwdParams& p, int dtype_is_f16, int max_tiles, hipStream_t stream);
hipError_t launch_bwd_dkv(const BwdParams& p, int dtype_is_f16, int max_tiles, hipStream_t stream);
int dkv_key_tile(const BwdParams& p);
bool chain_supported(const BwdParams& p);
hipError_t launch_bwd_chain(const BwdParams& p, int dtype_is_f16, int max_tiles, hipStream_t stream);
hipError_t launch_fwd_f32(const FwdParams& p, int max_tiles, hipStream_t stream);
hipError_t launch_bwd_f32(const BwdParams& p, int batches, int64_t tokens, int max_q_tiles, hipStream_t stream);
}  // namespace sba

namespace {

constexpr double kLog2e = 1.4426950408889634;
constexpr int kBlockQ = 128, kBlockK = 64;

inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }
inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

struct Layout {
  int64_t max_q_tiles, max_k_tiles, carry_slots_per_head;
  size_t off_counts, off_q_tiles, off_k_tiles, off_carry_base, off_prefix, off_drem, off_queue, off_carry;
  size_t fwd_bytes, bwd_bytes, carry_bytes;
  size_t pass_bytes;                        // what ONE pass over these heads needs (bwd_bytes: what sba_bwd wants, see split_heads)
  // One-kernel backward: its buffers share the prefix plane's region (only one of the two backwards runs).
  int64_t chain_rows;                       // rows per head
  size_t off_chain_zero, chain_zero_bytes;  // {C, tag} per row, the flags and the heads' XCC ids: cleared by every launch
  size_t off_chain_c, off_chain_flags, off_chain_xcc, off_chain_dq;
  int32_t split_heads;                      // > 0: sba_bwd takes this many heads (a multiple of 8) through the one-kernel
                                            // backward and the rest through the two kernels
};

int plan(const SbaArgs* a, Layout* out) {
  if (a->num_heads <= 0 || a->num_seqs <= 0 || a->total_tokens <= 0) return SBA_ERR_SHAPE;
  if (a->head_dim < 1 || a->head_dim > 128) return SBA_ERR_HEAD_DIM;
  if (a->dtype != SBA_BF16 && a->dtype != SBA_F16 && a->dtype != SBA_F32) return SBA_ERR_DTYPE;
  if (a->total_tokens > (int64_t)1 << 30) return SBA_ERR_SHAPE;
  if ((a->recompute_carry != 0 && a->recompute_carry != 1) || a->carry_slots < 0) return SBA_ERR_SHAPE;
  if (a->backward_kernels < 0 || a->backward_kernels > 2) return SBA_ERR_SHAPE;
  if (a->recompute_carry && a->dtype == SBA_F32) return SBA_ERR_DTYPE;      // the fp32 path always keeps its products
  Layout L{};
  const int64_t T = a->total_tokens, B = a->num_seqs;
  const bool fixed = a->cu_seqlens == nullptr;
  int64_t max_len = (a->max_seqlen > 0 && a->max_seqlen < T) ? a->max_seqlen : T;
  if (fixed) {
    L.max_q_tiles = B * cdiv(T, kBlockQ);
    L.max_k_tiles = B * cdiv(T, kBlockK);
    L.carry_slots_per_head = B * sba::carry_slots(cdiv(T, kBlockQ));
  } else {
    L.max_q_tiles = cdiv(T, kBlockQ) + B;
    L.max_k_tiles = cdiv(T, kBlockK) + B;
    // sum_s 256 M_s (M_s + 1) with M_s <= L_s/128 + 1 and sum_s L_s^2 <= T * max_len
    L.carry_slots_per_head = cdiv(T * max_len, 64) + 6 * T + 512 * B;
  }
  // A caller that knows the lengths passes the exact count (sba_plan_host); the scheduler checks it on the device.
  // (Fixed-length mode knows its exact count above; a caller's figure is not needed there and is ignored.)
  if (a->carry_slots > 0 && !fixed) L.carry_slots_per_head = a->carry_slots;
  size_t off = 0;
  L.off_counts = off;      off = align_up(off + 256, 256);
  L.off_q_tiles = off;     off = align_up(off + (size_t)L.max_q_tiles * sizeof(sba::Tile), 256);
  L.off_carry_base = off;  off = align_up(off + (size_t)B * sizeof(int64_t), 256);
  L.fwd_bytes = off;
  L.off_k_tiles = off;     off = align_up(off + (size_t)L.max_k_tiles * sizeof(sba::Tile), 256);
  L.carry_bytes = align_up((size_t)L.carry_slots_per_head * a->num_heads * sizeof(float), 256);
  size_t chain_bytes = 0;
  L.chain_rows = fixed ? B * T : T;
  // The one-kernel backward is laid out when it is asked for, or (backward_kernels 0) where it is the faster one.
  // Measured on 256 compute units with the two backwards alternating in one process (uniform lengths and log-normal
  // mixes, 8 to 64 heads): it wins by 9-13 % when no sequence exceeds two key tiles (nothing is handed over then), and
  // by 2-6 % while the sequences give each of a head's workgroups between one and four key tiles of 128 (mean length
  // x heads >= 32768, longest x heads <= 131072) at up to 32 heads; it loses 2-10 % on sequences of 512-1024 tokens
  // (two more slots per tile than the dK/dV kernel) and 6-20 % beyond four tiles per workgroup (the partial dQ a
  // tile finds was written too long ago to still be in the L2).
  const bool chain_shape = a->dtype != SBA_F32 && a->head_dim == 128 && (a->num_heads & 7) == 0 && !a->add_remainder;
  const int64_t mean_len = fixed ? T : T / B;
  const bool chain_pays = max_len <= 256 ||
                          (a->num_heads <= 32 && mean_len * a->num_heads >= 32768 && max_len * a->num_heads <= (int64_t)512 * 256);
  if (chain_shape && (a->backward_kernels == 2 || (a->backward_kernels == 0 && chain_pays))) {
    size_t c = off;
    L.off_chain_zero = c;
    L.off_chain_c = c;      c = align_up(c + (size_t)a->num_heads * L.chain_rows * 8, 256);
    L.off_chain_flags = c;  c = align_up(c + (size_t)a->num_heads * L.max_k_tiles * 32, 256);
    L.off_chain_xcc = c;    c = align_up(c + (size_t)a->num_heads * 4, 256);
    L.chain_zero_bytes = c - L.off_chain_zero;
    L.off_chain_dq = c;     c += (size_t)a->num_heads * L.chain_rows * 128 * sizeof(float);
    chain_bytes = align_up(c - off, 256);
  }
  L.off_prefix = off;      off += L.carry_bytes > chain_bytes ? L.carry_bytes : chain_bytes;
  // d_rem + d_o . v per row (fp32), used when the remainder term is fused
  L.off_drem = off;        off = align_up(off + (size_t)a->num_heads * (size_t)T * (fixed ? (size_t)B : 1) * sizeof(float), 256);
  L.off_queue = off;       off = align_up(off + (size_t)a->num_heads * sizeof(int32_t), 256);      // per-head tile cursors
  // the forward's products, rebuilt inside the backward when the caller did not keep them
  L.off_carry = off;       if (a->recompute_carry) off += L.carry_bytes;
  L.bwd_bytes = L.pass_bytes = off;
  // A head count that is not a multiple of 8 (the reference's own benchmarks use 12) cannot run the one-kernel backward,
  // whose workgroups of a head must share an XCD.  Left to choose, sba_bwd then takes the largest multiple of 8 through
  // it and the remaining heads through the two kernels, one pass after the other on the stream -- where that pays: two
  // passes have two tails and two schedules, and on the reference's sweep (12 heads, 4 sequences) the split costs 12 %
  // at 4096 tokens and 2 % at 8192 and gains 4 % at 12288 and 16384.  The workspace must hold either pass.
  if (a->backward_kernels == 0 && (a->num_heads & 7) != 0 && a->num_heads > 8 &&
      mean_len * (a->num_heads & ~7) >= (int64_t)12288 * 8) {
    SbaArgs c = *a;
    c.num_heads = a->num_heads & ~7;
    Layout L8;
    if (plan(&c, &L8) == SBA_OK && L8.chain_zero_bytes > 0) {
      L.split_heads = c.num_heads;
      if (L8.bwd_bytes > L.bwd_bytes) L.bwd_bytes = L8.bwd_bytes;
    }
  }
  *out = L;
  return SBA_OK;
}

size_t elem_size(int dtype) { return dtype == SBA_F32 ? 4 : 2; }

// A tensor is usable with 16-byte buffer accesses when its base and its row/head/batch strides are 16-byte
// multiples and the rows of one sequence span less than 2 GiB (32-bit offsets from the sequence's first row).
bool vec16(const SbaTensor& t, size_t es, bool fixed, int64_t max_rows) {
  const int64_t per = 16 / (int64_t)es;
  if (max_rows * t.stride_token * (int64_t)es >= ((int64_t)1 << 31)) return false;
  if (((uintptr_t)t.ptr & 15) != 0) return false;
  if (t.stride_token % per || t.stride_head % per) return false;
  if (fixed && (t.stride_batch % per)) return false;
  return true;
}
int check_tensor(const SbaTensor& t, bool required, bool fixed) {
  if (!t.ptr) return required ? SBA_ERR_NULL : SBA_OK;
  if (t.stride_token < 0 || t.stride_head < 0 || (fixed && t.stride_batch < 0)) return SBA_ERR_STRIDE;
  return SBA_OK;
}
sba::TensorRef ref(const SbaTensor& t, bool fixed) { return sba::TensorRef{t.ptr, fixed ? t.stride_batch : 0, t.stride_head, t.stride_token}; }
sba::VectorRef vref(const SbaVector& t, bool fixed) { return sba::VectorRef{t.ptr, fixed ? t.stride_batch : 0, t.stride_head, t.stride_token}; }

int run_sched(const SbaArgs* a, char* ws, const Layout& L, bool want_key_tiles, bool want_carry_base, int key_tile, hipStream_t stream,
              bool clear_chain = false) {
  sba::SchedParams sp{};
  if (clear_chain) {
    sp.zero_fill = (uint32_t*)(ws + L.off_chain_zero);
    sp.zero_bytes = (int64_t)L.chain_zero_bytes;
  }
  sp.cu = a->cu_seqlens;
  sp.cu_is_int64 = a->cu_is_int64;
  sp.cu_has_leading_zero = a->cu_has_leading_zero;
  sp.num_seqs = a->num_seqs;
  sp.fixed_len = (int32_t)a->total_tokens;
  sp.total_tokens = a->total_tokens;
  sp.carry_capacity = L.carry_slots_per_head;
  sp.attend_current = a->attend_current ? 1 : 0;
  sp.want_key_tiles = want_key_tiles ? 1 : 0;
  sp.want_carry_base = want_carry_base ? 1 : 0;
  sp.q_tiles = (sba::Tile*)(ws + L.off_q_tiles);
  sp.k_tiles = (sba::Tile*)(ws + L.off_k_tiles);
  sp.counts = (int32_t*)(ws + L.off_counts);
  sp.carry_base = (int64_t*)(ws + L.off_carry_base);
  sp.head_queue = (int32_t*)(ws + L.off_queue);
  sp.num_heads = a->num_heads;
  sp.key_tile = key_tile;
  return sba::launch_sched(sp, stream) == hipSuccess ? SBA_OK : SBA_ERR_LAUNCH;
}

}  // namespace

extern "C" {

int sba_version(void) { return SBA_VERSION; }

const char* sba_strerror(int status) {
  switch (status) {
    case SBA_OK: return "ok";
    case SBA_ERR_NULL: return "a required pointer is NULL";
    case SBA_ERR_DTYPE: return "unsupported dtype";
    case SBA_ERR_HEAD_DIM: return "head_dim must be in 1..128";
    case SBA_ERR_STRIDE: return "negative or unsupported stride";
    case SBA_ERR_ALIGN: return "tensor base pointer is not aligned to its element size";
    case SBA_ERR_SHAPE: return "sizes must be positive (and total_tokens <= 2^30)";
    case SBA_ERR_WORKSPACE: return "workspace missing, misaligned or too small";
    case SBA_ERR_LAUNCH: return "kernel launch failed";
    case SBA_ERR_TOO_LARGE: return "the problem needs more scratch than the library's static array holds";
    default: return "unknown status";
  }
}

int sba_workspace_bytes(const SbaArgs* args, size_t* fwd_bytes, size_t* bwd_bytes, size_t* carry_bytes) {
  if (!args) return SBA_ERR_NULL;
  Layout L;
  const int st = plan(args, &L);
  if (st != SBA_OK) return st;
  if (fwd_bytes) *fwd_bytes = L.fwd_bytes;
  if (bwd_bytes) *bwd_bytes = L.bwd_bytes;
  if (carry_bytes) *carry_bytes = L.carry_bytes;
  return SBA_OK;
}

int sba_plan_host(const SbaArgs* a, const void* cu_host, SbaPlan* out) {
  if (!a || !out) return SBA_ERR_NULL;
  if (a->num_seqs <= 0 || a->total_tokens <= 0 || a->total_tokens > (int64_t)1 << 30) return SBA_ERR_SHAPE;
  SbaPlan pl{};
  const int ac = a->attend_current ? 1 : 0;
  for (int s = 0; s < a->num_seqs; s++) {
    int32_t start = 0, len = (int32_t)a->total_tokens;
    if (cu_host && !sba::seq_span(cu_host, a->cu_is_int64, a->cu_has_leading_zero, s, a->total_tokens, &start, &len))
      pl.status = SBA_SCHED_BAD_CU_SEQLENS;
    const int64_t n = len, m = cdiv(n, kBlockQ);
    pl.query_tiles += m;
    pl.key_tiles += cdiv(n, kBlockK);
    pl.carry_slots += sba::carry_slots(m);
    pl.pairs += n * (n - 1) / 2 + (ac ? n : 0);
    if (len > pl.longest) pl.longest = len;
    pl.covered_tokens = cu_host ? (int64_t)start + len : a->total_tokens;
  }
  if (pl.status != SBA_SCHED_OK) {      // the device scheduler voids the whole schedule
    pl.query_tiles = pl.key_tiles = pl.carry_slots = pl.pairs = pl.covered_tokens = 0;
    pl.longest = 0;
  }
  *out = pl;
  return SBA_OK;
}

}  // extern "C"

namespace {

// Scratch of sba_fwd_static: the forward's tile schedule (counts, query-tile list, per-sequence carry offsets) kept in
// a device array of the library instead of a caller workspace.  Every GPU the library runs on holds its own copy
// until the process ends.  Host code never uses the array's name as an address: the device address is looked up
// once per device with hipGetSymbolAddress and that pointer is what the kernels receive.
constexpr size_t kStaticScratchBytes = SBA_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

int static_scratch(char** out) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return SBA_ERR_LAUNCH;
  void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!ptr) {
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return SBA_ERR_LAUNCH;
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);
  }
  *out = (char*)ptr;
  return SBA_OK;
}

// The forward on a given workspace (the caller's, or the library's static scratch).
int fwd_on(const SbaArgs* a, char* ws, size_t ws_bytes, bool ws_is_static) {
  Layout L;
  int st = plan(a, &L);
  if (st != SBA_OK) return st;
  const bool fixed = a->cu_seqlens == nullptr;
  const size_t es = elem_size(a->dtype);
  if ((st = check_tensor(a->q, true, fixed)) || (st = check_tensor(a->k, true, fixed)) ||
      (st = check_tensor(a->v, true, fixed)) || (st = check_tensor(a->o, true, fixed)))
    return st;
  if (!a->rem.ptr || !a->row_stat) return SBA_ERR_NULL;
  for (const SbaTensor* t : {&a->q, &a->k, &a->v, &a->o})
    if (t->ptr && ((uintptr_t)t->ptr % es)) return SBA_ERR_ALIGN;
  if (ws_is_static && ws_bytes < L.fwd_bytes) return SBA_ERR_TOO_LARGE;
  if (!ws || ((uintptr_t)ws & 255) || ws_bytes < L.fwd_bytes) return SBA_ERR_WORKSPACE;
  hipStream_t stream = (hipStream_t)a->stream;
  // The carry offsets are laid out (and the capacity checked) when products are recorded, and also when the backward
  // will rebuild them: both passes then agree on whether the schedule stands.
  if ((st = run_sched(a, ws, L, false, a->carry != nullptr || a->recompute_carry, kBlockK, stream)) != SBA_OK) return st;

  sba::FwdParams p{};
  p.q = ref(a->q, fixed); p.k = ref(a->k, fixed); p.v = ref(a->v, fixed); p.o = ref(a->o, fixed);
  p.rem = vref(a->rem, fixed);
  p.row_stat = a->row_stat;
  p.carry = a->carry;
  p.carry_base = (const int64_t*)(ws + L.off_carry_base);
  p.carry_head_stride = L.carry_slots_per_head;
  p.stat_sb = fixed ? (int64_t)a->num_heads * a->total_tokens : 0;
  p.stat_sh = a->total_tokens;
  p.tiles = (const sba::Tile*)(ws + L.off_q_tiles);
  p.counts = (const int32_t*)(ws + L.off_counts);
  p.num_heads = a->num_heads;
  p.head_dim = a->head_dim;
  p.scale_log2 = (float)((double)a->logit_scale * kLog2e);
  p.attend_current = a->attend_current ? 1 : 0;
  p.add_rem = a->add_remainder ? 1 : 0;
  p.max_tiles = (int32_t)L.max_q_tiles;
  p.total_tokens = a->total_tokens;
  const int64_t max_rows = (a->max_seqlen > 0 && a->max_seqlen < a->total_tokens) ? a->max_seqlen : a->total_tokens;
  bool v16 = (a->head_dim % (16 / (int)es)) == 0;
  for (const SbaTensor* t : {&a->q, &a->k, &a->v, &a->o}) v16 = v16 && vec16(*t, es, fixed, max_rows);
  p.vec_ok = v16 ? 1 : 0;
  hipEvent_t* ev = (hipEvent_t*)a->trace_events;
  if (ev && hipEventRecord(ev[0], stream) != hipSuccess) return SBA_ERR_LAUNCH;
  hipError_t e = (a->dtype == SBA_F32) ? sba::launch_fwd_f32(p, (int)L.max_q_tiles, stream)
                                       : sba::launch_fwd(p, a->dtype == SBA_F16, (int)L.max_q_tiles, stream);
  if (e != hipSuccess) return SBA_ERR_LAUNCH;
  if (ev && hipEventRecord(ev[1], stream) != hipSuccess) return SBA_ERR_LAUNCH;
  return SBA_OK;
}

}  // namespace

extern "C" {

int sba_fwd(const SbaArgs* a) {
  if (!a) return SBA_ERR_NULL;
  return fwd_on(a, (char*)a->workspace, a->workspace_bytes, false);
}

int sba_fwd_static(const SbaArgs* a) {
  if (!a) return SBA_ERR_NULL;
  char* ws = nullptr;
  const int st = static_scratch(&ws);
  if (st != SBA_OK) return st;
  return fwd_on(a, ws, kStaticScratchBytes, true);
}

}  // extern "C"

namespace {

// Whether every tensor of the backward allows 16-byte accesses.
bool bwd_vec_ok(const SbaArgs* a) {
  const bool fixed = a->cu_seqlens == nullptr;
  const size_t es = elem_size(a->dtype);
  const int64_t max_rows = (a->max_seqlen > 0 && a->max_seqlen < a->total_tokens) ? a->max_seqlen : a->total_tokens;
  bool v16 = (a->head_dim % (16 / (int)es)) == 0;
  for (const SbaTensor* t : {&a->q, &a->k, &a->v, &a->d_o, &a->dq, &a->dk, &a->dv})
    if (t->ptr) v16 = v16 && vec16(*t, es, fixed, max_rows);
  return v16;
}
// Whether one pass over the heads `a` describes runs the one-kernel backward (its buffers are laid out and the
// tensors and the device allow it).
bool bwd_is_chained(const SbaArgs* a, const Layout& L) {
  sba::BwdParams p{};
  p.vec_ok = bwd_vec_ok(a) ? 1 : 0;
  p.head_dim = a->head_dim;
  p.num_heads = a->num_heads;
  p.add_rem = a->add_remainder ? 1 : 0;
  return a->dtype != SBA_F32 && L.chain_zero_bytes > 0 && sba::chain_supported(p);
}

// One pass of the backward over the heads `a` describes (all of them, or one group of a larger call: `stat_heads` is
// the head count of the caller's row_stat array, `first`/`last` say which trace events this pass records).
int bwd_pass(const SbaArgs* a, int64_t stat_heads, bool first, bool last) {
  Layout L;
  int st = plan(a, &L);
  if (st != SBA_OK) return st;
  const bool fixed = a->cu_seqlens == nullptr;
  const size_t es = elem_size(a->dtype);
  if ((st = check_tensor(a->q, true, fixed)) || (st = check_tensor(a->k, true, fixed)) ||
      (st = check_tensor(a->v, true, fixed)) || (st = check_tensor(a->d_o, true, fixed)) ||
      (st = check_tensor(a->dq, true, fixed)) || (st = check_tensor(a->dk, true, fixed)) ||
      (st = check_tensor(a->dv, true, fixed)))
    return st;
  if (!a->carry && !a->recompute_carry) return SBA_ERR_NULL;
  if (a->add_remainder && !a->row_stat) return SBA_ERR_NULL;
  for (const SbaTensor* t : {&a->q, &a->k, &a->v, &a->d_o, &a->dq, &a->dk, &a->dv})
    if (t->ptr && ((uintptr_t)t->ptr % es)) return SBA_ERR_ALIGN;
  if (!a->workspace || ((uintptr_t)a->workspace & 255) || a->workspace_bytes < L.pass_bytes) return SBA_ERR_WORKSPACE;
  hipStream_t stream = (hipStream_t)a->stream;

  char* ws = (char*)a->workspace;
  sba::BwdParams p{};
  p.q = ref(a->q, fixed); p.k = ref(a->k, fixed); p.v = ref(a->v, fixed);
  p.d_o = ref(a->d_o, fixed);
  p.dq = ref(a->dq, fixed); p.dk = ref(a->dk, fixed); p.dv = ref(a->dv, fixed);
  p.d_rem = vref(a->d_rem, fixed);
  p.q_tiles = (const sba::Tile*)(ws + L.off_q_tiles);
  p.k_tiles = (const sba::Tile*)(ws + L.off_k_tiles);
  p.counts = (const int32_t*)(ws + L.off_counts);
  p.carry_base = (const int64_t*)(ws + L.off_carry_base);
  p.carry = a->recompute_carry ? (const float*)(ws + L.off_carry) : a->carry;
  p.prefix = (float*)(ws + L.off_prefix);
  p.carry_head_stride = L.carry_slots_per_head;
  p.num_heads = a->num_heads;
  p.head_dim = a->head_dim;
  p.scale_log2 = (float)((double)a->logit_scale * kLog2e);
  p.logit_scale = a->logit_scale;
  p.attend_current = a->attend_current ? 1 : 0;
  p.add_rem = a->add_remainder ? 1 : 0;
  p.row_stat = a->row_stat;
  p.stat_sb = fixed ? stat_heads * a->total_tokens : 0;
  p.stat_sh = a->total_tokens;
  p.drem_sb = fixed ? (int64_t)a->num_heads * a->total_tokens : 0;
  p.drem_eff = (float*)(ws + L.off_drem);
  p.head_queue = (int32_t*)(ws + L.off_queue);
  p.max_tiles = (int32_t)L.max_q_tiles;
  p.total_tokens = a->total_tokens;
  p.vec_ok = bwd_vec_ok(a) ? 1 : 0;
  // One kernel (the key tiles of a sequence hand C and partial dQ to each other) where it applies, else dQ then dK/dV.
  const bool chain = bwd_is_chained(a, L);
  if (chain) {
    p.chain_c = (uint32_t*)(ws + L.off_chain_c);
    p.chain_flags = (int32_t*)(ws + L.off_chain_flags);
    p.chain_head_xcc = (int32_t*)(ws + L.off_chain_xcc);
    p.chain_dq = (float*)(ws + L.off_chain_dq);
    p.status = (int32_t*)(ws + L.off_counts) + sba::kCountStatus;
    p.chain_rows = L.chain_rows;
    p.chain_sb = fixed ? a->total_tokens : 0;
    p.chain_tile_cap = (int32_t)L.max_k_tiles;
  }
  // The key-tile list is built for the dK/dV kernel that will run (the fp32 kernels do not use it).
  const int key_tile = a->dtype == SBA_F32 ? kBlockK : sba::dkv_key_tile(p);
  if ((st = run_sched(a, ws, L, true, true, key_tile, stream, chain)) != SBA_OK) return st;
  hipEvent_t* ev = (hipEvent_t*)a->trace_events;
  if (ev && first && hipEventRecord(ev[0], stream) != hipSuccess) return SBA_ERR_LAUNCH;
  if (a->dtype == SBA_F32) {
    if (sba::launch_bwd_f32(p, fixed ? a->num_seqs : 1, a->total_tokens, (int)L.max_q_tiles, stream) != hipSuccess) return SBA_ERR_LAUNCH;
    if (ev && last && (hipEventRecord(ev[1], stream) != hipSuccess || hipEventRecord(ev[2], stream) != hipSuccess)) return SBA_ERR_LAUNCH;
    return SBA_OK;
  }
  if (a->recompute_carry) {
    // O(L) state between the passes: the products the forward would have recorded are rebuilt from q and k by the
    // forward kernel stripped of everything else (timed with the dQ kernel by trace_events).
    sba::FwdParams f{};
    f.q = p.q; f.k = p.k; f.v = p.v; f.o = p.q;
    f.carry = (float*)(ws + L.off_carry);
    f.carry_base = p.carry_base;
    f.carry_head_stride = L.carry_slots_per_head;
    f.tiles = p.q_tiles;
    f.counts = p.counts;
    f.num_heads = a->num_heads;
    f.head_dim = a->head_dim;
    f.scale_log2 = p.scale_log2;
    f.attend_current = p.attend_current;
    f.max_tiles = (int32_t)L.max_q_tiles;
    f.total_tokens = a->total_tokens;
    const int64_t max_rows = (a->max_seqlen > 0 && a->max_seqlen < a->total_tokens) ? a->max_seqlen : a->total_tokens;
    bool fv16 = (a->head_dim % (16 / (int)es)) == 0;
    for (const SbaTensor* t : {&a->q, &a->k}) fv16 = fv16 && vec16(*t, es, fixed, max_rows);
    f.vec_ok = fv16 ? 1 : 0;
    if (sba::launch_fwd_carry_only(f, a->dtype == SBA_F16, (int)L.max_q_tiles, stream) != hipSuccess) return SBA_ERR_LAUNCH;
  }
  if (chain) {
    if (ev && last && hipEventRecord(ev[1], stream) != hipSuccess) return SBA_ERR_LAUNCH;
    if (sba::launch_bwd_chain(p, a->dtype == SBA_F16, (int)L.max_k_tiles, stream) != hipSuccess) return SBA_ERR_LAUNCH;
    if (ev && last && hipEventRecord(ev[2], stream) != hipSuccess) return SBA_ERR_LAUNCH;
    return SBA_OK;
  }
  if (sba::launch_bwd_dq(p, a->dtype == SBA_F16, (int)L.max_q_tiles, stream) != hipSuccess) return SBA_ERR_LAUNCH;
  if (ev && last && hipEventRecord(ev[1], stream) != hipSuccess) return SBA_ERR_LAUNCH;
  if (sba::launch_bwd_dkv(p, a->dtype == SBA_F16, (int)L.max_k_tiles, stream) != hipSuccess) return SBA_ERR_LAUNCH;
  if (ev && last && hipEventRecord(ev[2], stream) != hipSuccess) return SBA_ERR_LAUNCH;
  return SBA_OK;
}


}  // namespace

extern "C" {

int sba_bwd_kernels(const SbaArgs* a) {
  if (!a) return SBA_ERR_NULL;
  Layout L;
  const int st = plan(a, &L);
  if (st != SBA_OK) return st;
  return bwd_is_chained(a, L) ? 1 : 2;
}

int sba_bwd(const SbaArgs* a) {
  if (!a) return SBA_ERR_NULL;
  Layout L;
  int st = plan(a, &L);
  if (st != SBA_OK) return st;
  const size_t es = elem_size(a->dtype);
  // the heads of a call from h0 on, as a call of their own
  auto heads_from = [&](int64_t h0, int64_t count) {
    SbaArgs c = *a;
    c.num_heads = (int32_t)count;
    for (SbaTensor* t : {&c.q, &c.k, &c.v, &c.d_o, &c.dq, &c.dk, &c.dv})
      if (t->ptr) t->ptr = (char*)t->ptr + h0 * t->stride_head * (int64_t)es;
    if (c.d_rem.ptr) c.d_rem.ptr = (char*)c.d_rem.ptr + h0 * c.d_rem.stride_head * (int64_t)es;
    if (c.carry) c.carry += h0 * L.carry_slots_per_head;          // slots per head do not depend on the head count
    if (c.row_stat) c.row_stat += h0 * a->total_tokens;
    return c;
  };
  if (L.split_heads > 0 && a->workspace_bytes >= L.bwd_bytes) {
    SbaArgs c = heads_from(0, L.split_heads);
    Layout L8;
    if (plan(&c, &L8) == SBA_OK && bwd_is_chained(&c, L8)) {      // (the tensors and the device allow the one kernel)
      if ((st = bwd_pass(&c, a->num_heads, true, false)) != SBA_OK) return st;
      c = heads_from(L.split_heads, a->num_heads - L.split_heads);
      c.backward_kernels = 1;
      return bwd_pass(&c, a->num_heads, false, true);
    }
  }
  if (a->workspace_bytes >= L.pass_bytes || a->num_heads == 1) return bwd_pass(a, a->num_heads, true, true);
  // A workspace smaller than the whole call needs: the heads are independent, so they go through in groups of as many
  // as fit (the per-head planes dominate the workspace), one group after the other on the stream.
  SbaArgs c = *a;
  int64_t lo = 0, hi = a->num_heads;           // largest head count whose layout fits: plan() grows with num_heads
  while (lo < hi) {
    c.num_heads = (int32_t)((lo + hi + 1) / 2);
    if (plan(&c, &L) == SBA_OK && L.pass_bytes <= a->workspace_bytes) lo = c.num_heads; else hi = c.num_heads - 1;
  }
  if (lo < 1) return SBA_ERR_WORKSPACE;
  const int64_t passes = cdiv(a->num_heads, lo), group = cdiv(a->num_heads, passes);
  // The one-kernel backward's layout is the larger one and is only laid out for head counts it applies to, so a group
  // size below `lo` need not fit although `lo` does: every pass then takes the two-kernel backward, whose layout grows
  // with the head count and therefore fits.
  int32_t kernels = a->backward_kernels;
  for (int64_t heads : {group, a->num_heads % group}) {
    c.num_heads = (int32_t)heads;
    if (heads > 0 && (plan(&c, &L) != SBA_OK || L.pass_bytes > a->workspace_bytes)) kernels = 1;
  }
  for (int64_t h0 = 0; h0 < a->num_heads; h0 += group) {
    c = heads_from(h0, a->num_heads - h0 < group ? a->num_heads - h0 : group);
    c.backward_kernels = kernels;
    if ((st = bwd_pass(&c, a->num_heads, h0 == 0, h0 + group >= a->num_heads)) != SBA_OK) return st;
  }
  return SBA_OK;
}

}  // extern "C"
