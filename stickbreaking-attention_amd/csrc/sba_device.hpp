// Device-side building blocks shared by the gfx950 stick-breaking attention kernels.
//
// Register-level conventions used everywhere in this library
// ----------------------------------------------------------
// Scores are produced TRANSPOSED, S^T = K Q^T, with v_mfma_f32_32x32x16_{bf16,f16}: the 32 MFMA rows
// are keys, the 32 MFMA columns are queries.  In the 32x32 accumulator lane l holds column l%32 and
// the 16 rows 8*(r/4) + 4*(l/32) + r%4 (r = register index).  The key <-> MFMA-row assignment is free
// (it only decides which LDS row a lane fetches for the A operand), and it is chosen so that for a
// key tile of 64 keys (two MFMA row tiles mt = 0, 1) lane l owns query l%32 and the 32 CONSECUTIVE
// keys 32*(l/32) + 16*mt + r.  The stick-breaking products along the key axis are then serial
// in-register scans with a single exchange between the two half-waves per tile, and the registers
// feed the next MFMA (P.V, dZ.K) directly as its A operand (k index = 8*(l/32) + t  <->  key
// 32*(l/32) + 8*c + t for k-step c).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "sba_params.hpp"

namespace sba {

typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) short s16x4;

constexpr int kBlockQ = 128;   // query rows per workgroup tile (4 waves x 32)
constexpr int kBlockK = 64;    // keys per tile
constexpr int kWaves = 4;
constexpr int kThreads = kWaves * 64;

// Element-type traits: 16-bit storage types with an MFMA 32x32x16 variant.
template <typename T> struct Elem;
template <> struct Elem<__bf16> {
  typedef bf16x8 vec8;
  static __device__ __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct Elem<_Float16> {
  typedef f16x8 vec8;
  static __device__ __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

// Two fp32 -> packed 16-bit (round to nearest even), low half = a.
template <typename T> __device__ __forceinline__ uint32_t pack2(float a, float b);
template <> __device__ __forceinline__ uint32_t pack2<__bf16>(float a, float b) {
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
  bf16x2 v = {(__bf16)a, (__bf16)b};
  return __builtin_bit_cast(uint32_t, v);
}
template <> __device__ __forceinline__ uint32_t pack2<_Float16>(float a, float b) {
  typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
  f16x2 v = {(_Float16)a, (_Float16)b};
  return __builtin_bit_cast(uint32_t, v);
}
template <typename T> __device__ __forceinline__ float to_f32(T x) { return (float)x; }

template <typename T> __device__ __forceinline__ typename Elem<T>::vec8 as_vec8(u32x4 x) {
  return __builtin_bit_cast(typename Elem<T>::vec8, x);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }   // v_exp_f32
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }    // v_log_f32
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }     // v_rcp_f32
__device__ __forceinline__ float fast_min(float a, float b) {
  float r;
  asm("v_min_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}

// Value held by the other half-wave (lane ^ 32).
__device__ __forceinline__ float other_half(float x, int half) {
  uint32_t u = __builtin_bit_cast(uint32_t, x);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  // r[0]: low lanes keep their own value, high lanes receive lane-32's; r[1]: low lanes receive lane+32's.
  uint32_t o = half ? r[0] : r[1];
  return __builtin_bit_cast(float, o);
}

// LDS row-major tiles of 16-bit elements.  Row strides of 304 bytes (128 + 24 elements) and 144 bytes
// (64 + 8 elements) were measured conflict-free for both access patterns used here: 16-byte reads along 16
// consecutive rows (MFMA operands contracted over the row) and the 8-byte transpose reads that gather an
// operand down 4 consecutive rows.  (272 bytes halves the transpose-read rate; 288 and 320 hurt the row reads.)
template <int W> constexpr int lds_stride() { return W == 128 ? 152 : W + 8; }

// 8 consecutive elements of one row (A operand for contractions over head_dim, or over a row's own axis).
template <typename T>
__device__ __forceinline__ typename Elem<T>::vec8 lds_row8(const T* tile, int row_stride, int row, int col) {
  return *reinterpret_cast<const typename Elem<T>::vec8*>(tile + row * row_stride + col);
}

// B operand gathered DOWN the rows of a row-major tile with the gfx950 LDS transpose read:
// returns, for this lane's column `col0 + l%32`, the 8 elements of rows row0 .. row0+7.
// Within each 16-lane group, lane s fetches the 8-byte chunk (row row0 + 4*t + s/4, columns
// cbase + 4*(s%4) .. +3) and receives rows row0+4*t .. +3 of column cbase + s.
template <typename T>
__device__ __forceinline__ typename Elem<T>::vec8 lds_col8(const T* tile, int row_stride, int row0, int col0, int lane) {
  const int s = lane & 15;
  const int cbase = col0 + ((lane >> 4) & 1) * 16;
  const T* p0 = tile + (row0 + (s >> 2)) * row_stride + cbase + 4 * (s & 3);
  const T* p1 = p0 + 4 * row_stride;
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p0));
  s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p1));
  typedef __attribute__((ext_vector_type(8))) short s16x8;
  s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(typename Elem<T>::vec8, v);
}

// MFMA row m (A-operand lane index l%32) of row tile mt -> key offset inside the 64-key tile such that
// accumulator register r of half-wave h holds key 32*h + 16*mt + r.  (m = 8a + 4h + b, r = 4a + b.)
__device__ __forceinline__ int mfma_row_to_key(int mt, int m) {
  return ((m >> 2) & 1) * 32 + mt * 16 + (m >> 3) * 4 + (m & 3);
}
// Same for a 32-key sub-tile handled as ONE row tile: register r of half-wave h holds key 16*h + r.
__device__ __forceinline__ int mfma_row_to_key32(int m) { return ((m >> 2) & 1) * 16 + (m >> 3) * 4 + (m & 3); }

// The rows of one (head, sequence) of a [.., token, head_dim] tensor, as the tile copies see them.  The fast path
// addresses them through a raw buffer resource: scalar base, out-of-range rows read as zero for free, and one
// loop-invariant 32-bit lane offset instead of 64-bit pointer arithmetic per chunk.
template <typename T>
struct RowSource {
  const T* base;
  int64_t stride;                 // elements between token rows
  int rows, d;                    // valid rows, valid head_dim
  __amdgpu_buffer_rsrc_t rsrc;    // base .. last valid element (fast path only)
  int stride_bytes;
};
template <typename T, bool kFast>
__device__ __forceinline__ RowSource<T> make_row_source(const T* base, int64_t stride, int rows, int d) {
  RowSource<T> r;
  r.base = base; r.stride = stride; r.rows = rows; r.d = d;
  r.stride_bytes = (int)(stride * (int64_t)sizeof(T));
  if (kFast) {
    const int bytes = rows > 0 ? (rows - 1) * r.stride_bytes + d * (int)sizeof(T) : 0;
    r.rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, bytes, 0x00020000);
  }
  return r;
}

// Cooperative global -> register -> LDS copy of a [kRows x DH] tile of 16-bit elements, 16 bytes per access.
// Rows beyond the source and columns at or beyond head_dim are zero-filled.  kFast: head_dim == DH, every row
// start 16-byte aligned and the sequence's rows span < 2 GiB, so the copy is straight-line buffer loads.
template <typename T, int DH, int kRows, bool kFast, int kNumThreads = kThreads>
struct TileCopy {
  static constexpr int kChunksPerRow = DH / 8;
  static constexpr int kRowsPerPass = kNumThreads / kChunksPerRow;
  static constexpr int kPerThread = kRows / kRowsPerPass;
  static_assert(kRows % kRowsPerPass == 0, "tile must divide evenly over the workgroup");
  u32x4 regs[kPerThread];

  __device__ __forceinline__ void load(const RowSource<T>& src, int row0) {
    const int tr = (threadIdx.x % kNumThreads) / kChunksPerRow, col = ((threadIdx.x % kNumThreads) % kChunksPerRow) * 8;
    if (kFast) {
      const int voff = tr * src.stride_bytes + col * (int)sizeof(T);
#pragma unroll
      for (int i = 0; i < kPerThread; i++)
        regs[i] = __builtin_amdgcn_raw_buffer_load_b128(src.rsrc, voff, (row0 + i * kRowsPerPass) * src.stride_bytes, 0);
    } else {
#pragma unroll
      for (int i = 0; i < kPerThread; i++) {
        const int row = row0 + tr + i * kRowsPerPass;
        u32x4 v = {0, 0, 0, 0};
        if (row < src.rows) {
          const uint16_t* p = reinterpret_cast<const uint16_t*>(src.base + row * src.stride + col);
          uint16_t e[8];
#pragma unroll
          for (int t = 0; t < 8; t++) e[t] = (col + t < src.d) ? p[t] : (uint16_t)0;
          v[0] = e[0] | ((uint32_t)e[1] << 16); v[1] = e[2] | ((uint32_t)e[3] << 16);
          v[2] = e[4] | ((uint32_t)e[5] << 16); v[3] = e[6] | ((uint32_t)e[7] << 16);
        }
        regs[i] = v;
      }
    }
  }
  __device__ __forceinline__ void store(T* tile) const {
    const int tr = (threadIdx.x % kNumThreads) / kChunksPerRow, col = ((threadIdx.x % kNumThreads) % kChunksPerRow) * 8;
#pragma unroll
    for (int i = 0; i < kPerThread; i++)
      *reinterpret_cast<u32x4*>(tile + (tr + i * kRowsPerPass) * lds_stride<DH>() + col) = regs[i];
  }
};

// Load 8 consecutive head_dim elements of one token row from global memory (zero beyond head_dim / when !valid).
template <typename T, bool kFast>
__device__ __forceinline__ u32x4 load_row8(const T* row, int d0, int d_valid, bool valid) {
  u32x4 v = {0, 0, 0, 0};
  if (valid) {
    if (kFast) {
      v = *reinterpret_cast<const u32x4*>(row + d0);
    } else {
      uint16_t e[8];
#pragma unroll
      for (int t = 0; t < 8; t++) e[t] = (d0 + t < d_valid) ? reinterpret_cast<const uint16_t*>(row + d0)[t] : (uint16_t)0;
      v[0] = e[0] | ((uint32_t)e[1] << 16); v[1] = e[2] | ((uint32_t)e[3] << 16);
      v[2] = e[4] | ((uint32_t)e[5] << 16); v[3] = e[6] | ((uint32_t)e[7] << 16);
    }
  }
  return v;
}


// Element-wise backward math of one 64-key tile for the 32 keys this lane owns (see the conventions above).
//   s, dp     : S^T = K Q^T and dP^T = V dO^T accumulators (row tile mt, register r  <->  key 32*half + 16*mt + r)
//   lim       : key R of this lane is visible iff R < lim (only consulted when `diagonal`)
//   NT        : MFMA row tiles per key tile: 2 for a 64-key tile (keys 32*half + 16*mt + r), 1 for a 32-key
//               sub-tile (keys 16*half + r)
//   prod_in   : prod over the keys ABOVE this tile (between the tile and the row) of (1 - sigma); recorded by
//               the forward, which sweeps in that direction
//   prefix_in : sum over the keys BELOW this tile of g, with g_ij = A_ij (dO_i.v_j - drem_i)
// Produces P (pk) and dZ = g - sigma * C (dzk), C_ij = sum_{j' <= j} g_ij', packed to 16 bit two keys per
// word, and the prefix sum for the next tile up.  (The reference evaluates the same quantities tile by tile at
// stickbreaking_attention/sb_varlen/sb_varlen_bwd.py:438-447.)
template <typename T, int NT, bool kDiagonal, bool kNeedP = true>
__device__ __forceinline__ void bwd_tile_math_impl(const f32x16 (&s)[NT], const f32x16 (&dp)[NT], float scale_log2, int lim,
                                                   int half, float drem, float prod_in, float prefix_in,
                                                   uint32_t (&pk)[8 * NT], uint32_t (&dzk)[8 * NT], float& prod_lower,
                                                   float& prefix_upper, float& prefix_out) {
  constexpr int N = 16 * NT;      // keys per lane
  // sigma = 1 - 1/(1+e) needs no clamp on e: e = inf gives 1/(1+e) = 0 and sigma = 1 exactly, and the absolute
  // error of the subtraction (6e-8) is far below the 16-bit rounding of P and dZ.
  float beta[N], pe[N];
  float run = 1.f;
#pragma unroll
  for (int R = N - 1; R >= 0; --R) {
    float x = s[R >> 4][R & 15] * scale_log2;
    if (kDiagonal) x = (R < lim) ? x : -INFINITY;
    const float omb = fast_rcp(1.f + fast_exp2(x));
    beta[R] = 1.f - omb;
    pe[R] = run;           // product over this lane's higher keys
    run *= omb;
  }
  const float oth = other_half(run, half);
  prod_lower = prod_in * (half ? run : oth);               // product above the lower half-wave's keys
  const float seed = half ? prod_in : prod_lower;           // the upper half-wave holds the higher keys
  // Running C as if this lane's keys were preceded only by the keys below the tile; the upper half-wave's
  // share of the lower half-wave's total is added afterwards (fixup).
  float acc = prefix_in;
  float dz[N];
  const float neg_drem_seed = -drem * seed;
#pragma unroll
  for (int R = 0; R < N; R++) {
    float g;
    if (kNeedP) {
      const float a = beta[R] * (pe[R] * seed);
      g = a * (dp[R >> 4][R & 15] - drem);
      pe[R] = a;
    } else {
      // A is not wanted for itself: the seed goes into (dP - drem) with one fma instead of a multiply of its own
      g = (beta[R] * pe[R]) * fmaf(dp[R >> 4][R & 15], seed, neg_drem_seed);
    }
    acc += g;
    dz[R] = g - beta[R] * acc;
  }
  const float tot = acc - prefix_in;
  const float oth_g = other_half(tot, half);
  const float fixup = half ? oth_g : 0.f;                   // the lower half-wave holds the lower keys
  prefix_upper = prefix_in + (half ? oth_g : tot);          // C just below the upper half-wave's keys
  prefix_out = acc + oth_g;
#pragma unroll
  for (int R = 0; R < N; R += 2) {
    pk[R >> 1] = kNeedP ? pack2<T>(pe[R], pe[R + 1]) : 0u;
    dzk[R >> 1] = pack2<T>(dz[R] - beta[R] * fixup, dz[R + 1] - beta[R + 1] * fixup);
  }
}

// prod_lower / prefix_upper: the same two carries at the boundary between the two half-waves' keys (the middle of
// the tile), for consumers that work on half the keys at a time.
template <typename T, int NT, bool kNeedP = true>
__device__ __forceinline__ void bwd_tile_math(const f32x16 (&s)[NT], const f32x16 (&dp)[NT], float scale_log2, bool diagonal,
                                              int lim, int half, float drem, float prod_in, float prefix_in,
                                              uint32_t (&pk)[8 * NT], uint32_t (&dzk)[8 * NT], float& prod_lower,
                                              float& prefix_upper, float& prefix_out) {
  if (diagonal)
    bwd_tile_math_impl<T, NT, true, kNeedP>(s, dp, scale_log2, lim, half, drem, prod_in, prefix_in, pk, dzk, prod_lower,
                                    prefix_upper, prefix_out);
  else
    bwd_tile_math_impl<T, NT, false, kNeedP>(s, dp, scale_log2, lim, half, drem, prod_in, prefix_in, pk, dzk, prod_lower,
                                     prefix_upper, prefix_out);
}

// Epilogue stores of the fast path.  An MFMA accumulator tile holds, per lane, one column and 16 rows
// (8*(r/4) + 4*half + r%4); writing it element by element through 64-bit pointers with a bounds test per row costs
// ~15 instructions per 2-byte store.  Here the rows of one (head, sequence) are addressed through a raw buffer
// resource instead: a per-lane byte offset (half-wave row offset + column), a scalar byte offset per register (row
// * stride), and rows beyond the sequence are dropped by the buffer's range check.  Requires the same conditions as
// the buffer loads (32-bit offsets within one sequence's rows, head_dim == DH).
template <typename T>
struct RowSink {
  __amdgpu_buffer_rsrc_t rsrc;
  int stride_bytes;
};
template <typename T>
__device__ __forceinline__ RowSink<T> make_row_sink(T* base, int64_t stride, int rows, int d) {
  RowSink<T> r;
  r.stride_bytes = (int)(stride * (int64_t)sizeof(T));
  const int bytes = rows > 0 ? (rows - 1) * r.stride_bytes + d * (int)sizeof(T) : 0;
  r.rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, bytes, 0x00020000);
  return r;
}
// acc[r] -> row (row0 + 8*(r/4) + 4*half + r%4), column col0 + (lane % 32), scaled; row0 and col0 wave-uniform.
template <typename T>
__device__ __forceinline__ void store_acc_tile(const RowSink<T>& sink, const f32x16& acc, float scale, int row0, int col0,
                                               int half, int col) {
  const int voff = 4 * half * sink.stride_bytes + col * (int)sizeof(T);
  const int sbase = __builtin_amdgcn_readfirstlane(row0 * sink.stride_bytes + col0 * (int)sizeof(T));
#pragma unroll
  for (int r = 0; r < 16; r++) {
    const T v = (T)(acc[r] * scale);
    __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(short, v), sink.rsrc, voff,
                                          sbase + (8 * (r >> 2) + (r & 3)) * sink.stride_bytes, 0);
  }
}

// The same tile through a wave-private LDS scratch of 32 x lds_stride<32>() elements, so that it leaves as two
// 16-byte stores per lane instead of sixteen 2-byte ones: each lane writes its column's 4-key groups transposed
// ([column][row] layout, 8 bytes per write), and the transpose read hands every lane 8 consecutive columns of one row.
template <typename T>
__device__ __forceinline__ void store_acc_tile_wide(const RowSink<T>& sink, const f32x16& acc, float scale, int row0, int col0,
                                                    int half, int col, int lane, T* scratch) {
  constexpr int kStride = lds_stride<32>();
#pragma unroll
  for (int g = 0; g < 4; g++) {
    uint32_t lo = pack2<T>(acc[4 * g] * scale, acc[4 * g + 1] * scale), hi = pack2<T>(acc[4 * g + 2] * scale, acc[4 * g + 3] * scale);
    *reinterpret_cast<uint64_t*>(scratch + col * kStride + 8 * g + 4 * half) = (uint64_t)lo | ((uint64_t)hi << 32);
  }
  const int voff = col * sink.stride_bytes + 8 * half * (int)sizeof(T);
  const int sbase = __builtin_amdgcn_readfirstlane(row0 * sink.stride_bytes + col0 * (int)sizeof(T));
#pragma unroll
  for (int c = 0; c < 2; c++) {
    const typename Elem<T>::vec8 v = lds_col8<T>(scratch, kStride, 16 * c + 8 * half, 0, lane);   // row `col`, columns 16c+8half..+7
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), sink.rsrc, voff, sbase + 16 * c * (int)sizeof(T), 0);
  }
}

// Rows of the packed token axis that belong to no sequence (total_tokens beyond the last cu_seqlens entry, or every
// row when the scheduler voided the schedule) are zero-filled by the workgroups that find no tile: idle slot
// `slot - counts[kCountQ]` of a head clears `rows` rows of that head starting at counts[kCountCovered].  The launch
// provides ceil(total_tokens / 128) + num_seqs slots per head, which leaves at least ceil(uncovered / 128) idle.
// (The reference allocates zero-filled gradients and rem: sb_varlen_bwd.py:506-508, sb_varlen_fwd.py:418.)
__device__ __forceinline__ bool uncovered_rows(const int32_t* counts, int slot, int64_t total_tokens, int sub, int rows,
                                               int64_t* r0, int64_t* r1) {
  *r0 = (int64_t)counts[kCountCovered] + (int64_t)kBlockQ * (slot - counts[kCountQ]) + (int64_t)sub * rows;
  *r1 = *r0 + rows < total_tokens ? *r0 + rows : total_tokens;
  return *r0 < *r1;
}
template <typename T>
__device__ __forceinline__ void zero_rows(const TensorRef& t, int head, int64_t r0, int64_t r1, int d) {
  T* b = (T*)t.ptr + head * t.sh;
  const int64_t n = (r1 - r0) * d;
  for (int64_t idx = threadIdx.x; idx < n; idx += blockDim.x) b[(r0 + idx / d) * t.st + idx % d] = (T)0;
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also drains the vector-memory counter, which
// would stall on global loads that are deliberately left in flight across the barrier (staging registers, the next
// tile's operands).  For kernels in which nothing is communicated through global memory.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Map the linear workgroup id to (head, tile slot) so that the workgroups of one head land on one XCD
// (workgroups are dealt round-robin to the 8 XCDs, each with a private L2): K/V of a head are then
// re-read from that XCD's L2 rather than from HBM.
__device__ __forceinline__ void xcd_head_tile(int wg, int num_heads, int* head, int* slot) {
  if ((num_heads & 7) == 0) {
    const int hpx = num_heads >> 3;
    const int xcd = wg & 7, r = wg >> 3;
    *head = xcd * hpx + (r % hpx);
    *slot = r / hpx;
  } else {
    *head = wg % num_heads;
    *slot = wg / num_heads;
  }
}

}  // namespace sba
