// Backward, kernel 1 of 2: dQ, plus the per-(row, key tile) prefix sums that make the dK/dV kernel lock-free.
//
// One workgroup per tile of 128 query rows (wave w owns rows 32w..32w+31, lane l owns query l%32), key tiles
// of KT keys (32 on the fast paths, else 64) swept FORWARDS from key 0 to the diagonal.  With g_ij = A_ij (dO_i.v_j - drem_i) the logit gradient is
//     dz_ij = g_ij - sigma_ij * C_ij,     C_ij = sum_{j' <= j} g_ij'        (sb_varlen_bwd.py:438-447)
// so C is a running prefix sum in this direction and needs no anchor.  (sigma does not decay with distance, so
// any constant error in C would be multiplied into every key of the row; C has to be built from exactly the g
// values it sums.)  A_ij needs the product of (1 - sigma) over the keys ABOVE j instead.  The reference gets
// it by subtracting a running log-sum from the saved row total (sb_varlen_fwd.py:52-53), which cancels badly
// on long rows with saturated logits; here the forward, which sweeps downwards from the diagonal, has
// recorded that product at every tile boundary, and the scan inside a tile runs downwards in registers.
//
// Before each key tile J the kernel records C just below J for every row: together with the forward's
// products the key-stationary dK/dV kernel can start its per-tile scans from these, so no tile of dK or dV
// is ever accumulated by more than one workgroup (the reference serialises that accumulation behind a spin
// lock per key tile: sb_varlen_bwd.py:11-53).
#include "sba_device.hpp"
#include "sba_params.hpp"

#include <type_traits>

namespace sba {

template <typename T, int DH, bool kFast, int KT>
__global__ __launch_bounds__(kThreads, KT == 32 ? 2 : 1) void bwd_dq_kernel(BwdParams p) {
  constexpr int NT = KT / 32;         // MFMA row tiles per key tile: a lane owns 16*NT consecutive keys
  typedef typename Elem<T>::vec8 vec8;
  constexpr int kRowStride = lds_stride<DH>();
  constexpr int kSteps = DH / 16;
  constexpr int kDTiles = DH / 32;
  __shared__ __attribute__((aligned(16))) T k_lds[KT * kRowStride];
  __shared__ __attribute__((aligned(16))) T v_lds[KT * kRowStride];

  int head, slot;
  xcd_head_tile(blockIdx.x, p.num_heads, &head, &slot);
  if (slot >= p.counts[kCountQ]) {
    int64_t r0, r1;
    if (uncovered_rows(p.counts, slot, p.total_tokens, 0, kBlockQ, &r0, &r1)) {      // rows of no sequence: zero gradients
      zero_rows<T>(p.dq, head, r0, r1, p.head_dim);
      zero_rows<T>(p.dk, head, r0, r1, p.head_dim);
      zero_rows<T>(p.dv, head, r0, r1, p.head_dim);
    }
    return;
  }
  const Tile tile = p.q_tiles[slot];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, half = lane >> 5, col = lane & 31;
  const int L = tile.seq_len, q0 = tile.origin, ac = p.attend_current, D = p.head_dim;
  const int64_t tok0 = tile.seq_start;

  const T* qb = (const T*)p.q.ptr + tile.seq_id * p.q.sb + head * p.q.sh + tok0 * p.q.st;
  const T* kb = (const T*)p.k.ptr + tile.seq_id * p.k.sb + head * p.k.sh + tok0 * p.k.st;
  const T* vb = (const T*)p.v.ptr + tile.seq_id * p.v.sb + head * p.v.sh + tok0 * p.v.st;
  const T* dob = (const T*)p.d_o.ptr + tile.seq_id * p.d_o.sb + head * p.d_o.sh + tok0 * p.d_o.st;

  const int qi = q0 + wave * 32 + col;
  const bool row_ok = qi < L;
  vec8 qf[kSteps], dof[kSteps];
#pragma unroll
  for (int kk = 0; kk < kSteps; kk++) {
    const int d0 = 16 * kk + 8 * half;
    qf[kk] = as_vec8<T>(load_row8<T, kFast>(qb + (int64_t)qi * p.q.st, d0, D, row_ok));
    dof[kk] = as_vec8<T>(load_row8<T, kFast>(dob + (int64_t)qi * p.d_o.st, d0, D, row_ok));
  }
  float drem = 0.f;
  if (row_ok && p.d_rem.ptr)
    drem = (float)((const T*)p.d_rem.ptr)[tile.seq_id * p.d_rem.sb + head * p.d_rem.sh + (tok0 + qi) * p.d_rem.st];
  if (p.add_rem) {
    // The forward wrote o + rem * v: the gradient reaching rem is d_rem + d_o . v_i.
    float dot = 0.f;
#pragma unroll
    for (int kk = 0; kk < kSteps; kk++) {
      const vec8 vv = as_vec8<T>(load_row8<T, kFast>(vb + (int64_t)qi * p.v.st, 16 * kk + 8 * half, D, row_ok));
#pragma unroll
      for (int t = 0; t < 8; t++) dot = fmaf((float)dof[kk][t], (float)vv[t], dot);
    }
    drem += dot + other_half(dot, half);
  }
  // The dK/dV kernel reads the gradient of rem back from this fp32 plane (one value per row).
  if (half == 0 && row_ok) p.drem_eff[tile.seq_id * p.drem_sb + head * p.stat_sh + tok0 + qi] = drem;
  float prefix = 0.f;      // sum of g over the keys already swept (both half-waves hold the same value)

  const int last_row = min(q0 + kBlockQ, L) - 1;
  const int last_key = last_row - 1 + ac;
  const int n_kt = last_key < 0 ? 0 : last_key / KT + 1;
  const int w_first = q0 + wave * 32, w_last = w_first + 31;
  const int64_t n_qt = (L + kBlockQ - 1) / kBlockQ;
  const int64_t slot0 = (int64_t)head * p.carry_head_stride + tile.carry_base;
  const float* carry = p.carry + slot0;
  float* prefix_out = p.prefix + slot0;

  f32x16 dqacc[kDTiles];
#pragma unroll
  for (int dt = 0; dt < kDTiles; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) dqacc[dt][r] = 0.f;

  // The forward's product above the next key tile (above its upper sub-tile), fetched one tile ahead.
  // sub-tile whose upper edge is the upper edge of key tile t, and the first row that owns slots for tile t
  auto carry_slot = [&](int t) {
    const int u = NT == 2 ? 2 * t + 1 : t;
    return carry_offset(u, n_qt) + (qi - kBlockQ * (u >> 2));
  };
  float n_prod = 1.f;
  const RowSource<T> ksrc = make_row_source<T, kFast>(kb, p.k.st, L, D), vsrc = make_row_source<T, kFast>(vb, p.v.st, L, D);
  TileCopy<T, DH, KT, kFast> ck, cv;
  if (n_kt > 0) {
    ck.load(ksrc, 0);
    cv.load(vsrc, 0);
    n_prod = carry[carry_slot(0)];
  }
  for (int jt = 0; jt < n_kt; ++jt) {
    const int j0 = jt * KT;
    __syncthreads();
    ck.store(k_lds);
    cv.store(v_lds);
    __syncthreads();
    const float prod_in = n_prod;
    if (jt + 1 < n_kt) {
      const int jn = j0 + KT;
      ck.load(ksrc, jn);
      cv.load(vsrc, jn);
      n_prod = carry[carry_slot(jt + 1)];
    }
    // For the key-stationary kernel: C just below each 32-key sub-tile, for every row of the tile.
    const int u_lo = NT == 2 ? 2 * jt : jt;
    const int64_t slot_lo = carry_offset(u_lo, n_qt) + (qi - kBlockQ * (u_lo >> 2));
    const int64_t slot_hi = carry_offset(u_lo + 1, n_qt) + (qi - kBlockQ * (u_lo >> 2));     // NT == 2 only
    if (half == 0) prefix_out[slot_lo] = prefix;
    if (j0 > w_last - 1 + ac) {
      if (NT == 2 && half == 0) prefix_out[slot_hi] = prefix;
      continue;
    }
    const bool diagonal = (j0 + KT - 1) > (w_first - 1 + ac) || w_last >= L;

    f32x16 s[NT], dp[NT];
    const int lim = row_ok ? qi + ac - j0 - (KT / 2) * half : 0;
    uint32_t pk[8 * NT], dzk[8 * NT];
    float prod_lower, prefix_upper;
    if (NT == 1 && kFast) {
      // 32-key steps: S^T first; the dP^T MFMAs are dealt among the element-wise math (its first phase only needs
      // S), one MFMA per kGap vector-ALU instructions, so that the matrix pipe runs under the vector ALU.
      const int krow = mfma_row_to_key32(col);
#pragma unroll
      for (int r = 0; r < 16; r++) { s[0][r] = 0.f; dp[0][r] = 0.f; }
#pragma unroll
      for (int kk = 0; kk < kSteps; kk++) s[0] = Elem<T>::mfma(lds_row8<T>(k_lds, kRowStride, krow, 16 * kk + 8 * half), qf[kk], s[0]);
      auto math = [&](auto diag_tag) {
        constexpr bool kDiag = decltype(diag_tag)::value;
        constexpr int kGap = 96 / kSteps;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int kk = 0; kk < kSteps; kk++) dp[0] = Elem<T>::mfma(lds_row8<T>(v_lds, kRowStride, krow, 16 * kk + 8 * half), dof[kk], dp[0]);
        bwd_tile_math_impl<T, NT, kDiag, false>(s, dp, p.scale_log2, lim, half, drem, prod_in, prefix, pk, dzk, prod_lower, prefix_upper, prefix);
        __builtin_amdgcn_sched_group_barrier(0x100, kSteps, 0);
        __builtin_amdgcn_sched_group_barrier(0x402, 8, 0);
#pragma unroll
        for (int kk = 0; kk < kSteps; kk++) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x402, kGap, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      };
      if (diagonal) math(std::true_type{}); else math(std::false_type{});
    } else {
#pragma unroll
      for (int mt = 0; mt < NT; mt++) {
#pragma unroll
        for (int r = 0; r < 16; r++) { s[mt][r] = 0.f; dp[mt][r] = 0.f; }
        const int krow = NT == 2 ? mfma_row_to_key(mt, col) : mfma_row_to_key32(col);
#pragma unroll
        for (int kk = 0; kk < kSteps; kk++) {
          vec8 a = lds_row8<T>(k_lds, kRowStride, krow, 16 * kk + 8 * half);
          s[mt] = Elem<T>::mfma(a, qf[kk], s[mt]);
        }
#pragma unroll
        for (int kk = 0; kk < kSteps; kk++) {
          vec8 a = lds_row8<T>(v_lds, kRowStride, krow, 16 * kk + 8 * half);
          dp[mt] = Elem<T>::mfma(a, dof[kk], dp[mt]);
        }
      }
      bwd_tile_math<T, NT, false>(s, dp, p.scale_log2, diagonal, lim, half, drem, prod_in, prefix, pk, dzk, prod_lower,
                           prefix_upper, prefix);
    }
    if (NT == 2 && half == 0) prefix_out[slot_hi] = prefix_upper;

    // dQ += dZ K: A = dZ from registers, B = K gathered down the keys.
#pragma unroll
    for (int c = 0; c < KT / 16; c++) {
      u32x4 av = {dzk[4 * c], dzk[4 * c + 1], dzk[4 * c + 2], dzk[4 * c + 3]};
      vec8 a = as_vec8<T>(av);
#pragma unroll
      for (int dt = 0; dt < kDTiles; dt++) {
        vec8 b = lds_col8<T>(k_lds, kRowStride, (KT / 2) * half + 8 * c, 32 * dt, lane);
        dqacc[dt] = Elem<T>::mfma(a, b, dqacc[dt]);
      }
    }
  }

  T* dqb = (T*)p.dq.ptr + tile.seq_id * p.dq.sb + head * p.dq.sh + tok0 * p.dq.st;
  if (kFast) {
    const RowSink<T> sink = make_row_sink<T>(dqb, p.dq.st, L, D);
#pragma unroll
    for (int dt = 0; dt < kDTiles; dt++) store_acc_tile<T>(sink, dqacc[dt], p.logit_scale, w_first, 32 * dt, half, col);
    return;
  }
#pragma unroll
  for (int dt = 0; dt < kDTiles; dt++) {
    const int d = 32 * dt + col;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int row = w_first + 8 * (r >> 2) + 4 * half + (r & 3);
      if (row < L && d < D) dqb[(int64_t)row * p.dq.st + d] = (T)(dqacc[dt][r] * p.logit_scale);
    }
  }
}

template <typename T>
static hipError_t launch_t(const BwdParams& p, int max_tiles, hipStream_t stream) {
  const dim3 grid((unsigned)(max_tiles * p.num_heads)), block(kThreads);
  if (p.vec_ok && p.head_dim == 128) {
    hipLaunchKernelGGL((bwd_dq_kernel<T, 128, true, 32>), grid, block, 0, stream, p);
  } else if (p.vec_ok && p.head_dim == 64) {
    hipLaunchKernelGGL((bwd_dq_kernel<T, 64, true, 32>), grid, block, 0, stream, p);
  } else if (p.head_dim <= 64) {
    hipLaunchKernelGGL((bwd_dq_kernel<T, 64, false, 64>), grid, block, 0, stream, p);
  } else {
    hipLaunchKernelGGL((bwd_dq_kernel<T, 128, false, 64>), grid, block, 0, stream, p);
  }
  return hipGetLastError();
}

hipError_t launch_bwd_dq(const BwdParams& p, int dtype_is_f16, int max_tiles, hipStream_t stream) {
  return dtype_is_f16 ? launch_t<_Float16>(p, max_tiles, stream) : launch_t<__bf16>(p, max_tiles, stream);
}

}  // namespace sba
