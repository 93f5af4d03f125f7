// Forward stick-breaking attention for gfx950.
//
// One workgroup = one tile of 128 query rows of one (head, sequence); wave w owns rows 32w..32w+31, lane l
// owns query l%32.  Key tiles of KT keys (32 on the head_dim 128 fast path, else 64) are swept in REVERSE from the
// causal diagonal (the order in which the stick is broken:
// stickbreaking_attention/sb_varlen/sb_varlen_fwd.py:155-165), so the running product
// prod_{j<k<i} (1 - sigma(z_ik)) is carried forward in registers and never has to be divided out.
//
// Per element, in linear space (base-2 exponentials, as sb_varlen_fwd.py:296 and softplus.py:8-12 do):
//     e = 2^x, x = z log2(e)          1 - sigma = 1/(1+e)          R_ij = prod_{j<=k<i} 1/(1+e_ik)
//     A_ij = sigma_ij R_i,j+1 = R_i,j+1 - R_ij
// which needs two transcendentals (v_exp_f32, v_rcp_f32) where the log-space form
// log A = x - softplus2(x) + cumsum(-softplus2) needs three.  The product can only underflow where A itself is
// below 2^-126, and row_stat = log2(prod) is taken once per row at the end.
#include "sba_device.hpp"
#include "sba_params.hpp"

namespace sba {

// kCarryOnly: only the products of (1 - sigma) above every sub-tile are rebuilt (into `carry`), for a backward whose
// forward did not keep them: no V, no P V, no outputs.
template <typename T, int DH, bool kFast, int KT, int kMinWaves, bool kCarryOnly = false>
__global__ __launch_bounds__(kThreads, kMinWaves) void fwd_kernel(FwdParams p) {
  constexpr int NT = KT / 32;         // MFMA row tiles per key tile: a lane owns N = 16*NT consecutive keys
  constexpr int N = 16 * NT;
  typedef typename Elem<T>::vec8 vec8;
  constexpr int kRowStride = lds_stride<DH>();
  constexpr int kSteps = DH / 16;    // MFMA k-steps over head_dim
  constexpr int kDTiles = DH / 32;   // 32-wide output tiles over head_dim
  __shared__ __attribute__((aligned(16))) T k_lds[KT * kRowStride];
  __shared__ __attribute__((aligned(16))) T v_lds[KT * kRowStride];

  int head, slot;
  xcd_head_tile(blockIdx.x, p.num_heads, &head, &slot);
  if (slot >= p.counts[kCountQ]) {
    int64_t r0, r1;
    if (!kCarryOnly && uncovered_rows(p.counts, slot, p.total_tokens, 0, kBlockQ, &r0, &r1)) {      // rows of no sequence: o = rem = 0
      zero_rows<T>(p.o, head, r0, r1, p.head_dim);
      for (int64_t r = r0 + threadIdx.x; r < r1; r += kThreads) {
        ((T*)p.rem.ptr)[head * p.rem.sh + r * p.rem.st] = (T)0;
        p.row_stat[head * p.stat_sh + r] = 0.f;
      }
    }
    return;
  }
  const Tile tile = p.tiles[slot];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, half = lane >> 5, col = lane & 31;
  const int L = tile.seq_len, q0 = tile.origin, ac = p.attend_current, D = p.head_dim;

  const T* qb = (const T*)p.q.ptr + tile.seq_id * p.q.sb + head * p.q.sh + (int64_t)tile.seq_start * p.q.st;
  const T* kb = (const T*)p.k.ptr + tile.seq_id * p.k.sb + head * p.k.sh + (int64_t)tile.seq_start * p.k.st;
  const T* vb = (const T*)p.v.ptr + tile.seq_id * p.v.sb + head * p.v.sh + (int64_t)tile.seq_start * p.v.st;

  // This lane's query row as the B operand of S^T = K Q^T: 8 consecutive head_dim elements per k-step.
  const int qi = q0 + wave * 32 + col;
  vec8 qf[kSteps];
#pragma unroll
  for (int kk = 0; kk < kSteps; kk++)
    qf[kk] = as_vec8<T>(load_row8<T, kFast>(qb + (int64_t)qi * p.q.st, 16 * kk + 8 * half, D, qi < L));

  const int last_row = min(q0 + kBlockQ, L) - 1;
  const int last_key = last_row - 1 + ac;                    // last key any row of this tile can see
  const int n_kt = last_key < 0 ? 0 : last_key / KT + 1;
  const int w_first = q0 + wave * 32, w_last = w_first + 31;   // this wave's rows

  f32x16 oacc[kDTiles];
#pragma unroll
  for (int dt = 0; dt < kDTiles; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) oacc[dt][r] = 0.f;
  float prod = 1.f;    // prod over the keys already swept of (1 - sigma): both half-waves hold the same value
  const int64_t n_qt = (L + kBlockQ - 1) / kBlockQ;
  float* carry = p.carry ? p.carry + (int64_t)head * p.carry_head_stride + tile.carry_base : nullptr;

  const RowSource<T> ksrc = make_row_source<T, kFast>(kb, p.k.st, L, D), vsrc = make_row_source<T, kFast>(vb, p.v.st, L, D);
  TileCopy<T, DH, KT, kFast> ck, cv;
  if (n_kt > 0) {
    ck.load(ksrc, (n_kt - 1) * KT);
    if (!kCarryOnly) cv.load(vsrc, (n_kt - 1) * KT);
  }
  // The recorded products are read per 64-key tile by the backward kernels that sweep 64 keys at a time, whichever
  // forward variant ran: a 32-key sweep that ends on the lower half of such a tile also records the (empty) product
  // above the upper half.
  if (NT == 1 && carry && half == 0 && (n_kt & 1)) carry[carry_offset(n_kt, n_qt) + (qi - kBlockQ * (n_kt >> 2))] = 1.f;
  for (int jt = n_kt - 1; jt >= 0; --jt) {
    const int j0 = jt * KT;
    __syncthreads();
    ck.store(k_lds);
    if (!kCarryOnly) cv.store(v_lds);
    __syncthreads();
    if (jt > 0) {
      const int jn = j0 - KT;
      ck.load(ksrc, jn);
      if (!kCarryOnly) cv.load(vsrc, jn);
    }
    // For the backward: the product over the keys between the upper 32-key sub-tile and the row, for every row
    // of the tile (the lower sub-tile's value follows once this tile's upper half is known).
    const int u_hi = NT == 2 ? 2 * jt + 1 : jt;                // sub-tile at the upper edge of this tile
    const int64_t cslot = qi - kBlockQ * (u_hi >> 2);
    if (carry && half == 0) carry[carry_offset(u_hi, n_qt) + cslot] = prod;
    if (j0 > w_last - 1 + ac) {                               // nothing visible to this wave yet
      if (NT == 2 && carry && half == 0) carry[carry_offset(u_hi - 1, n_qt) + cslot] = prod;
      continue;
    }
    const bool diagonal = (j0 + KT - 1) > (w_first - 1 + ac);

    // The two MFMA phases of a step run at raised wave priority, the element-wise math at the default: a wave whose
    // next MFMA is ready then gets the issue port ahead of the other waves' vector-ALU streams (measured: -3 %).
    __builtin_amdgcn_s_setprio(3);
    // S^T tile: rows = keys (permuted so that a lane ends up with 32 consecutive keys), columns = queries.
    f32x16 s[NT];
#pragma unroll
    for (int mt = 0; mt < NT; mt++) {
#pragma unroll
      for (int r = 0; r < 16; r++) s[mt][r] = 0.f;
      const int krow = NT == 2 ? mfma_row_to_key(mt, col) : mfma_row_to_key32(col);
      if (NT == 1 && kFast) {
        // The K operands are requested four ahead of the MFMA that uses them: requested two at a time (what the
        // register allocator otherwise settles for) the wave pays the LDS latency four times per step.
        vec8 a[kSteps];
#pragma unroll
        for (int kk = 0; kk < 4; kk++) a[kk] = lds_row8<T>(k_lds, kRowStride, krow, 16 * kk + 8 * half);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int kk = 0; kk < kSteps; kk++) {
          s[mt] = Elem<T>::mfma(a[kk], qf[kk], s[mt]);
          if (kk + 4 < kSteps) a[kk + 4] = lds_row8<T>(k_lds, kRowStride, krow, 16 * (kk + 4) + 8 * half);
          __builtin_amdgcn_sched_barrier(0);
        }
      } else {
#pragma unroll
        for (int kk = 0; kk < kSteps; kk++) {
          vec8 a = lds_row8<T>(k_lds, kRowStride, krow, 16 * kk + 8 * half);
          s[mt] = Elem<T>::mfma(a, qf[kk], s[mt]);
        }
      }
    }

    // This lane's N keys are j0 + N*half + R, R = 16*mt + r, swept from R = N-1 down.
    //   t[R] = sigma[R] * prod_{R' > R} (1 - sigma[R']) = run_before - run_after   with run *= 1/(1+e[R])
    // (the weight of key R up to the product carried into the tile).  The difference form needs neither sigma
    // nor a clamp: e = inf gives a factor 0 and the whole remaining stick as weight; its absolute error is one
    // ulp of the running product.  Hidden keys (diagonal tiles only) get e = 0: factor 1, weight 0.
    __builtin_amdgcn_s_setprio(0);
    float t[N];
    float run = 1.f;
    if (diagonal) {
      const int lim = qi + ac - j0 - N * half;                // key R is visible iff R < lim
#pragma unroll
      for (int R = N - 1; R >= 0; --R) {
        float x = s[R >> 4][R & 15] * p.scale_log2;
        x = (R < lim) ? x : -INFINITY;
        const float before = run;
        run *= fast_rcp(1.f + fast_exp2(x));
        t[R] = before - run;
      }
    } else {
#pragma unroll
      for (int R = N - 1; R >= 0; --R) {
        const float before = run;
        run *= fast_rcp(1.f + fast_exp2(s[R >> 4][R & 15] * p.scale_log2));
        t[R] = before - run;
      }
    }
    const float oth = other_half(run, half);
    // The upper half-wave holds the higher keys, which come first in the sweep.
    const float seed = half ? prod : prod * oth;
    if (NT == 2 && carry && half == 0) carry[carry_offset(u_hi - 1, n_qt) + cslot] = seed;   // product above the lower sub-tile
    prod = (prod * oth) * run;
    if (kCarryOnly) continue;

    __builtin_amdgcn_s_setprio(3);
    // O += P V: A = P from registers (k index <-> key 32*half + 8c + t), B = V gathered down the keys.
#pragma unroll
    for (int c = 0; c < KT / 16; c++) {
      u32x4 av;
#pragma unroll
      for (int i = 0; i < 4; i++) av[i] = pack2<T>(t[8 * c + 2 * i] * seed, t[8 * c + 2 * i + 1] * seed);
      vec8 a = as_vec8<T>(av);
#pragma unroll
      for (int dt = 0; dt < kDTiles; dt++) {
        vec8 b = lds_col8<T>(v_lds, kRowStride, N * half + 8 * c, 32 * dt, lane);
        oacc[dt] = Elem<T>::mfma(a, b, oacc[dt]);
      }
    }
    __builtin_amdgcn_s_setprio(0);
  }

  if (kCarryOnly) return;
  // Epilogue.  oacc[dt][r]: query row 8*(r/4) + 4*half + r%4 of this wave, column 32*dt + col.
  T* ob = (T*)p.o.ptr + tile.seq_id * p.o.sb + head * p.o.sh + (int64_t)tile.seq_start * p.o.st;
  if (p.add_rem) {
    // o + rem * v (the step callers of the reference apply to its outputs, tests/test_varlen.py:103): the row's
    // remainder is held by the lane whose query it is.
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int lr = 8 * (r >> 2) + 4 * half + (r & 3);
      const int row = w_first + lr;
      const float rem_row = __shfl(prod, lr);
#pragma unroll
      for (int dt = 0; dt < kDTiles; dt++) {
        const int d = 32 * dt + col;
        if (row < L && d < D)
          ob[(int64_t)row * p.o.st + d] = (T)(oacc[dt][r] + rem_row * (float)vb[(int64_t)row * p.v.st + d]);
      }
    }
  } else if (kFast) {
    const RowSink<T> sink = make_row_sink<T>(ob, p.o.st, L, D);
#pragma unroll
    for (int dt = 0; dt < kDTiles; dt++) store_acc_tile<T>(sink, oacc[dt], 1.f, w_first, 32 * dt, half, col);
  } else {
#pragma unroll
    for (int dt = 0; dt < kDTiles; dt++) {
      const int d = 32 * dt + col;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int row = w_first + 8 * (r >> 2) + 4 * half + (r & 3);
        if (row < L && d < D) ob[(int64_t)row * p.o.st + d] = (T)oacc[dt][r];
      }
    }
  }
  if (half == 0 && qi < L) {
    T* rb = (T*)p.rem.ptr + tile.seq_id * p.rem.sb + head * p.rem.sh + (int64_t)(tile.seq_start + qi) * p.rem.st;
    *rb = (T)prod;
    p.row_stat[tile.seq_id * p.stat_sb + head * p.stat_sh + tile.seq_start + qi] = fast_log2(prod);
  }
}

template <typename T, bool kCarryOnly>
static hipError_t launch_fwd_t(const FwdParams& p, int max_tiles, hipStream_t stream) {
  const dim3 grid((unsigned)(max_tiles * p.num_heads)), block(kThreads);
  if (p.vec_ok && p.head_dim == 128) {
    hipLaunchKernelGGL((fwd_kernel<T, 128, true, 32, 3, kCarryOnly>), grid, block, 0, stream, p);
  } else if (p.vec_ok && p.head_dim == 64) {
    hipLaunchKernelGGL((fwd_kernel<T, 64, true, 64, 2, kCarryOnly>), grid, block, 0, stream, p);
  } else if (p.head_dim <= 64) {
    hipLaunchKernelGGL((fwd_kernel<T, 64, false, 64, 2, kCarryOnly>), grid, block, 0, stream, p);
  } else {
    hipLaunchKernelGGL((fwd_kernel<T, 128, false, 64, 2, kCarryOnly>), grid, block, 0, stream, p);
  }
  return hipGetLastError();
}

hipError_t launch_fwd(const FwdParams& p, int dtype_is_f16, int max_tiles, hipStream_t stream) {
  return dtype_is_f16 ? launch_fwd_t<_Float16, false>(p, max_tiles, stream)
                      : launch_fwd_t<__bf16, false>(p, max_tiles, stream);
}

// The products the backward starts from, rebuilt from q and k alone (p.carry must be set; o, rem, row_stat, v unused).
hipError_t launch_fwd_carry_only(const FwdParams& p, int dtype_is_f16, int max_tiles, hipStream_t stream) {
  return dtype_is_f16 ? launch_fwd_t<_Float16, true>(p, max_tiles, stream)
                      : launch_fwd_t<__bf16, true>(p, max_tiles, stream);
}

}  // namespace sba
