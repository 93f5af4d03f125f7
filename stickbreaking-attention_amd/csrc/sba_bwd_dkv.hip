// Backward, kernel 2 of 2: dK and dV, key-stationary and lock-free.
//
// One workgroup owns one tile of 64 keys of one (head, sequence) and sweeps every tile of 128 query rows that
// can see it.  For each query tile it recomputes, in the same lane-owns-a-query layout as the other kernels,
//     P^T  and  dZ^T = (g - sigma * C)^T        for its 64 keys,
// starting the per-row scans from the values recorded for (row, this key tile) -- the product of (1 - sigma)
// over the keys above the tile by the forward, the prefix sum of g below the tile by the dQ kernel --, writes both as
// 16-bit [query][key] tiles to LDS, and contracts them over the 128 queries on the MFMA:
//     dV += P^T dO        dK += dZ^T Q
// with the LDS transpose read supplying every operand that has to be gathered down the rows of a row-major
// tile.  Each element of dK/dV is accumulated in fp32 registers by exactly one workgroup and stored once, in
// place of the reference's spin-locked read-modify-write of 16-bit dK/dV tiles
// (stickbreaking_attention/sb_varlen/sb_varlen_bwd.py:11-53, :450-465).
#include "sba_device.hpp"
#include "sba_params.hpp"

namespace sba {

template <int DH> struct DkvLds {
  static constexpr int kRowStride = lds_stride<DH>();
  static constexpr int kPStride = lds_stride<kBlockK>();
  static constexpr int kQ = 0;
  static constexpr int kDo = kQ + kBlockQ * kRowStride;
  static constexpr int kK = kDo + kBlockQ * kRowStride;
  static constexpr int kV = kK + kBlockK * kRowStride;
  static constexpr int kP = kV + kBlockK * kRowStride;
  static constexpr int kDz = kP + kBlockQ * kPStride;
  static constexpr int kElems = kDz + kBlockQ * kPStride;
};

template <typename T, int DH, bool kFast>
__global__ __launch_bounds__(kThreads) void bwd_dkv_kernel(BwdParams p) {
  typedef typename Elem<T>::vec8 vec8;
  typedef DkvLds<DH> Lds;
  constexpr int kRowStride = Lds::kRowStride, kPStride = Lds::kPStride;
  constexpr int kSteps = DH / 16;
  constexpr int kOutBlocks = 2 * (DH / 32) / kWaves;    // 32x32 output blocks of dK (and of dV) per wave
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  T* lds = reinterpret_cast<T*>(lds_raw);
  T* q_lds = lds + Lds::kQ;
  T* do_lds = lds + Lds::kDo;
  T* k_lds = lds + Lds::kK;
  T* v_lds = lds + Lds::kV;
  T* p_lds = lds + Lds::kP;
  T* dz_lds = lds + Lds::kDz;

  int head, slot;
  xcd_head_tile(blockIdx.x, p.num_heads, &head, &slot);
  if (slot >= p.counts[1]) return;
  const Tile tile = p.k_tiles[slot];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, half = lane >> 5, col = lane & 31;
  const int L = tile.seq_len, j0 = tile.origin, ac = p.attend_current, D = p.head_dim;
  const int64_t tok0 = tile.seq_start;
  const int jt = j0 / kBlockK;

  const T* qb = (const T*)p.q.ptr + tile.seq_id * p.q.sb + head * p.q.sh + tok0 * p.q.st;
  const T* kb = (const T*)p.k.ptr + tile.seq_id * p.k.sb + head * p.k.sh + tok0 * p.k.st;
  const T* vb = (const T*)p.v.ptr + tile.seq_id * p.v.sb + head * p.v.sh + tok0 * p.v.st;
  const T* dob = (const T*)p.d_o.ptr + tile.seq_id * p.d_o.sb + head * p.d_o.sh + tok0 * p.d_o.st;

  // Output blocks of this wave: (row tile mt over keys, column tile dt over head_dim).
  int out_mt[kOutBlocks], out_dt[kOutBlocks];
  if (DH == 128) { out_mt[0] = 0; out_dt[0] = wave; out_mt[kOutBlocks - 1] = 1; out_dt[kOutBlocks - 1] = wave; }
  else { out_mt[0] = wave >> 1; out_dt[0] = wave & 1; }
  f32x16 dkacc[kOutBlocks], dvacc[kOutBlocks];
#pragma unroll
  for (int b = 0; b < kOutBlocks; b++)
#pragma unroll
    for (int r = 0; r < 16; r++) { dkacc[b][r] = 0.f; dvacc[b][r] = 0.f; }

  {
    TileCopy<T, DH, kBlockK, kFast> ck, cv;
    ck.load(kb + (int64_t)j0 * p.k.st, p.k.st, L - j0, D);
    cv.load(vb + (int64_t)j0 * p.v.st, p.v.st, L - j0, D);
    ck.store(k_lds);
    cv.store(v_lds);
  }

  const int first_row = j0 + 1 - ac;                                  // first row that sees key j0
  const int n_qt = (L + kBlockQ - 1) / kBlockQ;
  const int qt_begin = first_row < L ? first_row / kBlockQ : n_qt;    // == jt / 2 whenever any row sees the tile
  const int64_t slot0 = (int64_t)head * p.carry_head_stride + p.carry_base[tile.seq_id] + carry_offset(jt, n_qt) -
                        (int64_t)kBlockQ * (jt >> 1);      // + row
  const float* carry = p.carry + slot0;
  const float* prefix = p.prefix + slot0;

  for (int qt = qt_begin; qt < n_qt; ++qt) {
    const int q0 = qt * kBlockQ;
    __syncthreads();      // previous contraction finished reading q/do/p/dz tiles
    {
      TileCopy<T, DH, kBlockQ, kFast> cq;
      cq.load(qb + (int64_t)q0 * p.q.st, p.q.st, L - q0, D);
      cq.store(q_lds);
      cq.load(dob + (int64_t)q0 * p.d_o.st, p.d_o.st, L - q0, D);
      cq.store(do_lds);
    }
    __syncthreads();

    const int w_first = q0 + wave * 32, w_last = w_first + 31;
    const int qi = w_first + col;
    const bool row_ok = qi < L;
    uint32_t pk[16], dzk[16];
    if (j0 > w_last - 1 + ac) {
      // no row of this wave sees the tile: contributes zeros
#pragma unroll
      for (int i = 0; i < 16; i++) { pk[i] = 0; dzk[i] = 0; }
    } else {
      const bool diagonal = (j0 + kBlockK - 1) > (w_first - 1 + ac) || w_last >= L;
      float drem = 0.f;
      if (row_ok && p.d_rem.ptr)
        drem = (float)((const T*)p.d_rem.ptr)[tile.seq_id * p.d_rem.sb + head * p.d_rem.sh + (tok0 + qi) * p.d_rem.st];
      const float prod_in = carry[qi], prefix_in = prefix[qi];
      f32x16 s[2], dp[2];
#pragma unroll
      for (int mt = 0; mt < 2; mt++) {
#pragma unroll
        for (int r = 0; r < 16; r++) { s[mt][r] = 0.f; dp[mt][r] = 0.f; }
        const int krow = mfma_row_to_key(mt, col);
#pragma unroll
        for (int kk = 0; kk < kSteps; kk++) {
          vec8 a = lds_row8<T>(k_lds, kRowStride, krow, 16 * kk + 8 * half);
          vec8 b = lds_row8<T>(q_lds, kRowStride, wave * 32 + col, 16 * kk + 8 * half);
          s[mt] = Elem<T>::mfma(a, b, s[mt]);
        }
#pragma unroll
        for (int kk = 0; kk < kSteps; kk++) {
          vec8 a = lds_row8<T>(v_lds, kRowStride, krow, 16 * kk + 8 * half);
          vec8 b = lds_row8<T>(do_lds, kRowStride, wave * 32 + col, 16 * kk + 8 * half);
          dp[mt] = Elem<T>::mfma(a, b, dp[mt]);
        }
      }
      const int lim = row_ok ? qi + ac - j0 - 32 * half : 0;
      float prefix_next;
      bwd_tile_math<T>(s, dp, p.scale_log2, diagonal, lim, half, drem, prod_in, prefix_in, pk, dzk, prefix_next);
    }
    // [query][key] tiles: this lane's 32 consecutive keys start at column 32*half of row 32*wave + col.
    {
      u32x4* pp = reinterpret_cast<u32x4*>(p_lds + (wave * 32 + col) * kPStride + 32 * half);
      u32x4* dd = reinterpret_cast<u32x4*>(dz_lds + (wave * 32 + col) * kPStride + 32 * half);
#pragma unroll
      for (int c = 0; c < 4; c++) {
        pp[c] = u32x4{pk[4 * c], pk[4 * c + 1], pk[4 * c + 2], pk[4 * c + 3]};
        dd[c] = u32x4{dzk[4 * c], dzk[4 * c + 1], dzk[4 * c + 2], dzk[4 * c + 3]};
      }
    }
    __syncthreads();

    // dV[key][d] += sum_i P[i][key] dO[i][d];  dK[key][d] += sum_i dZ[i][key] Q[i][d]   (i over the 128 rows)
#pragma unroll
    for (int b = 0; b < kOutBlocks; b++) {
#pragma unroll
      for (int c = 0; c < kBlockQ / 16; c++) {
        const int row0 = 16 * c + 8 * half;
        vec8 ap = lds_col8<T>(p_lds, kPStride, row0, 32 * out_mt[b], lane);
        vec8 bd = lds_col8<T>(do_lds, kRowStride, row0, 32 * out_dt[b], lane);
        dvacc[b] = Elem<T>::mfma(ap, bd, dvacc[b]);
        vec8 az = lds_col8<T>(dz_lds, kPStride, row0, 32 * out_mt[b], lane);
        vec8 bq = lds_col8<T>(q_lds, kRowStride, row0, 32 * out_dt[b], lane);
        dkacc[b] = Elem<T>::mfma(az, bq, dkacc[b]);
      }
    }
  }

  // acc[b][r]: key 32*mt + 8*(r/4) + 4*half + r%4 of the tile, column 32*dt + col.
  T* dkb = (T*)p.dk.ptr + tile.seq_id * p.dk.sb + head * p.dk.sh + tok0 * p.dk.st;
  T* dvb = (T*)p.dv.ptr + tile.seq_id * p.dv.sb + head * p.dv.sh + tok0 * p.dv.st;
#pragma unroll
  for (int b = 0; b < kOutBlocks; b++) {
    const int d = 32 * out_dt[b] + col;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int key = j0 + 32 * out_mt[b] + 8 * (r >> 2) + 4 * half + (r & 3);
      if (key < L && d < D) {
        dkb[(int64_t)key * p.dk.st + d] = (T)(dkacc[b][r] * p.logit_scale);
        dvb[(int64_t)key * p.dv.st + d] = (T)dvacc[b][r];
      }
    }
  }
}

template <typename T, int DH, bool kFast>
static hipError_t launch_one(const BwdParams& p, int max_tiles, hipStream_t stream) {
  const size_t lds_bytes = (size_t)DkvLds<DH>::kElems * sizeof(T);
  // The tile set exceeds the default 64 KB dynamic-LDS cap; the attribute is per device and cheap to set.
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&bwd_dkv_kernel<T, DH, kFast>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
  if (e != hipSuccess) return e;
  const dim3 grid((unsigned)(max_tiles * p.num_heads)), block(kThreads);
  hipLaunchKernelGGL((bwd_dkv_kernel<T, DH, kFast>), grid, block, lds_bytes, stream, p);
  return hipGetLastError();
}

template <typename T>
static hipError_t launch_t(const BwdParams& p, int max_tiles, hipStream_t stream) {
  if (p.vec_ok && p.head_dim == 128) return launch_one<T, 128, true>(p, max_tiles, stream);
  if (p.vec_ok && p.head_dim == 64) return launch_one<T, 64, true>(p, max_tiles, stream);
  return p.head_dim <= 64 ? launch_one<T, 64, false>(p, max_tiles, stream) : launch_one<T, 128, false>(p, max_tiles, stream);
}

hipError_t launch_bwd_dkv(const BwdParams& p, int dtype_is_f16, int max_tiles, hipStream_t stream) {
  return dtype_is_f16 ? launch_t<_Float16>(p, max_tiles, stream) : launch_t<__bf16>(p, max_tiles, stream);
}

}  // namespace sba
