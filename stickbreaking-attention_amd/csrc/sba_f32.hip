// fp32 path: the same operator evaluated entirely in fp32 on the vector ALU (no MFMA), for fp32 inputs.
//
// This is the correctness path behind the 1e-4 tolerance, not a tuned one: one wave walks one query row at a
// time, 64 keys per step with one key per lane, so the stick-breaking product and the prefix sum along the keys
// are wave-level scans.  Workgroup = 4 waves = 16 consecutive rows of a 128-row query tile from the scheduler's
// list (eight workgroups per tile, so that small problems still spread over the chip); wave w owns 4 of them.
//
//   forward : keys swept in reverse from the diagonal (as sb_varlen_fwd.py:155-165), running product per row;
//             records the product above every 64-key step in `carry` (slot of the step's upper 32-key sub-tile).
//   backward: ONE kernel.  Keys swept forwards; per (row, step) it recomputes A from the recorded product,
//             g = A (dO.v - drem), C = prefix sum of g, dz = g - sigma C  (sb_varlen_bwd.py:438-447);
//             dq of the tile's 128 rows and the dk/dv contributions of the current 64-key step are summed in
//             LDS; dk/dv are flushed once per step with fp32 atomics (and zero-filled by a fill kernel first).
//             Summation order across workgroups is therefore not fixed; differences are at the 1e-7 level.
#include "sba_device.hpp"
#include "sba_host.hpp"
#include "sba_params.hpp"

namespace sba {

constexpr int kF32Keys = 64;          // keys per step (one per lane)
constexpr int kMaxD = 128;
constexpr int kF32Rows = 16;          // query rows per workgroup
constexpr int kF32Split = kBlockQ / kF32Rows;
constexpr int kF32RowsPerWave = kF32Rows / kWaves;

__device__ __forceinline__ float wave_bcast(float x, int lane) { return __shfl(x, lane); }

// Inclusive scan over the lanes of a wave from the HIGHEST lane downwards (lane l gets op over lanes >= l).
__device__ __forceinline__ float scan_down_mul(float x, int lane) {
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const float y = __shfl_down(x, d);
    if (lane + d < 64) x *= y;
  }
  return x;
}
// Inclusive scan over the lanes from lane 0 upwards (lane l gets the sum over lanes <= l).
__device__ __forceinline__ float scan_up_add(float x, int lane) {
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const float y = __shfl_up(x, d);
    if (lane >= d) x += y;
  }
  return x;
}

// z_j = scale_log2 * q . k_j for this lane's key (row pointer `krow`, nullptr when the key does not exist).
__device__ __forceinline__ float dot_row(const float* q_lds, const float* krow, int D) {
  float acc = 0.f;
  if (krow)
    for (int d = 0; d < D; d++) acc = fmaf(q_lds[d], krow[d], acc);
  return acc;
}

__global__ __launch_bounds__(kThreads) void fwd_f32_kernel(FwdParams p) {
  __shared__ float q_lds[kWaves][kMaxD];
  int head, slot;
  xcd_head_tile(blockIdx.x / kF32Split, p.num_heads, &head, &slot);
  if (slot >= p.counts[kCountQ]) {
    int64_t r0, r1;
    if (uncovered_rows(p.counts, slot, p.total_tokens, blockIdx.x % kF32Split, kF32Rows, &r0, &r1)) {
      zero_rows<float>(p.o, head, r0, r1, p.head_dim);      // rows of no sequence: o = rem = 0
      for (int64_t r = r0 + threadIdx.x; r < r1; r += kThreads) {
        ((float*)p.rem.ptr)[head * p.rem.sh + r * p.rem.st] = 0.f;
        p.row_stat[head * p.stat_sh + r] = 0.f;
      }
    }
    return;
  }
  const Tile tile = p.tiles[slot];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int row_base = tile.origin + (blockIdx.x % kF32Split) * kF32Rows + wave * kF32RowsPerWave;
  const int L = tile.seq_len, ac = p.attend_current, D = p.head_dim;
  const int64_t tok0 = tile.seq_start;
  const float* qb = (const float*)p.q.ptr + tile.seq_id * p.q.sb + head * p.q.sh + tok0 * p.q.st;
  const float* kb = (const float*)p.k.ptr + tile.seq_id * p.k.sb + head * p.k.sh + tok0 * p.k.st;
  const float* vb = (const float*)p.v.ptr + tile.seq_id * p.v.sb + head * p.v.sh + tok0 * p.v.st;
  float* ob = (float*)p.o.ptr + tile.seq_id * p.o.sb + head * p.o.sh + tok0 * p.o.st;
  const int64_t n_qt = (L + kBlockQ - 1) / kBlockQ;
  float* carry = p.carry ? p.carry + (int64_t)head * p.carry_head_stride + tile.carry_base : nullptr;

  for (int r = 0; r < kF32RowsPerWave; r++) {
    const int i = row_base + r;
    if (i >= L) break;                                       // wave-uniform
    for (int d = lane; d < D; d += 64) q_lds[wave][d] = qb[(int64_t)i * p.q.st + d];
    const int last_key = i - 1 + ac;
    float prod = 1.f, o0 = 0.f, o1 = 0.f;                      // this lane's output columns: lane, lane + 64
    // The backward reads the product above every 64-key step the row's 128-row tile sweeps, visible or not.
    const int tile_last_key = min(tile.origin + kBlockQ, L) - 2 + ac;
    const int n_steps_tile = tile_last_key < 0 ? 0 : tile_last_key / kF32Keys + 1;
    for (int c = n_steps_tile - 1; c >= 0; --c) {
      const int j0 = c * kF32Keys;
      if (carry && lane == 0) carry[carry_offset(2 * c + 1, n_qt) + (i - kBlockQ * (c >> 1))] = prod;
      if (j0 > last_key) continue;
      const int j = j0 + lane;
      const bool vis = j <= last_key;
      const float x = dot_row(q_lds[wave], vis ? kb + (int64_t)j * p.k.st : nullptr, D) * p.scale_log2;
      const float e = vis ? exp2f(fminf(x, 100.f)) : 0.f;
      const float omb = 1.f / (1.f + e);
      const float w = scan_down_mul(omb, lane);               // product over this step's keys >= j
      const float a = e * (w * prod);
      prod *= wave_bcast(w, 0);
      const int nk = min(kF32Keys, last_key - j0 + 1);
      for (int t = 0; t < nk; t++) {
        const float at = wave_bcast(a, t);
        const float* vrow = vb + (int64_t)(j0 + t) * p.v.st;
        if (lane < D) o0 = fmaf(at, vrow[lane], o0);
        if (lane + 64 < D) o1 = fmaf(at, vrow[lane + 64], o1);
      }
    }
    if (p.add_rem) {                                         // o + rem * v
      if (lane < D) o0 = fmaf(prod, vb[(int64_t)i * p.v.st + lane], o0);
      if (lane + 64 < D) o1 = fmaf(prod, vb[(int64_t)i * p.v.st + lane + 64], o1);
    }
    if (lane < D) ob[(int64_t)i * p.o.st + lane] = o0;
    if (lane + 64 < D) ob[(int64_t)i * p.o.st + lane + 64] = o1;
    if (lane == 0) {
      ((float*)p.rem.ptr)[tile.seq_id * p.rem.sb + head * p.rem.sh + (tok0 + i) * p.rem.st] = prod;
      p.row_stat[tile.seq_id * p.stat_sb + head * p.stat_sh + tok0 + i] = log2f(prod);
    }
  }
}

__global__ void fill_zero_rows_kernel(TensorRef t, int batches, int heads, int64_t tokens, int D) {
  const int64_t n = (int64_t)batches * heads * tokens * D;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += (int64_t)gridDim.x * blockDim.x) {
    const int d = (int)(idx % D);
    const int64_t tk = (idx / D) % tokens;
    const int h = (int)((idx / D / tokens) % heads);
    const int b = (int)(idx / D / tokens / heads);
    ((float*)t.ptr)[b * t.sb + h * t.sh + tk * t.st + d] = 0.f;
  }
}

struct BwdF32Lds {
  float q[kWaves][kMaxD];
  float d_o[kWaves][kMaxD];
  float dk[kF32Keys][kMaxD];
  float dv[kF32Keys][kMaxD];
  float dq[kF32Rows][kMaxD];
};

__global__ __launch_bounds__(kThreads) void bwd_f32_kernel(BwdParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  BwdF32Lds& lds = *reinterpret_cast<BwdF32Lds*>(lds_raw);
  int head, slot;
  xcd_head_tile(blockIdx.x / kF32Split, p.num_heads, &head, &slot);
  if (slot >= p.counts[kCountQ]) return;
  const Tile tile = p.q_tiles[slot];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wg_row0 = tile.origin + (blockIdx.x % kF32Split) * kF32Rows;      // first row of this workgroup
  const int L = tile.seq_len, ac = p.attend_current, D = p.head_dim;
  const int64_t tok0 = tile.seq_start;
  const float* qb = (const float*)p.q.ptr + tile.seq_id * p.q.sb + head * p.q.sh + tok0 * p.q.st;
  const float* kb = (const float*)p.k.ptr + tile.seq_id * p.k.sb + head * p.k.sh + tok0 * p.k.st;
  const float* vb = (const float*)p.v.ptr + tile.seq_id * p.v.sb + head * p.v.sh + tok0 * p.v.st;
  const float* dob = (const float*)p.d_o.ptr + tile.seq_id * p.d_o.sb + head * p.d_o.sh + tok0 * p.d_o.st;
  float* dqb = (float*)p.dq.ptr + tile.seq_id * p.dq.sb + head * p.dq.sh + tok0 * p.dq.st;
  float* dkb = (float*)p.dk.ptr + tile.seq_id * p.dk.sb + head * p.dk.sh + tok0 * p.dk.st;
  float* dvb = (float*)p.dv.ptr + tile.seq_id * p.dv.sb + head * p.dv.sh + tok0 * p.dv.st;
  const int64_t n_qt = (L + kBlockQ - 1) / kBlockQ;
  const float* carry = p.carry + (int64_t)head * p.carry_head_stride + tile.carry_base;

  const int wg_last_key = min(wg_row0 + kF32Rows, L) - 2 + ac;
  const int n_steps = (wg_last_key < 0 || wg_row0 >= L) ? 0 : wg_last_key / kF32Keys + 1;
  for (int idx = threadIdx.x; idx < kF32Rows * kMaxD; idx += kThreads) (&lds.dq[0][0])[idx] = 0.f;
  float prefix_row = 0.f;      // lane r (< rows per wave) holds the running prefix sum C of this wave's row r
  if (p.add_rem) {
    // The forward wrote o + rem * v: dv_i gains rem_i * d_o_i, for every row including those that see no key.
    for (int r = 0; r < kF32RowsPerWave; r++) {
      const int i = wg_row0 + wave * kF32RowsPerWave + r;
      if (i >= L) break;
      const float rem_i = exp2f(p.row_stat[tile.seq_id * p.stat_sb + head * p.stat_sh + tok0 + i]);
      for (int d = lane; d < D; d += 64) atomicAdd(&dvb[(int64_t)i * p.dv.st + d], rem_i * dob[(int64_t)i * p.d_o.st + d]);
    }
  }

  for (int c = 0; c < n_steps; ++c) {
    const int j0 = c * kF32Keys;
    for (int idx = threadIdx.x; idx < kF32Keys * kMaxD; idx += kThreads) { (&lds.dk[0][0])[idx] = 0.f; (&lds.dv[0][0])[idx] = 0.f; }
    __syncthreads();
    for (int r = 0; r < kF32RowsPerWave; r++) {
      const int i = wg_row0 + wave * kF32RowsPerWave + r;
      const int last_key = i - 1 + ac;
      if (i >= L || j0 > last_key) continue;                  // wave-uniform
      for (int d = lane; d < D; d += 64) {
        lds.q[wave][d] = qb[(int64_t)i * p.q.st + d];
        lds.d_o[wave][d] = dob[(int64_t)i * p.d_o.st + d];
      }
      float drem = p.d_rem.ptr ? ((const float*)p.d_rem.ptr)[tile.seq_id * p.d_rem.sb + head * p.d_rem.sh + (tok0 + i) * p.d_rem.st] : 0.f;
      if (p.add_rem) {
        // The forward wrote o + rem * v: the gradient reaching rem gains d_o . v_i.
        const float* vrow = vb + (int64_t)i * p.v.st;
        float dot = 0.f;
        for (int d = lane; d < D; d += 64) dot = fmaf(lds.d_o[wave][d], vrow[d], dot);
        for (int m = 32; m >= 1; m >>= 1) dot += __shfl_xor(dot, m);
        drem += dot;
      }
      const float prod_in = carry[carry_offset(2 * c + 1, n_qt) + (i - kBlockQ * (c >> 1))];
      const float prefix_in = wave_bcast(prefix_row, r);
      const int j = j0 + lane;
      const bool vis = j <= last_key;
      const float x = dot_row(lds.q[wave], vis ? kb + (int64_t)j * p.k.st : nullptr, D) * p.scale_log2;
      const float dpv = dot_row(lds.d_o[wave], vis ? vb + (int64_t)j * p.v.st : nullptr, D);
      const float e = vis ? exp2f(fminf(x, 100.f)) : 0.f;
      const float omb = 1.f / (1.f + e);
      const float beta = e * omb;
      const float w = scan_down_mul(omb, lane);
      const float a = e * (w * prod_in);                      // A_ij
      const float g = a * (dpv - drem);
      const float cum = scan_up_add(g, lane);
      const float dz = vis ? g - beta * (prefix_in + cum) : 0.f;
      const float tot = wave_bcast(cum, 63);
      if (lane == r) prefix_row = prefix_in + tot;
      const int nk = min(kF32Keys, last_key - j0 + 1);
      float dq0 = 0.f, dq1 = 0.f;
      for (int t = 0; t < nk; t++) {
        const float dzt = wave_bcast(dz, t), at = wave_bcast(a, t);
        const float* krow = kb + (int64_t)(j0 + t) * p.k.st;
        if (lane < D) {
          dq0 = fmaf(dzt, krow[lane], dq0);
          atomicAdd(&lds.dk[t][lane], dzt * lds.q[wave][lane]);
          atomicAdd(&lds.dv[t][lane], at * lds.d_o[wave][lane]);
        }
        if (lane + 64 < D) {
          dq1 = fmaf(dzt, krow[lane + 64], dq1);
          atomicAdd(&lds.dk[t][lane + 64], dzt * lds.q[wave][lane + 64]);
          atomicAdd(&lds.dv[t][lane + 64], at * lds.d_o[wave][lane + 64]);
        }
      }
      lds.dq[wave * kF32RowsPerWave + r][lane] += dq0;        // this wave is the only writer of its rows
      lds.dq[wave * kF32RowsPerWave + r][lane + 64] += dq1;
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < kF32Keys * D; idx += kThreads) {
      const int t = idx / D, d = idx % D, j = j0 + t;
      if (j < L) {
        atomicAdd(&dkb[(int64_t)j * p.dk.st + d], lds.dk[t][d] * p.logit_scale);
        atomicAdd(&dvb[(int64_t)j * p.dv.st + d], lds.dv[t][d]);
      }
    }
    __syncthreads();
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < kF32Rows * D; idx += kThreads) {
    const int r = idx / D, d = idx % D, i = wg_row0 + r;
    if (i < L) dqb[(int64_t)i * p.dq.st + d] = lds.dq[r][d] * p.logit_scale;
  }
}

hipError_t launch_fwd_f32(const FwdParams& p, int max_tiles, hipStream_t stream) {
  hipLaunchKernelGGL(fwd_f32_kernel, dim3((unsigned)(max_tiles * p.num_heads * kF32Split)), dim3(kThreads), 0, stream, p);
  return hipGetLastError();
}

hipError_t launch_bwd_f32(const BwdParams& p, int batches, int64_t tokens, int max_q_tiles, hipStream_t stream) {
  hipLaunchKernelGGL(fill_zero_rows_kernel, dim3(1024), dim3(256), 0, stream, p.dk, batches, p.num_heads, tokens, p.head_dim);
  hipLaunchKernelGGL(fill_zero_rows_kernel, dim3(1024), dim3(256), 0, stream, p.dv, batches, p.num_heads, tokens, p.head_dim);
  // dq is stored, not accumulated, but only for rows that belong to a sequence: the fill covers the others.
  hipLaunchKernelGGL(fill_zero_rows_kernel, dim3(1024), dim3(256), 0, stream, p.dq, batches, p.num_heads, tokens, p.head_dim);
  if (hipGetLastError() != hipSuccess) return hipErrorLaunchFailure;
  static std::atomic<uint64_t> lds_done{0};
  int dev = 0, cus = 0;
  hipError_t e = device_cus(&dev, &cus);
  if (e != hipSuccess) return e;
  if ((e = raise_lds_limit(&bwd_f32_kernel, lds_done, dev, sizeof(BwdF32Lds))) != hipSuccess) return e;
  hipLaunchKernelGGL(bwd_f32_kernel, dim3((unsigned)(max_q_tiles * p.num_heads * kF32Split)), dim3(kThreads), sizeof(BwdF32Lds), stream, p);
  return hipGetLastError();
}

}  // namespace sba
