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
#include "sba_host.hpp"
#include "sba_params.hpp"

#include <atomic>
#include <type_traits>

namespace sba {

template <int DH> struct DkvLds {
  static constexpr int kRowStride = lds_stride<DH>();
  static constexpr int kPStride = lds_stride<kBlockK>();
  static constexpr int kQ = 0;
  static constexpr int kDo = kQ + kBlockQ * kRowStride;
  static constexpr int kP = kDo + kBlockQ * kRowStride;
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

  // This tile's K and V as MFMA A operands, stationary in registers: row tile mt, lane row l%32 -> key
  // mfma_row_to_key(mt, l%32), 8 head_dim elements per k-step.  Keys beyond the sequence read as zero.
  vec8 kf[2][kSteps], vf[2][kSteps];
#pragma unroll
  for (int mt = 0; mt < 2; mt++) {
    const int key = j0 + mfma_row_to_key(mt, col);
#pragma unroll
    for (int kk = 0; kk < kSteps; kk++) {
      kf[mt][kk] = as_vec8<T>(load_row8<T, kFast>(kb + (int64_t)key * p.k.st, 16 * kk + 8 * half, D, key < L));
      vf[mt][kk] = as_vec8<T>(load_row8<T, kFast>(vb + (int64_t)key * p.v.st, 16 * kk + 8 * half, D, key < L));
    }
  }

  const int first_row = j0 + 1 - ac;                                  // first row that sees key j0
  const int n_qt = (L + kBlockQ - 1) / kBlockQ;
  const int qt_begin = first_row < L ? first_row / kBlockQ : n_qt;    // == jt / 2 whenever any row sees the tile
  // product above the tile = above its upper 32-key sub-tile; prefix below the tile = below its lower sub-tile
  const int64_t seq0 = (int64_t)head * p.carry_head_stride + tile.carry_base - (int64_t)kBlockQ * (jt >> 1);
  const float* carry = p.carry + seq0 + carry_offset(2 * jt + 1, n_qt);      // + row
  const float* prefix = p.prefix + seq0 + carry_offset(2 * jt, n_qt);

  const RowSource<T> qsrc = make_row_source<T, kFast>(qb, p.q.st, L, D), dosrc = make_row_source<T, kFast>(dob, p.d_o.st, L, D);
  TileCopy<T, DH, kBlockQ, kFast> cq, cdo;
  if (qt_begin < n_qt) {
    cq.load(qsrc, qt_begin * kBlockQ);
    cdo.load(dosrc, qt_begin * kBlockQ);
  }
  for (int qt = qt_begin; qt < n_qt; ++qt) {
    const int q0 = qt * kBlockQ;
    __syncthreads();      // previous contraction finished reading the q/do/p/dz tiles
    cq.store(q_lds);
    cdo.store(do_lds);
    __syncthreads();
    if (qt + 1 < n_qt) {  // prefetch the next query tile while this one is processed
      const int qn = q0 + kBlockQ;
      cq.load(qsrc, qn);
      cdo.load(dosrc, qn);
    }

    const int w_first = q0 + wave * 32, w_last = w_first + 31;
    const int qi = w_first + col;
    const bool row_ok = qi < L;
    uint32_t pk[16], dzk[16];
    if (j0 > min(w_last, L - 1) - 1 + ac) {
      // no row of this wave that belongs to the sequence sees the tile: contributes zeros
#pragma unroll
      for (int i = 0; i < 16; i++) { pk[i] = 0; dzk[i] = 0; }
    } else {
      const bool diagonal = (j0 + kBlockK - 1) > (w_first - 1 + ac) || w_last >= L;
      // gradient of rem per row, as the dQ kernel left it (d_rem, plus d_o . v when the remainder term is fused)
      const float drem = row_ok ? p.drem_eff[tile.seq_id * p.drem_sb + head * p.stat_sh + tok0 + qi] : 0.f;
      const float prod_in = carry[qi], prefix_in = prefix[qi];
      f32x16 s[2], dp[2];
#pragma unroll
      for (int mt = 0; mt < 2; mt++) {
#pragma unroll
        for (int r = 0; r < 16; r++) { s[mt][r] = 0.f; dp[mt][r] = 0.f; }
#pragma unroll
        for (int kk = 0; kk < kSteps; kk++) {
          vec8 b = lds_row8<T>(q_lds, kRowStride, wave * 32 + col, 16 * kk + 8 * half);
          s[mt] = Elem<T>::mfma(kf[mt][kk], b, s[mt]);
        }
#pragma unroll
        for (int kk = 0; kk < kSteps; kk++) {
          vec8 b = lds_row8<T>(do_lds, kRowStride, wave * 32 + col, 16 * kk + 8 * half);
          dp[mt] = Elem<T>::mfma(vf[mt][kk], b, dp[mt]);
        }
      }
      const int lim = row_ok ? qi + ac - j0 - 32 * half : 0;
      float prod_lower, prefix_upper, prefix_next;
      bwd_tile_math<T, 2>(s, dp, p.scale_log2, diagonal, lim, half, drem, prod_in, prefix_in, pk, dzk, prod_lower,
                          prefix_upper, prefix_next);
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
        float dvv = dvacc[b][r];
        if (p.add_rem)     // the remainder term o += rem * v contributes rem_j * d_o_j to dv_j
          dvv += fast_exp2(p.row_stat[tile.seq_id * p.stat_sb + head * p.stat_sh + tok0 + key]) * (float)dob[(int64_t)key * p.d_o.st + d];
        dvb[(int64_t)key * p.dv.st + d] = (T)dvv;
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------------------
// Fast path, producer / consumer waves (runs head_dim 64; head_dim 128 runs the software-pipelined kernel below).
//
// One workgroup = 8 waves = one 64-key tile, swept by query tiles of 64 rows.  Waves 0-3 are PRODUCERS: wave
// (rg, g) takes rows 32*rg .. +31 against the 32-key sub-tile g (one MFMA row tile, 16 keys per lane, that
// sub-tile's K/V operands stationary in registers), recomputes P^T and dZ^T and writes them to LDS.  Waves 4-7
// are CONSUMERS: they stage the query tiles (Q, dO) into LDS and, one step behind, wave cw contracts P^T/dZ^T
// with dO/Q over the 64 rows into the 64-key x 32-column block cw of dV and dK.  Every SIMD hosts one producer (exp/rcp/VALU bound) and one consumer
// (MFMA/LDS bound), so the two pipelines overlap, and there is ONE barrier per step: P/dZ are double-buffered
// and Q/dO triple-buffered (written for step t+1, read by producers for step t and by consumers for step t-1).
// The per-(row, sub-tile) carries are what the forward and the dQ kernel recorded at 32-key granularity.
constexpr int kDkvRows = 64;      // query rows per step
constexpr int kDkv3Threads = 512;
template <int DH> struct Dkv3Lds {
  static constexpr int kRowStride = lds_stride<DH>();
  static constexpr int kPStride = lds_stride<kBlockK>();
  static constexpr int kQdoTile = kDkvRows * kRowStride;     // one Q (or dO) tile
  static constexpr int kPTile = kDkvRows * kPStride;         // one P (or dZ) tile
  static constexpr int kQ = 0;                               // 3 buffers of {Q, dO}
  static constexpr int kP = 6 * kQdoTile;                    // 2 buffers of {P, dZ}
  static constexpr int kElems = kP + 4 * kPTile;
};

template <typename T, int DH>
__global__ __launch_bounds__(kDkv3Threads) void bwd_dkv3_kernel(BwdParams p) {
  typedef typename Elem<T>::vec8 vec8;
  typedef Dkv3Lds<DH> Lds;
  constexpr int kRowStride = Lds::kRowStride, kPStride = Lds::kPStride;
  constexpr int kSteps = DH / 16;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  T* lds = reinterpret_cast<T*>(lds_raw);

  // Persistent workgroups: LDS allows one workgroup per CU, so a workgroup per key tile would leave every tile's
  // start-up (tile record, K/V operands, first query tiles) and its final stores exposed.  Each workgroup walks
  // the tile list with the grid's stride instead; the producers run ahead into the next tile's start-up while the
  // consumers store the previous tile's results.  The walk keeps the workgroup on one head (and one XCD).
  const int n_tiles = p.counts[1];
  const int lane = threadIdx.x & 63, wave = (threadIdx.x >> 6) & 3;
  const bool producer = threadIdx.x < 256;
  const int half = lane >> 5, col = lane & 31;
  const int ac = p.attend_current;
  // The `wph` workgroups of a head start with the head's first wph tiles (the list is heaviest first) and then take
  // the next tile from a per-head cursor whenever they finish one, so the load balances itself.  The cursor is read
  // a tile ahead: thread 0 takes the slot after next before a tile's start-up barrier and publishes it through LDS.
  const int wph = p.wgs_per_head;
  int head, w;
  if ((p.num_heads & 7) == 0) {
    const int hpx = p.num_heads >> 3, r0 = blockIdx.x >> 3;
    head = (blockIdx.x & 7) * hpx + r0 % hpx;
    w = r0 / hpx;
  } else {
    head = blockIdx.x % p.num_heads;
    w = blockIdx.x / p.num_heads;
  }
  int* next_slot_lds = reinterpret_cast<int*>(lds_raw + (size_t)Lds::kElems * sizeof(T));
  auto first_row_block = [&](const Tile& tl) {               // first 64-row step that sees the tile's first key
    const int first_row = tl.origin + 1 - ac;
    return first_row < tl.seq_len ? (first_row / kDkvRows) * kDkvRows : tl.seq_len;
  };
  // The tile record of the next round is fetched a round ahead; the consumers also request the first query rows
  // of the next tile before they store the results of the current one.
  Tile next_tile = p.k_tiles[w < n_tiles ? w : 0];
  TileCopy<T, DH, kDkvRows, true> cq, cdo;                   // staging registers (consumer waves)
  auto stage_first = [&](const Tile& tl) {
    const T* qb = (const T*)p.q.ptr + tl.seq_id * p.q.sb + head * p.q.sh + (int64_t)tl.seq_start * p.q.st;
    const T* dob = (const T*)p.d_o.ptr + tl.seq_id * p.d_o.sb + head * p.d_o.sh + (int64_t)tl.seq_start * p.d_o.st;
    const int rb = first_row_block(tl);
    if (rb < tl.seq_len) {
      cq.load(make_row_source<T, true>(qb, p.q.st, tl.seq_len, DH), rb);
      cdo.load(make_row_source<T, true>(dob, p.d_o.st, tl.seq_len, DH), rb);
    }
  };
  // Producer waves: the K and V operands of the next tile's 32-key sub-tile are requested a tile ahead as well.
  vec8 kf_next[kSteps], vf_next[kSteps];
  auto load_kv = [&](const Tile& tl) {
    const T* kb = (const T*)p.k.ptr + tl.seq_id * p.k.sb + head * p.k.sh + (int64_t)tl.seq_start * p.k.st;
    const T* vb = (const T*)p.v.ptr + tl.seq_id * p.v.sb + head * p.v.sh + (int64_t)tl.seq_start * p.v.st;
    const int key = tl.origin + 32 * (wave & 1) + mfma_row_to_key32(col);
    const RowSource<T> ks = make_row_source<T, true>(kb, p.k.st, tl.seq_len, DH), vs = make_row_source<T, true>(vb, p.v.st, tl.seq_len, DH);
#pragma unroll
    for (int kk = 0; kk < kSteps; kk++) {       // keys beyond the sequence are outside the buffer and read as zero
      kf_next[kk] = as_vec8<T>(__builtin_amdgcn_raw_buffer_load_b128(ks.rsrc, key * ks.stride_bytes + (16 * kk + 8 * half) * (int)sizeof(T), 0, 0));
      vf_next[kk] = as_vec8<T>(__builtin_amdgcn_raw_buffer_load_b128(vs.rsrc, key * vs.stride_bytes + (16 * kk + 8 * half) * (int)sizeof(T), 0, 0));
    }
  };
  // Each role runs its own walk over the same rounds (same tiles, same number of barriers), so that what one role
  // carries from tile to tile does not occupy registers in the other role's code.
  if (producer) {
    if (w < n_tiles) load_kv(next_tile);
  for (int slot = w; slot < n_tiles;) {
  const Tile tile = next_tile;
  if (threadIdx.x == 0) *next_slot_lds = wph + atomicAdd(p.head_queue + head, 1);
  const int L = tile.seq_len, j0 = tile.origin, ac = p.attend_current;
  const int64_t tok0 = tile.seq_start;
  const int jt = j0 / kBlockK;

  const int first_row = j0 + 1 - ac;                         // first row that sees key j0
  const int n_qt = (L + kBlockQ - 1) / kBlockQ;
  const int row_begin = first_row < L ? (first_row / kDkvRows) * kDkvRows : L;
  const int n_steps = (L - row_begin + kDkvRows - 1) / kDkvRows;

    const int rg = wave >> 1, group = wave & 1;
    const int jb = j0 + 32 * group;          // first key of this wave's sub-tile
    [[maybe_unused]] const T* qb = (const T*)p.q.ptr + tile.seq_id * p.q.sb + head * p.q.sh + tok0 * p.q.st;
    [[maybe_unused]] const T* kb = (const T*)p.k.ptr + tile.seq_id * p.k.sb + head * p.k.sh + tok0 * p.k.st;
    [[maybe_unused]] const T* vb = (const T*)p.v.ptr + tile.seq_id * p.v.sb + head * p.v.sh + tok0 * p.v.st;
    [[maybe_unused]] const T* dob = (const T*)p.d_o.ptr + tile.seq_id * p.d_o.sb + head * p.d_o.sh + tok0 * p.d_o.st;
    const int64_t slot0 = (int64_t)head * p.carry_head_stride + tile.carry_base +
                          carry_offset(2 * jt + group, n_qt) - (int64_t)kBlockQ * (jt >> 1);      // + row
    const float* carry = p.carry + slot0;
    const float* prefix = p.prefix + slot0;

    // This sub-tile's K and V as MFMA A operands, stationary in registers (keys beyond the sequence read as zero).
    vec8 kf[kSteps], vf[kSteps];
#pragma unroll
    for (int kk = 0; kk < kSteps; kk++) { kf[kk] = kf_next[kk]; vf[kk] = vf_next[kk]; }
    // Per-row scalars (drem, product above the sub-tile, C below it), fetched one step ahead.
    const float* drem_eff = p.drem_eff + tile.seq_id * p.drem_sb + head * p.stat_sh + tok0;
    float n_drem = 0.f, n_prod = 1.f, n_prefix = 0.f;
    auto fetch_row_scalars = [&](int row0) {
      const int r = row0 + rg * 32 + col;
      n_drem = r < L ? drem_eff[r] : 0.f;      // as the dQ kernel left it: d_rem (+ d_o . v with the remainder term)
      n_prod = carry[r];
      n_prefix = prefix[r];
    };
    if (n_steps > 0) fetch_row_scalars(row_begin);
    __syncthreads();
    slot = *next_slot_lds;                                   // the tile after this one
    const bool have_next = slot < n_tiles;
    if (have_next) {
      next_tile = p.k_tiles[slot];
      load_kv(next_tile);
    }
    for (int t = 0; t <= n_steps; ++t) {
      if (t < n_steps) {
        const int q0 = row_begin + t * kDkvRows;
        const T* q_lds = lds + Lds::kQ + (t % 3) * 2 * Lds::kQdoTile;
        const T* do_lds = q_lds + Lds::kQdoTile;
        T* p_lds = lds + Lds::kP + (t & 1) * 2 * Lds::kPTile;
        T* dz_lds = p_lds + Lds::kPTile;
        const float drem = n_drem, prod_in = n_prod, prefix_in = n_prefix;
        if (t + 1 < n_steps) fetch_row_scalars(q0 + kDkvRows);
        const int w_first = q0 + rg * 32, w_last = w_first + 31;
        const int qi = w_first + col;
        const bool row_ok = qi < L;
        uint32_t pk[8], dzk[8];
        // Skipped unless a row of the SEQUENCE sees the sub-tile: the forward and the dQ kernel record the per-row
        // scalars only for sub-tiles that hold a key visible to the last row of their query tile, so a sub-tile that
        // merely lies below rows beyond the sequence's end has no recorded values to start from.
        if (jb > min(w_last, L - 1) - 1 + ac) {
#pragma unroll
          for (int i = 0; i < 8; i++) { pk[i] = 0; dzk[i] = 0; }
        } else {
          const bool diagonal = (jb + 31) > (w_first - 1 + ac) || w_last >= L;
          f32x16 s[1], dp[1];
#pragma unroll
          for (int r = 0; r < 16; r++) { s[0][r] = 0.f; dp[0][r] = 0.f; }
          // The B operands are requested in two batches of eight, each before its MFMAs: the consumers keep the LDS
          // queue long, and a read-two / wait / multiply-two schedule pays that queueing latency eight times over.
          {
            vec8 bq[kSteps];
#pragma unroll
            for (int kk = 0; kk < kSteps; kk++) bq[kk] = lds_row8<T>(q_lds, kRowStride, rg * 32 + col, 16 * kk + 8 * half);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int kk = 0; kk < kSteps; kk++) s[0] = Elem<T>::mfma(kf[kk], bq[kk], s[0]);
          }
          __builtin_amdgcn_sched_barrier(0);
          {
            vec8 bdo[kSteps];
#pragma unroll
            for (int kk = 0; kk < kSteps; kk++) bdo[kk] = lds_row8<T>(do_lds, kRowStride, rg * 32 + col, 16 * kk + 8 * half);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int kk = 0; kk < kSteps; kk++) dp[0] = Elem<T>::mfma(vf[kk], bdo[kk], dp[0]);
          }
          const int lim = row_ok ? qi + ac - jb - 16 * half : 0;
          float prod_lower, prefix_upper, prefix_next;
          bwd_tile_math<T, 1>(s, dp, p.scale_log2, diagonal, lim, half, drem, prod_in, prefix_in, pk, dzk, prod_lower,
                              prefix_upper, prefix_next);
        }
        // [query][key] tiles: this lane's 16 consecutive keys start at column 32*group + 16*half of row 32*rg + col.
        u32x4* pp = reinterpret_cast<u32x4*>(p_lds + (rg * 32 + col) * kPStride + 32 * group + 16 * half);
        u32x4* dd = reinterpret_cast<u32x4*>(dz_lds + (rg * 32 + col) * kPStride + 32 * group + 16 * half);
#pragma unroll
        for (int c = 0; c < 2; c++) {
          pp[c] = u32x4{pk[4 * c], pk[4 * c + 1], pk[4 * c + 2], pk[4 * c + 3]};
          dd[c] = u32x4{dzk[4 * c], dzk[4 * c + 1], dzk[4 * c + 2], dzk[4 * c + 3]};
        }
      }
      __syncthreads();
    }
    }  // rounds of the tile walk (producers)
  } else {
    if (w < n_tiles) stage_first(next_tile);
    // Output blocks of this consumer wave.  head_dim 128: both 32-key row tiles x columns 32*wave .. +31;
    // head_dim 64: row tile wave/2 x columns 32*(wave%2) .. +31.
    constexpr int kMT = DH == 128 ? 2 : 1;
    const int mt0 = DH == 128 ? 0 : wave >> 1, ct = DH == 128 ? wave : wave & 1;
    f32x16 dkacc[kMT], dvacc[kMT];
    // The results of a tile are stored during the first step of the NEXT tile, when the consumers have nothing to
    // contract yet (and after the last tile): acc[mt][r] is key origin + 32*(mt0 + mt) + 8*(r/4) + 4*half + r%4,
    // column 32*ct + col.
    bool pending = false;
    Tile done_tile = next_tile;
    auto store_results = [&](const Tile& tl) {
      const int tl_len = tl.seq_len, tl_j0 = tl.origin;
      const int64_t tl_tok0 = tl.seq_start;
      T* dkb = (T*)p.dk.ptr + tl.seq_id * p.dk.sb + head * p.dk.sh + tl_tok0 * p.dk.st;
      T* dvb = (T*)p.dv.ptr + tl.seq_id * p.dv.sb + head * p.dv.sh + tl_tok0 * p.dv.st;
      if (p.add_rem) {
        // the remainder term o += rem * v contributes rem_j * d_o_j to dv_j
        const T* dob = (const T*)p.d_o.ptr + tl.seq_id * p.d_o.sb + head * p.d_o.sh + tl_tok0 * p.d_o.st;
        const int d = 32 * ct + col;
#pragma unroll
        for (int mt = 0; mt < kMT; mt++)
#pragma unroll
          for (int r = 0; r < 16; r++) {
            const int key = tl_j0 + 32 * (mt0 + mt) + 8 * (r >> 2) + 4 * half + (r & 3);
            if (key < tl_len)
              dvacc[mt][r] += fast_exp2(p.row_stat[tl.seq_id * p.stat_sb + head * p.stat_sh + tl_tok0 + key]) *
                              (float)dob[(int64_t)key * p.d_o.st + d];
          }
      }
      const RowSink<T> dk_sink = make_row_sink<T>(dkb, p.dk.st, tl_len, DH), dv_sink = make_row_sink<T>(dvb, p.dv.st, tl_len, DH);
      // Wave-private transposition scratch in the third Q/dO buffer: free during a tile's first step and after the
      // last one.
      T* scratch = lds + Lds::kQ + 4 * Lds::kQdoTile + wave * (32 * lds_stride<32>());
#pragma unroll
      for (int mt = 0; mt < kMT; mt++) {
        store_acc_tile_wide<T>(dk_sink, dkacc[mt], p.logit_scale, tl_j0 + 32 * (mt0 + mt), 32 * ct, half, col, lane, scratch);
        store_acc_tile_wide<T>(dv_sink, dvacc[mt], 1.f, tl_j0 + 32 * (mt0 + mt), 32 * ct, half, col, lane, scratch);
      }
    };
  for (int slot = w; slot < n_tiles;) {
  const Tile tile = next_tile;
  const int L = tile.seq_len, j0 = tile.origin, ac = p.attend_current, D = DH;
  const int64_t tok0 = tile.seq_start;

  const int first_row = j0 + 1 - ac;                         // first row that sees key j0
  const int row_begin = first_row < L ? (first_row / kDkvRows) * kDkvRows : L;
  const int n_steps = (L - row_begin + kDkvRows - 1) / kDkvRows;

    // The consumers also move the query tiles global -> registers -> LDS (they have the issue slots to spare):
    // tile t+1 is written at the top of step t from registers loaded during step t-1, then tile t+2 is requested;
    // the barrier that ends a step is the only point that waits for those loads.
    [[maybe_unused]] const T* qb = (const T*)p.q.ptr + tile.seq_id * p.q.sb + head * p.q.sh + tok0 * p.q.st;
    [[maybe_unused]] const T* dob = (const T*)p.d_o.ptr + tile.seq_id * p.d_o.sb + head * p.d_o.sh + tok0 * p.d_o.st;
    const RowSource<T> qsrc = make_row_source<T, true>(qb, p.q.st, L, D), dosrc = make_row_source<T, true>(dob, p.d_o.st, L, D);
    if (n_steps > 0) {                                       // rows of step 0 were requested a tile ago
      cq.store(lds + Lds::kQ);
      cdo.store(lds + Lds::kQ + Lds::kQdoTile);
      if (n_steps > 1) {
        cq.load(qsrc, row_begin + kDkvRows);
        cdo.load(dosrc, row_begin + kDkvRows);
      }
    }
    __syncthreads();
    slot = *next_slot_lds;                                   // the tile after this one
    const bool have_next = slot < n_tiles;
    if (have_next) next_tile = p.k_tiles[slot];
    auto stage_step = [&](int t) {          // rows of step t+1 into LDS, rows of step t+2 requested
      if (t + 1 < n_steps) {
        T* nq_lds = lds + Lds::kQ + ((t + 1) % 3) * 2 * Lds::kQdoTile;
        cq.store(nq_lds);
        cdo.store(nq_lds + Lds::kQdoTile);
        if (t + 2 < n_steps) {
          const int qn = row_begin + (t + 2) * kDkvRows;
          cq.load(qsrc, qn);
          cdo.load(dosrc, qn);
        }
      }
    };
    // Step 0: nothing to contract yet, so the previous tile's results leave now.
    stage_step(0);
    if (pending) store_results(done_tile);
#pragma unroll
    for (int b = 0; b < kMT; b++)
#pragma unroll
      for (int r = 0; r < 16; r++) { dkacc[b][r] = 0.f; dvacc[b][r] = 0.f; }
    __syncthreads();
    for (int t = 1; t <= n_steps; ++t) {
      stage_step(t);
      {
        const int u = t - 1;
        const T* q_lds = lds + Lds::kQ + (u % 3) * 2 * Lds::kQdoTile;
        const T* do_lds = q_lds + Lds::kQdoTile;
        const T* p_lds = lds + Lds::kP + (u & 1) * 2 * Lds::kPTile;
        const T* dz_lds = p_lds + Lds::kPTile;
        // dV[key][d] += sum_i P[i][key] dO[i][d];  dK[key][d] += sum_i dZ[i][key] Q[i][d]   (i over the 64 rows)
#pragma unroll
        for (int c = 0; c < kDkvRows / 16; c++) {
          const int row0 = 16 * c + 8 * half;
          vec8 bd = lds_col8<T>(do_lds, kRowStride, row0, 32 * ct, lane);
          vec8 bq = lds_col8<T>(q_lds, kRowStride, row0, 32 * ct, lane);
#pragma unroll
          for (int mt = 0; mt < kMT; mt++) {
            vec8 ap = lds_col8<T>(p_lds, kPStride, row0, 32 * (mt0 + mt), lane);
            dvacc[mt] = Elem<T>::mfma(ap, bd, dvacc[mt]);
            vec8 az = lds_col8<T>(dz_lds, kPStride, row0, 32 * (mt0 + mt), lane);
            dkacc[mt] = Elem<T>::mfma(az, bq, dkacc[mt]);
          }
        }
      }
      __syncthreads();
    }
    if (have_next) stage_first(next_tile);
    pending = true;
    done_tile = tile;
      }  // rounds of the tile walk (consumers)
    if (pending) store_results(done_tile);
  }
}

template <typename T, int DH>
static hipError_t launch_dkv3(const BwdParams& p_in, int max_tiles, hipStream_t stream) {
  const size_t lds_bytes = (size_t)Dkv3Lds<DH>::kElems * sizeof(T) + 256;      // + the published queue slot
  // The tile set exceeds the default 64 KB dynamic-LDS cap: the limit is raised once per device.
  static std::atomic<uint64_t> lds_done{0};
  int dev = 0, cus = 0;
  hipError_t e = device_cus(&dev, &cus);
  if (e != hipSuccess) return e;
  if ((e = raise_lds_limit(&bwd_dkv3_kernel<T, DH>, lds_done, dev, lds_bytes)) != hipSuccess) return e;
  BwdParams p = p_in;
  // One workgroup per CU: the same number of workgroups for every head, and with a head count that is a multiple of
  // 8 the workgroups of a head share an XCD (workgroup ids are dealt round-robin to the 8 XCDs).
  p.wgs_per_head = cus / p.num_heads > 0 ? cus / p.num_heads : 1;
  if (p.wgs_per_head > max_tiles) p.wgs_per_head = max_tiles;
  const dim3 grid((unsigned)(p.wgs_per_head * p.num_heads)), block(kDkv3Threads);
  hipLaunchKernelGGL((bwd_dkv3_kernel<T, DH>), grid, block, lds_bytes, stream, p);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------------------
// Software-pipelined producer / consumer kernel: 128-key tiles swept by steps of 32 query rows.
//
// In the kernel above a producer wave's step is one serial chain -- wait for the B operands from LDS, 16 MFMAs,
// the element-wise math, the LDS writes, the barrier -- and with one producer per SIMD nothing else on that SIMD
// has vector-ALU work to fill the waits.  Here the producer issues the MFMAs of step t+1 (S^T and dP^T of the
// next 32 rows) inside the same straight-line block as the math of step t, so the matrix pipe runs under the
// vector ALU and the LDS latency is off the chain.  That needs the query rows in LDS one step earlier (4 stages
// of {Q, dO} instead of 3), which fits because a step is 32 rows; the tile is 128 keys so that a step still has
// one 32x32 block per producer wave.  Wave g of the producers owns the 32-key sub-tile g (K/V operands stationary
// in registers) and all four sweep the same rows; consumer wave (mp, cp) owns keys 64*mp..+63 x columns
// (DH/2)*cp..+DH/2-1 of dK and dV, which halves the LDS operand reads per MFMA of the narrower layout.
//
// Rows of step r (relative to the tile's first step): requested from global memory at step r-4, written to LDS
// stage r%4 at step r-2, read by the producers at step r-1 (MFMAs) and by the consumers at step r+1; P/dZ of
// step r are written at step r into buffer r%2 and contracted at step r+1.
constexpr int kDkv4Keys = 128;
constexpr int kDkv4Rows = 32;
constexpr int kDkv4Threads = 512;
template <int DH> struct Dkv4Lds {
  static constexpr int kRowStride = lds_stride<DH>();
  static constexpr int kPStride = lds_stride<kDkv4Keys>();
  static constexpr int kQdoTile = kDkv4Rows * kRowStride;    // one Q (or dO) tile
  static constexpr int kPTile = kDkv4Rows * kPStride;        // one P (or dZ) tile
  static constexpr int kQ = 0;                               // 4 stages of {Q, dO}
  static constexpr int kP = 8 * kQdoTile;                    // 2 buffers of {P, dZ}
  static constexpr int kScratch = kP + 4 * kPTile;           // one transposition scratch per consumer wave
  static constexpr int kElems = kScratch + 4 * 32 * lds_stride<32>();
};


template <typename T, int DH>
__global__ __launch_bounds__(kDkv4Threads) void bwd_dkv4_kernel(BwdParams p) {
  typedef typename Elem<T>::vec8 vec8;
  typedef Dkv4Lds<DH> Lds;
  constexpr int kRowStride = Lds::kRowStride, kPStride = Lds::kPStride;
  constexpr int kSteps = DH / 16;
  constexpr int kRows = kDkv4Rows;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  T* lds = reinterpret_cast<T*>(lds_raw);

  // Persistent workgroups, one per CU, each walking the key-tile list of one head (see the kernel above).
  const int n_tiles = p.counts[1];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane((threadIdx.x >> 6) & 3);
  const bool producer = threadIdx.x < 256;
  const int half = lane >> 5, col = lane & 31;
  const int ac = p.attend_current;
  const int wph = p.wgs_per_head;
  int head, w;
  if ((p.num_heads & 7) == 0) {
    const int hpx = p.num_heads >> 3, r0 = blockIdx.x >> 3;
    head = (blockIdx.x & 7) * hpx + r0 % hpx;
    w = r0 / hpx;
  } else {
    head = blockIdx.x % p.num_heads;
    w = blockIdx.x / p.num_heads;
  }
  int* next_slot_lds = reinterpret_cast<int*>(lds_raw + (size_t)Lds::kElems * sizeof(T));
  auto first_row_block = [&](const Tile& tl) {               // first 32-row step that sees the tile's first key
    const int first_row = tl.origin + 1 - ac;
    return first_row < tl.seq_len ? (first_row / kRows) * kRows : tl.seq_len;
  };
  Tile next_tile = p.k_tiles[w < n_tiles ? w : 0];

  if (producer) {
    const int g = wave;                                      // this wave's 32-key sub-tile of the tile
    // K and V of the sub-tile as MFMA A operands, stationary in registers.  The next tile's are requested into the
    // same registers as soon as the last MFMAs of this tile have been issued.
    vec8 kf[kSteps], vf[kSteps];
    auto load_kv = [&](const Tile& tl) {
      const T* kb = (const T*)p.k.ptr + tl.seq_id * p.k.sb + head * p.k.sh + (int64_t)tl.seq_start * p.k.st;
      const T* vb = (const T*)p.v.ptr + tl.seq_id * p.v.sb + head * p.v.sh + (int64_t)tl.seq_start * p.v.st;
      const int key = tl.origin + 32 * g + mfma_row_to_key32(col);
      const RowSource<T> ks = make_row_source<T, true>(kb, p.k.st, tl.seq_len, DH), vs = make_row_source<T, true>(vb, p.v.st, tl.seq_len, DH);
#pragma unroll
      for (int kk = 0; kk < kSteps; kk++) {       // keys beyond the sequence are outside the buffer and read as zero
        kf[kk] = as_vec8<T>(__builtin_amdgcn_raw_buffer_load_b128(ks.rsrc, key * ks.stride_bytes + (16 * kk + 8 * half) * (int)sizeof(T), 0, 0));
        vf[kk] = as_vec8<T>(__builtin_amdgcn_raw_buffer_load_b128(vs.rsrc, key * vs.stride_bytes + (16 * kk + 8 * half) * (int)sizeof(T), 0, 0));
      }
    };
    if (w < n_tiles) load_kv(next_tile);
    for (int slot = w; slot < n_tiles;) {
      const Tile tile = next_tile;
      if (threadIdx.x == 0) *next_slot_lds = wph + atomicAdd(p.head_queue + head, 1);
      const int L = tile.seq_len, j0 = tile.origin;
      const int64_t tok0 = tile.seq_start;
      const int jt = j0 / kDkv4Keys;
      const int first_row = j0 + 1 - ac;                     // first row that sees key j0
      const int n_qt = (L + kBlockQ - 1) / kBlockQ;
      const int row_begin = first_row < L ? (first_row / kRows) * kRows : L;
      const int n_steps = (L - row_begin + kRows - 1) / kRows;
      const int jb = j0 + 32 * g;                            // first key of this wave's sub-tile
      const int64_t slot0 = (int64_t)head * p.carry_head_stride + tile.carry_base +
                            carry_offset(4 * jt + g, n_qt) - (int64_t)kBlockQ * jt;      // + row
      const float* carry = p.carry + slot0;
      const float* prefix = p.prefix + slot0;
      const float* drem_eff = p.drem_eff + tile.seq_id * p.drem_sb + head * p.stat_sh + tok0;
      // Per-row scalars (drem, product above the sub-tile, C below it), fetched two steps ahead: a step is shorter
      // than a global load.
      float n_drem = 0.f, n_prod = 1.f, n_prefix = 0.f, nn_drem = 0.f, nn_prod = 1.f, nn_prefix = 0.f;
      auto fetch_row_scalars = [&](int row0, float& drem_r, float& prod_r, float& prefix_r) {
        const int r = row0 + col;
        drem_r = r < L ? drem_eff[r] : 0.f;
        prod_r = carry[r];
        prefix_r = prefix[r];
      };
      if (n_steps > 0) fetch_row_scalars(row_begin, n_drem, n_prod, n_prefix);
      if (n_steps > 1) fetch_row_scalars(row_begin + kRows, nn_drem, nn_prod, nn_prefix);
      lds_barrier();                                         // rows of steps 0 and 1 are in LDS; the queue slot too
      slot = *next_slot_lds;                                 // the tile after this one
      const bool have_next = slot < n_tiles;
      if (have_next) next_tile = p.k_tiles[slot];

      // S^T and dP^T of the rows in stage `st` against this wave's sub-tile.
      auto scores = [&](int st, f32x16& s, f32x16& dp) {
        const T* q_lds = lds + Lds::kQ + st * 2 * Lds::kQdoTile;
        const T* do_lds = q_lds + Lds::kQdoTile;
#pragma unroll
        for (int r = 0; r < 16; r++) { s[r] = 0.f; dp[r] = 0.f; }
        {
          vec8 bq[kSteps];
#pragma unroll
          for (int kk = 0; kk < kSteps; kk++) bq[kk] = lds_row8<T>(q_lds, kRowStride, col, 16 * kk + 8 * half);
#pragma unroll
          for (int kk = 0; kk < kSteps; kk++) s = Elem<T>::mfma(kf[kk], bq[kk], s);
        }
        {
          vec8 bdo[kSteps];
#pragma unroll
          for (int kk = 0; kk < kSteps; kk++) bdo[kk] = lds_row8<T>(do_lds, kRowStride, col, 16 * kk + 8 * half);
#pragma unroll
          for (int kk = 0; kk < kSteps; kk++) dp = Elem<T>::mfma(vf[kk], bdo[kk], dp);
        }
      };
      // The math of one step on (s_cur, dp_cur) with the MFMAs of the next step (rows in stage `st`, results in
      // s_next / dp_next) dealt among it, so that the matrix pipe runs under the vector ALU instead of stalling the
      // wave.  The block is one scheduling region whose issue order is spelled out at the end: the Q operands are
      // requested first and the first elements' math covers their latency, then one MFMA per kGap vector-ALU
      // instructions, with the dO operands requested a few MFMAs in.
      auto fused = [&](auto diag_tag, int st, const f32x16& s_cur, const f32x16& dp_cur, f32x16& s_next, f32x16& dp_next,
                       int lim, float drem, float prod_in, float prefix_in, uint32_t (&pk)[8], uint32_t (&dzk)[8]) {
        constexpr bool kDiag = decltype(diag_tag)::value;
        constexpr int kLead = 24;                              // vector-ALU instructions ahead of the first MFMA
        // Vector-ALU instructions per MFMA.  The group solver is greedy: with a budget a little below the block's
        // instruction count it puts the last MFMAs back to back and the rest of the math behind them, so the values
        // were checked in the generated code (both element types, both copies of the unrolled step).
        constexpr int kGap = (kDiag ? 270 : 240) / (2 * kSteps);
        constexpr int kAlu = 0x402;                            // scheduling-group mask: vector ALU incl. transcendentals
        const T* q_lds = lds + Lds::kQ + st * 2 * Lds::kQdoTile;
        const T* do_lds = q_lds + Lds::kQdoTile;
        __builtin_amdgcn_sched_barrier(0);
        vec8 bq[kSteps], bdo[kSteps];
#pragma unroll
        for (int kk = 0; kk < kSteps; kk++) bq[kk] = lds_row8<T>(q_lds, kRowStride, col, 16 * kk + 8 * half);
#pragma unroll
        for (int kk = 0; kk < kSteps; kk++) bdo[kk] = lds_row8<T>(do_lds, kRowStride, col, 16 * kk + 8 * half);
#pragma unroll
        for (int r = 0; r < 16; r++) { s_next[r] = 0.f; dp_next[r] = 0.f; }
#pragma unroll
        for (int kk = 0; kk < kSteps; kk++) s_next = Elem<T>::mfma(kf[kk], bq[kk], s_next);
#pragma unroll
        for (int kk = 0; kk < kSteps; kk++) dp_next = Elem<T>::mfma(vf[kk], bdo[kk], dp_next);
        f32x16 sc[1], dpc[1];
        sc[0] = s_cur; dpc[0] = dp_cur;
        float prod_lower, prefix_upper, prefix_next;
        bwd_tile_math_impl<T, 1, kDiag>(sc, dpc, p.scale_log2, lim, half, drem, prod_in, prefix_in, pk, dzk, prod_lower,
                                        prefix_upper, prefix_next);
        __builtin_amdgcn_sched_group_barrier(0x100, kSteps, 0);
        __builtin_amdgcn_sched_group_barrier(kAlu, kLead, 0);
#pragma unroll
        for (int i = 0; i < 2 * kSteps; i++) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(kAlu, kGap, 0);
          if (i == kSteps / 2 - 1) __builtin_amdgcn_sched_group_barrier(0x100, kSteps, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      };
      // One step: P^T / dZ^T of step t to LDS, S^T / dP^T of step t+1 into the other pair of accumulators.
      auto step = [&](int t, f32x16& s_cur, f32x16& dp_cur, f32x16& s_next, f32x16& dp_next) {
        if (t >= n_steps) {                                  // the consumers' last step: only the barrier of the step before
          if (t > 0) lds_barrier();
          return;
        }
        const int q0 = row_begin + t * kRows;
        const float drem = n_drem, prod_in = n_prod, prefix_in = n_prefix;
        n_drem = nn_drem; n_prod = nn_prod; n_prefix = nn_prefix;
        if (t + 2 < n_steps) fetch_row_scalars(q0 + 2 * kRows, nn_drem, nn_prod, nn_prefix);
        const int w_last = q0 + kRows - 1;
        const int qi = q0 + col;
        const bool row_ok = qi < L;
        const int st_next = (t + 1) & 3;
        uint32_t pk[8], dzk[8];
        const int lim = row_ok ? qi + ac - jb - 16 * half : 0;
        // The barrier that ends the previous step is met here, behind this step's bookkeeping, which covers the
        // latency of the previous step's P / dZ writes.
        __builtin_amdgcn_sched_barrier(0);
        if (t > 0) lds_barrier();
        if (jb > min(w_last, L - 1) - 1 + ac) {              // no row of the sequence in this step sees the sub-tile (and
                                                             // no per-row scalars were recorded for it)
          scores(st_next, s_next, dp_next);
#pragma unroll
          for (int i = 0; i < 8; i++) { pk[i] = 0; dzk[i] = 0; }
        } else if ((jb + 31) > (q0 - 1 + ac) || w_last >= L) {
          fused(std::true_type{}, st_next, s_cur, dp_cur, s_next, dp_next, lim, drem, prod_in, prefix_in, pk, dzk);
        } else {
          fused(std::false_type{}, st_next, s_cur, dp_cur, s_next, dp_next, lim, drem, prod_in, prefix_in, pk, dzk);
        }
        // [query][key] tiles: this lane's 16 consecutive keys start at column 32*g + 16*half of row `col`.
        T* p_lds = lds + Lds::kP + (t & 1) * 2 * Lds::kPTile;
        u32x4* pp = reinterpret_cast<u32x4*>(p_lds + col * kPStride + 32 * g + 16 * half);
        u32x4* dd = reinterpret_cast<u32x4*>(p_lds + Lds::kPTile + col * kPStride + 32 * g + 16 * half);
#pragma unroll
        for (int c = 0; c < 2; c++) {
          pp[c] = u32x4{pk[4 * c], pk[4 * c + 1], pk[4 * c + 2], pk[4 * c + 3]};
          dd[c] = u32x4{dzk[4 * c], dzk[4 * c + 1], dzk[4 * c + 2], dzk[4 * c + 3]};
        }
        if (t == n_steps - 1 && have_next) load_kv(next_tile);   // kf / vf have fed their last MFMAs of this tile
      };
      f32x16 s_a, dp_a, s_b, dp_b;
      if (n_steps > 0) scores(0, s_a, dp_a);
      else if (have_next) load_kv(next_tile);
      for (int t = 0; t <= n_steps; t += 2) {
        step(t, s_a, dp_a, s_b, dp_b);
        if (t + 1 <= n_steps) step(t + 1, s_b, dp_b, s_a, dp_a);
      }
      lds_barrier();                                         // the barrier of the last step
    }  // tile walk (producers)
  } else {
    // Consumer wave (out, cp) owns, for ALL 128 keys of the tile, the columns 32*kCT*cp .. +32*kCT-1 of ONE of the two
    // outputs: dV (out = 0: P^T dO) or dK (out = 1: dZ^T Q).  Per 16 rows that is 4 weight operands + kCT row operands
    // for 4*kCT MFMAs: the LDS transpose reads, which bound this kernel, are a quarter fewer than with a wave that
    // holds 64 keys of both outputs.
    constexpr int kCT = DH / 64;                             // 32-column blocks per consumer wave
    const int out = wave >> 1, cp = wave & 1;
    f32x16 acc[4][kCT];
    // Two sets of staging registers, used alternately: a step's rows are requested two steps before they are
    // written to LDS (a step is shorter than a global load).
    TileCopy<T, DH, kRows, true> cq[2], cdo[2];
    auto stage_first = [&](const Tile& tl) {                 // rows of steps 0 and 1 of a tile
      const T* qb = (const T*)p.q.ptr + tl.seq_id * p.q.sb + head * p.q.sh + (int64_t)tl.seq_start * p.q.st;
      const T* dob = (const T*)p.d_o.ptr + tl.seq_id * p.d_o.sb + head * p.d_o.sh + (int64_t)tl.seq_start * p.d_o.st;
      const RowSource<T> qs = make_row_source<T, true>(qb, p.q.st, tl.seq_len, DH), ds = make_row_source<T, true>(dob, p.d_o.st, tl.seq_len, DH);
      const int rb = first_row_block(tl);
#pragma unroll
      for (int i = 0; i < 2; i++)                            // rows beyond the sequence read as zero
        if (rb + i * kRows < tl.seq_len) {
          cq[i].load(qs, rb + i * kRows);
          cdo[i].load(ds, rb + i * kRows);
        }
    };
    if (w < n_tiles) stage_first(next_tile);
    // The results of a tile are stored during the first step of the NEXT tile, when the consumers have nothing to
    // contract yet (and after the last tile): acc[m][n][r] is key origin + 32*m + 8*(r/4) + 4*half + r%4,
    // column 32*(kCT*cp + n) + col.
    bool pending = false;
    Tile done_tile = next_tile;
    auto store_results = [&](const Tile& tl) {
      const int tl_len = tl.seq_len, tl_j0 = tl.origin;
      const int64_t tl_tok0 = tl.seq_start;
      T* outb = out ? (T*)p.dk.ptr + tl.seq_id * p.dk.sb + head * p.dk.sh + tl_tok0 * p.dk.st
                    : (T*)p.dv.ptr + tl.seq_id * p.dv.sb + head * p.dv.sh + tl_tok0 * p.dv.st;
      const int64_t out_st = out ? p.dk.st : p.dv.st;
      if (p.add_rem && out == 0) {
        // the remainder term o += rem * v contributes rem_j * d_o_j to dv_j
        const T* dob = (const T*)p.d_o.ptr + tl.seq_id * p.d_o.sb + head * p.d_o.sh + tl_tok0 * p.d_o.st;
#pragma unroll
        for (int m = 0; m < 4; m++)
#pragma unroll
          for (int r = 0; r < 16; r++) {
            const int key = tl_j0 + 32 * m + 8 * (r >> 2) + 4 * half + (r & 3);
            if (key < tl_len) {
              const float rem = fast_exp2(p.row_stat[tl.seq_id * p.stat_sb + head * p.stat_sh + tl_tok0 + key]);
#pragma unroll
              for (int n = 0; n < kCT; n++)
                acc[m][n][r] += rem * (float)dob[(int64_t)key * p.d_o.st + 32 * (kCT * cp + n) + col];
            }
          }
      }
      const RowSink<T> sink = make_row_sink<T>(outb, out_st, tl_len, DH);
      const float scale = out ? p.logit_scale : 1.f;
      T* scratch = lds + Lds::kScratch + wave * (32 * lds_stride<32>());
#pragma unroll
      for (int m = 0; m < 4; m++)
#pragma unroll
        for (int n = 0; n < kCT; n++)
          store_acc_tile_wide<T>(sink, acc[m][n], scale, tl_j0 + 32 * m, 32 * (kCT * cp + n), half, col, lane, scratch);
    };
    for (int slot = w; slot < n_tiles;) {
      const Tile tile = next_tile;
      const int L = tile.seq_len, j0 = tile.origin;
      const int64_t tok0 = tile.seq_start;
      const int first_row = j0 + 1 - ac;
      const int row_begin = first_row < L ? (first_row / kRows) * kRows : L;
      const int n_steps = (L - row_begin + kRows - 1) / kRows;
      const T* qb = (const T*)p.q.ptr + tile.seq_id * p.q.sb + head * p.q.sh + tok0 * p.q.st;
      const T* dob = (const T*)p.d_o.ptr + tile.seq_id * p.d_o.sb + head * p.d_o.sh + tok0 * p.d_o.st;
      const RowSource<T> qsrc = make_row_source<T, true>(qb, p.q.st, L, DH), dosrc = make_row_source<T, true>(dob, p.d_o.st, L, DH);
      // Rows of step r into stage r%4 from register set r%2, then the rows of step r+2 requested into that set.
      auto stage_rows = [&](int r) {
        T* q_lds = lds + Lds::kQ + (r & 3) * 2 * Lds::kQdoTile;
        const int rn = row_begin + (r + 2) * kRows;
        if (r & 1) {
          cq[1].store(q_lds); cdo[1].store(q_lds + Lds::kQdoTile);
          if (rn < L) { cq[1].load(qsrc, rn); cdo[1].load(dosrc, rn); }
        } else {
          cq[0].store(q_lds); cdo[0].store(q_lds + Lds::kQdoTile);
          if (rn < L) { cq[0].load(qsrc, rn); cdo[0].load(dosrc, rn); }
        }
      };
      stage_rows(0);
      stage_rows(1);
      lds_barrier();
      slot = *next_slot_lds;                                 // the tile after this one
      const bool have_next = slot < n_tiles;
      if (have_next) next_tile = p.k_tiles[slot];
      // Step 0: nothing to contract yet, so the previous tile's results leave now.
      if (pending) store_results(done_tile);
      stage_rows(2);
#pragma unroll
      for (int m = 0; m < 4; m++)
#pragma unroll
        for (int n = 0; n < kCT; n++)
#pragma unroll
          for (int r = 0; r < 16; r++) acc[m][n][r] = 0.f;
      lds_barrier();
      for (int t = 1; t <= n_steps; ++t) {
        stage_rows(t + 2);
        const int u = t - 1;
        const T* q_lds = lds + Lds::kQ + (u & 3) * 2 * Lds::kQdoTile;
        const T* do_lds = q_lds + Lds::kQdoTile;
        const T* p_lds = lds + Lds::kP + (u & 1) * 2 * Lds::kPTile;
        const T* dz_lds = p_lds + Lds::kPTile;
        // dV[key][d] += sum_i P[i][key] dO[i][d]  or  dK[key][d] += sum_i dZ[i][key] Q[i][d]   (i over the 32 rows)
        const T* w_lds = out ? dz_lds : p_lds;               // weights: [row][key]
        const T* r_lds = out ? q_lds : do_lds;               // rows:    [row][column]
#pragma unroll
        for (int c = 0; c < kRows / 16; c++) {
          const int row0 = 16 * c + 8 * half;
          vec8 aw[4], br[kCT];
#pragma unroll
          for (int m = 0; m < 4; m++) aw[m] = lds_col8<T>(w_lds, kPStride, row0, 32 * m, lane);
#pragma unroll
          for (int n = 0; n < kCT; n++) br[n] = lds_col8<T>(r_lds, kRowStride, row0, 32 * (kCT * cp + n), lane);
#pragma unroll
          for (int m = 0; m < 4; m++)
#pragma unroll
            for (int n = 0; n < kCT; n++) acc[m][n] = Elem<T>::mfma(aw[m], br[n], acc[m][n]);
        }
        lds_barrier();
      }
      // The next tile's first rows are requested before this tile's results are stored.
      if (have_next) stage_first(next_tile);
      pending = true;
      done_tile = tile;
    }  // tile walk (consumers)
    if (pending) store_results(done_tile);
  }
}

template <typename T, int DH>
static hipError_t launch_dkv4(const BwdParams& p_in, int max_tiles, hipStream_t stream) {
  const size_t lds_bytes = (size_t)Dkv4Lds<DH>::kElems * sizeof(T) + 256;      // + the published queue slot
  static std::atomic<uint64_t> lds_done{0};
  int dev = 0, cus = 0;
  hipError_t e = device_cus(&dev, &cus);
  if (e != hipSuccess) return e;
  if ((e = raise_lds_limit(&bwd_dkv4_kernel<T, DH>, lds_done, dev, lds_bytes)) != hipSuccess) return e;
  BwdParams p = p_in;
  p.wgs_per_head = cus / p.num_heads > 0 ? cus / p.num_heads : 1;
  if (p.wgs_per_head > max_tiles) p.wgs_per_head = max_tiles;
  const dim3 grid((unsigned)(p.wgs_per_head * p.num_heads)), block(kDkv4Threads);
  hipLaunchKernelGGL((bwd_dkv4_kernel<T, DH>), grid, block, lds_bytes, stream, p);
  return hipGetLastError();
}

template <typename T, int DH, bool kFast>
static hipError_t launch_one(const BwdParams& p, int max_tiles, hipStream_t stream) {
  const size_t lds_bytes = (size_t)DkvLds<DH>::kElems * sizeof(T);
  static std::atomic<uint64_t> lds_done{0};
  int dev = 0, cus = 0;
  hipError_t e = device_cus(&dev, &cus);
  if (e != hipSuccess) return e;
  if ((e = raise_lds_limit(&bwd_dkv_kernel<T, DH, kFast>, lds_done, dev, lds_bytes)) != hipSuccess) return e;
  const dim3 grid((unsigned)(max_tiles * p.num_heads)), block(kThreads);
  hipLaunchKernelGGL((bwd_dkv_kernel<T, DH, kFast>), grid, block, lds_bytes, stream, p);
  return hipGetLastError();
}

template <typename T>
static hipError_t launch_t(const BwdParams& p, int max_tiles, hipStream_t stream) {
  // head_dim 64 measures slightly faster on the 64-key kernel (its steps are already short).
  if (p.vec_ok && p.head_dim == 128) return launch_dkv4<T, 128>(p, max_tiles, stream);
  if (p.vec_ok && p.head_dim == 64) return launch_dkv3<T, 64>(p, max_tiles, stream);
  return p.head_dim <= 64 ? launch_one<T, 64, false>(p, max_tiles, stream) : launch_one<T, 128, false>(p, max_tiles, stream);
}

// Keys per key tile of the kernel launch_bwd_dkv will pick for these parameters.
int dkv_key_tile(const BwdParams& p) {
  return (p.vec_ok && p.head_dim == 128) ? kDkv4Keys : kBlockK;
}

hipError_t launch_bwd_dkv(const BwdParams& p, int dtype_is_f16, int max_tiles, hipStream_t stream) {
  return dtype_is_f16 ? launch_t<_Float16>(p, max_tiles, stream) : launch_t<__bf16>(p, max_tiles, stream);
}

}  // namespace sba
