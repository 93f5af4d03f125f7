// Backward in ONE kernel for head_dim 128: dQ, dK and dV from a single evaluation of the tile math.
//
// The two-kernel backward (sba_bwd_dq.hip, sba_bwd_dkv.hip) evaluates S^T = K Q^T, dP^T = V dO^T and the whole
// element-wise math twice, because dK/dV of a key tile sum over rows while the logit gradient
//     dz_ij = g_ij - sigma_ij C_ij,   C_ij = sum_{j' <= j} g_ij',   g_ij = A_ij (dO_i . v_j - drem_i)
// needs a prefix sum along the keys of a row, which a key-stationary workgroup does not own
// (the reference keeps rows stationary and serialises dK/dV behind a spin lock per key tile instead:
// stickbreaking_attention/sb_varlen/sb_varlen_bwd.py:11-53, :405-473).  Here the workgroups that own the
// 128-key tiles J = 0, 1, 2, ... of one (head, sequence) form a CHAIN: every tile sweeps the 32-row blocks of the
// sequence from the LAST block down to its own diagonal, and hands two things per row block to the tile above it
// through L2: C below the next tile (one fp32 per row, tagged) and the rows' partial dQ (fp32).  Tile J adds its
// own share and passes them on; the tile that holds a row's diagonal converts that row's dQ to the output type.
// The order of every sum is fixed by the chain, so the results are bit-reproducible, and no element of dK, dV or
// dQ is ever accumulated by two workgroups at once.
//
// Workgroup = 8 waves, persistent, one per CU, taking the key tiles of one head from a cursor:
//   producers (waves 0-3, one per 32-key sub-tile g, K/V operands stationary in registers): per slot, the
//     element-wise math of row block k with the S^T / dP^T MFMAs of block k+1 dealt among it.  The math is split:
//     phase A leaves P, sigma, dz without the C term, and the sub-tile's row totals of g; phase B, one slot later
//     (after the barrier that makes all four sub-tiles' totals visible), subtracts sigma * C and writes dZ.
//   consumers (waves 4-7): bring Q/dO rows in with direct-to-LDS loads three slots ahead, contract
//     dV += P^T dO (one slot behind) or dK += dZ^T Q (two slots behind) for all 128 keys x 64 columns of one output,
//     and every consumer contracts 32 columns of dQ^T = K^T dZ^T over the tile's 128 keys on top of the partial sum
//     loaded from the chain.
// All workgroups of a head run on one XCD (workgroup ids are dealt round-robin to the XCDs), so the hand-over
// needs L2 coherence only: ordinary stores, completed (s_waitcnt vmcnt(0)) before a flag store, and loads that
// bypass the vector L1 (sc1).  Waits are bounded: a wait that runs out sets the status word and the kernel
// finishes with wrong results rather than hanging.
#include "sba_device.hpp"
#include "sba_host.hpp"
#include "sba_params.hpp"

#include <atomic>
#include <type_traits>

namespace sba {

constexpr int kChKeys = 128, kChRows = 32, kChThreads = 512;
constexpr int kChQStages = 6, kChDoStages = 5;   // Q rows live from the request (3 slots ahead) to the dK/dQ contraction
                                                 // (2 slots behind), dO rows to the dV contraction (1 slot behind)
constexpr int kChMinSlots = 6;                   // slots per tile: the next tile is claimed late (see below)
constexpr int kChSpinLimit = 1 << 17;

struct ChLds {   // byte offsets into the dynamic LDS segment
  static constexpr int kRowBytes = lds_stride<128>() * 2;            // 304: padded row of 128 16-bit elements
  static constexpr int kStage = kChRows * kRowBytes;                 // one 32-row tile (Q, dO, P or dZ)
  static constexpr int kQ = 0;
  static constexpr int kDo = kQ + kChQStages * kStage;
  static constexpr int kP = kDo + kChDoStages * kStage;              // P of the even / odd slots
  static constexpr int kDz = kP + 2 * kStage;                        // dZ likewise
  static constexpr int kScratchWave = 32 * lds_stride<32>() * 2;     // wave-private transposition scratch
  static constexpr int kScratch = kDz + 2 * kStage;
  static constexpr int kTot = kScratch + 4 * kScratchWave;           // float [2][4][32]: row totals of g per sub-tile
  static constexpr int kNext = kTot + 2 * 4 * 32 * 4;                // the next tile: 6 dwords of Tile + its slot
  static constexpr int kBytes = kNext + 64;
};

// ---------------------------------------------------------------------------------------------------------
// Element-wise math, phase A, for the 16 keys this lane owns of a 32-key sub-tile (layout as in sba_device.hpp).
//   pk    : P packed to 16 bit, two keys per word
//   beta  : sigma
//   dzl   : g - sigma * (sum of g over this lane's keys up to and including the key)
//   tot   : sum of g over all 32 keys of the sub-tile (both half-waves hold it)
//   fix   : what C holds below this lane's keys within the sub-tile (the lower half-wave's total, for the upper one)
template <typename T, bool kDiagonal>
__device__ __forceinline__ void chain_math_a(const f32x16& s, const f32x16& dp, float scale_log2, int lim, int half,
                                             float drem, float prod_in, uint32_t (&pk)[8], float (&beta)[16],
                                             float (&dzl)[16], float& tot, float& fix) {
  float pe[16];
  float run = 1.f;
#pragma unroll
  for (int R = 15; R >= 0; --R) {
    float x = s[R] * scale_log2;
    if (kDiagonal) x = (R < lim) ? x : -INFINITY;
    const float omb = fast_rcp(1.f + fast_exp2(x));
    beta[R] = 1.f - omb;
    pe[R] = run;
    run *= omb;
  }
  const float oth = other_half(run, half);
  const float seed = half ? prod_in : prod_in * oth;          // the upper half-wave holds the higher keys
  float acc = 0.f;
#pragma unroll
  for (int R = 0; R < 16; R++) {
    const float a = beta[R] * (pe[R] * seed);
    const float g = a * (dp[R] - drem);
    pe[R] = a;
    acc += g;
    dzl[R] = g - beta[R] * acc;
  }
  const float oth_g = other_half(acc, half);
  fix = half ? oth_g : 0.f;
  tot = acc + oth_g;
#pragma unroll
  for (int R = 0; R < 16; R += 2) pk[R >> 1] = pack2<T>(pe[R], pe[R + 1]);
}

// LDS reads of the consumer waves, as inline assembly: the compiler cannot tell the direct-to-LDS loads in flight
// (other stages) from these reads and would wait for all of them in front of every read it knows about.
template <int kOff>
__device__ __forceinline__ void ch_tr_read(u32x2& lo, u32x2& hi, int addr) {
  asm volatile("ds_read_b64_tr_b16 %0, %2 offset:%3\n\tds_read_b64_tr_b16 %1, %2 offset:%4"
               : "=&v"(lo), "=&v"(hi) : "v"(addr), "n"(kOff), "n"(kOff + 4 * ChLds::kRowBytes) : "memory");
}
template <int kOff>
__device__ __forceinline__ void ch_row_read(u32x4& v, int addr) {
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(v) : "v"(addr), "n"(kOff) : "memory");
}
// Wait until at most kLeft LDS reads of this wave are outstanding (they return in order); the operands passed
// through are the ones that may be used afterwards.
template <int kLeft>
__device__ __forceinline__ void ch_landed6(u32x2 (&a_lo)[4], u32x2 (&a_hi)[4], u32x2 (&b_lo)[2], u32x2 (&b_hi)[2]) {
  asm volatile("s_waitcnt lgkmcnt(%12)"
               : "+v"(a_lo[0]), "+v"(a_hi[0]), "+v"(a_lo[1]), "+v"(a_hi[1]), "+v"(a_lo[2]), "+v"(a_hi[2]), "+v"(a_lo[3]),
                 "+v"(a_hi[3]), "+v"(b_lo[0]), "+v"(b_hi[0]), "+v"(b_lo[1]), "+v"(b_hi[1])
               : "n"(kLeft));
}
template <int kLeft>
__device__ __forceinline__ void ch_landed4(u32x4& a, u32x4& b, u32x4& c, u32x4& d) {
  asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d) : "n"(kLeft));
}
__device__ __forceinline__ u32x4 ch_join(const u32x2& lo, const u32x2& hi) { return u32x4{lo[0], lo[1], hi[0], hi[1]}; }

// A load that bypasses the vector L1 (sc1): what another workgroup of this XCD stored and completed is seen.
// Loads of the chain by the consumer waves, as inline assembly: the wave waits for exactly these (loads return in
// order) and not for the younger row requests, which the compiler's own wait counts cannot express across the
// branches in between.  sc1: served by the L2, never by this compute unit's vector cache.
template <int kOff>
__device__ __forceinline__ void ch_chain_load(u32x4& v, int voff, u32x4 desc, int soff) {
  asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen offset:%4 sc1" : "=v"(v) : "v"(voff), "s"(desc), "s"(soff), "n"(kOff) : "memory");
}
__device__ __forceinline__ void ch_flag_request(int& v, const int32_t* f) {
  asm volatile("global_load_dword %0, %1, %2 sc1" : "=v"(v) : "v"(0), "s"(f) : "memory");
}
// Wait until at most kLeft vector memory operations of this wave are outstanding.
// Placed after the wait for the loads above: from here on the compiler may read their registers.  (One statement for
// all paths: two of these in the arms of a branch make the compiler merge their results with register copies placed
// in front of the waits.)
__device__ __forceinline__ void ch_chain_landed(u32x4 (&c)[4], int& flag) {
  asm volatile("" : "+v"(c[0]), "+v"(c[1]), "+v"(c[2]), "+v"(c[3]), "+v"(flag) :: "memory");
}
template <int kLeft>
__device__ __forceinline__ void ch_vm_wait() { asm volatile("s_waitcnt vmcnt(%0)" :: "n"(kLeft) : "memory"); }
__device__ __forceinline__ int ch_load_flag(const int32_t* f) {
  return __hip_atomic_load(f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
constexpr int kAuxSc1 = 16;

template <typename T>
__global__ __launch_bounds__(kChThreads) void bwd_chain_kernel(BwdParams p) {
  constexpr int DH = 128;
  typedef typename Elem<T>::vec8 vec8;
  constexpr int kRowStride = lds_stride<DH>();           // elements; P / dZ tiles use the same stride
  constexpr int kSteps = DH / 16;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  typedef __attribute__((address_space(3))) unsigned char lds_u8;
  typedef __attribute__((address_space(3))) void lds_void;

  const int n_tiles = p.counts[kCountK];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane((threadIdx.x >> 6) & 3);
  const bool producer = threadIdx.x < 256;
  const int half = lane >> 5, col = lane & 31;
  const int ac = p.attend_current;
  const int hpx = p.num_heads >> 3, r0 = blockIdx.x >> 3;
  const int head = (blockIdx.x & 7) * hpx + r0 % hpx;      // the launcher guarantees num_heads % 8 == 0
  const int w = r0 / hpx;
  int* next_lds = reinterpret_cast<int*>(lds_raw + ChLds::kNext);
  float* tot_lds = reinterpret_cast<float*>(lds_raw + ChLds::kTot);

  // All workgroups of a head must share an XCD (the hand-over relies on one L2): the first to arrive records its
  // XCC id for the head, the others compare.
  if (threadIdx.x == 0) {
    const int xcc = (int)(__builtin_amdgcn_s_getreg((20) | (0 << 6) | ((4 - 1) << 11)) & 15) + 1;     // HW_REG_XCC_ID
    const int old = atomicCAS(p.chain_head_xcc + head, 0, xcc);
    if (old != 0 && old != xcc) atomicMax(p.status, kSchedChainXcd);
  }
  // Rows of the packed token axis that belong to no sequence: zero gradients (the reference allocates zeros).
  {
    const int64_t covered = p.counts[kCountCovered];
    if (covered < p.total_tokens) {
      const int64_t n = p.total_tokens - covered, per = (n + p.wgs_per_head - 1) / p.wgs_per_head;
      const int64_t a = covered + per * w, b = a + per < p.total_tokens ? a + per : p.total_tokens;
      if (a < b) {
        zero_rows<T>(p.dq, head, a, b, DH);
        zero_rows<T>(p.dk, head, a, b, DH);
        zero_rows<T>(p.dv, head, a, b, DH);
      }
    }
  }
  // The first tile.  Tiles are taken from the head's cursor when a workgroup needs one, never ahead of time: the
  // chain wants the tiles of a sequence STARTED in key order, and the workgroups become free in that order only
  // if each takes its next tile late.
  if (threadIdx.x == 0) next_lds[8] = atomicAdd(p.head_queue + head, 1);
  __syncthreads();
  int slot_idx = next_lds[8];
  if (slot_idx >= n_tiles) return;
  Tile tile = p.k_tiles[slot_idx];
  __syncthreads();                                           // everyone has read the slot before it is rewritten

  // Per-tile facts shared by both roles.
  struct Facts { int L, j0, J, nb, n, S, a; int64_t tok0, crow; };
  auto facts_of = [&](const Tile& tl) {
    Facts f;
    f.L = tl.seq_len; f.j0 = tl.origin; f.J = f.j0 / kChKeys; f.tok0 = tl.seq_start;
    f.nb = (f.L + kChRows - 1) / kChRows;
    f.n = f.nb - 4 * f.J;                                    // row blocks from the last one down to the tile's diagonal
    f.S = f.n + 2 > kChMinSlots ? f.n + 2 : kChMinSlots;
    f.a = f.n > 5 ? f.n - 5 : 0;                             // slot in which the next tile is claimed
    f.crow = (int64_t)tl.seq_id * p.chain_sb + tl.seq_start; // first row of the sequence in the chain buffers
    return f;
  };
  bool aborted = false;
  auto give_up = [&]() { aborted = true; if (lane == 0) atomicMax(p.status, kSchedChainTimeout); };

  if (producer) {
    // =====================================================================================================
    const int g = wave;
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
    // Q / dO stages of the next row block to run MFMAs on (the stages rotate over the blocks in the order they
    // are requested, across tiles).
    int mq = 0, md = 0;
    auto advance = [&]() { mq = mq == kChQStages - 1 ? 0 : mq + 1; md = md == kChDoStages - 1 ? 0 : md + 1; };
    auto scores = [&](f32x16& s, f32x16& dp) {
      const T* q_lds = reinterpret_cast<const T*>(lds_raw + ChLds::kQ + mq * ChLds::kStage);
      const T* do_lds = reinterpret_cast<const T*>(lds_raw + ChLds::kDo + md * ChLds::kStage);
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
      advance();
    };
    load_kv(tile);
    f32x16 s_a, dp_a, s_b, dp_b;
    lds_barrier();                                           // the first three row blocks of the first tile are in LDS
    scores(s_a, dp_a);
    // The walk over the tiles is ONE loop over slots, so that the two accumulator sets keep alternating across the
    // tile boundaries (the last slot of a tile computes the first scores of the next one into the set that slot 0
    // of the next tile then reads).
    Tile next_tile = tile;
    bool have_next = false, done = false, first_slot = true;
    int s = 0;                                               // slot within the tile
    // Facts of the current tile (kept as scalars) and what derives from them.
    int L, J, nb, n, S, a_slot, jb;
    const float* carry = nullptr;
    const T* drem_p = nullptr;
    __amdgpu_buffer_rsrc_t crs;
    uint32_t* cbase = nullptr;
    auto enter_tile = [&](const Tile& tl) {
      const Facts f = facts_of(tl);
      L = f.L; J = f.J; nb = f.nb; n = f.n; S = f.S; a_slot = f.a; jb = f.j0 + 32 * g;
      const int n_qt = (f.L + kBlockQ - 1) / kBlockQ;
      carry = p.carry + (int64_t)head * p.carry_head_stride + tl.carry_base + carry_offset(4 * f.J + g, n_qt) - (int64_t)kBlockQ * f.J;
      drem_p = p.d_rem.ptr ? (const T*)p.d_rem.ptr + tl.seq_id * p.d_rem.sb + head * p.d_rem.sh + f.tok0 * p.d_rem.st : nullptr;
      // Chain: {C below this tile, tag} per row, written by the tile below (tag J), rewritten by this tile (tag J + 1).
      cbase = p.chain_c + 2 * ((int64_t)head * p.chain_rows + f.crow);
      crs = __builtin_amdgcn_make_buffer_rsrc((void*)cbase, 0, f.L * 8, 0x00020000);
    };
    // Per-row scalars of row block k of the CURRENT tile (gradient of rem, product above the sub-tile); fetched two
    // blocks ahead.  The first two blocks of a tile are requested when the tile is entered.
    T n_drem = (T)0.f, nn_drem = (T)0.f;
    float n_prod = 1.f, nn_prod = 1.f;
    auto row_scalars = [&](int k, T& drem_r, float& prod_r) {
      const int r = kChRows * (nb - 1 - k) + col;
      drem_r = (T)0.f;
      if (drem_p && r < L) drem_r = drem_p[r * p.d_rem.st];
      prod_r = carry[r];
    };
    // The same for the first two blocks of the NEXT tile, requested in the last two slots of the current one.
    auto next_row_scalars = [&](int k, T& drem_r, float& prod_r) {
      const Facts f = facts_of(next_tile);
      const int n_qt = (f.L + kBlockQ - 1) / kBlockQ;
      const float* c2 = p.carry + (int64_t)head * p.carry_head_stride + next_tile.carry_base + carry_offset(4 * f.J + g, n_qt) - (int64_t)kBlockQ * f.J;
      const int r = kChRows * (f.nb - 1 - k) + col;
      drem_r = (T)0.f;
      if (p.d_rem.ptr && r < f.L)
        drem_r = ((const T*)p.d_rem.ptr)[next_tile.seq_id * p.d_rem.sb + head * p.d_rem.sh + (f.tok0 + r) * p.d_rem.st];
      prod_r = f.n > k ? c2[r] : 1.f;
    };
    enter_tile(tile);
    row_scalars(0, n_drem, n_prod);
    if (n > 1) row_scalars(1, nn_drem, nn_prod);
    // Phase-B state of the row block whose phase A ran in the previous slot.
    float beta[16], dzl[16];
    float fix_half = 0.f, tot_own = 0.f;
    u32x2 cin = {0u, 0u};
#pragma unroll
    for (int i = 0; i < 16; i++) { beta[i] = 0.f; dzl[i] = 0.f; }
    auto slot_fn = [&](f32x16& s_cur, f32x16& dp_cur, f32x16& s_next, f32x16& dp_next) {
      const bool has_item = s < n, has_b = s >= 1 && s <= n;
      const int q0 = kChRows * (nb - 1 - s);                 // first row of block s (when has_item)
      const T drem_raw = n_drem;
      float prod_in = n_prod;
      if (has_item) { n_drem = nn_drem; n_prod = nn_prod; }
      if (s + 2 < n) row_scalars(s + 2, nn_drem, nn_prod);
      else if (have_next && s == S - 2) next_row_scalars(0, n_drem, n_prod);
      else if (have_next && s == S - 1) next_row_scalars(1, nn_drem, nn_prod);
      const int w_last = q0 + kChRows - 1;
      const int qi = q0 + col;
      const bool row_ok = qi < L;
      // A sub-tile no row of the sequence in this block can see goes through the masked form with every key hidden
      // (nothing was recorded for it to start from): all-zero P, dZ and totals.
      const bool unseen = jb > min(w_last, L - 1) - 1 + ac;
      const int lim = (row_ok && !unseen) ? qi + ac - jb - 16 * half : 0;
      if (unseen) prod_in = 1.f;
      // The barrier that ends the previous slot is met here, behind this slot's bookkeeping.
      __builtin_amdgcn_sched_barrier(0);
      if (!first_slot) lds_barrier();
      first_slot = false;
      if (s == a_slot + 3) {                                 // the next tile, as the claiming wave published it
        const int ns = __builtin_amdgcn_readfirstlane(next_lds[8]);
        have_next = ns < n_tiles;
        if (have_next) {
          next_tile.seq_start = __builtin_amdgcn_readfirstlane(next_lds[0]);
          next_tile.seq_len = __builtin_amdgcn_readfirstlane(next_lds[1]);
          next_tile.origin = __builtin_amdgcn_readfirstlane(next_lds[2]);
          next_tile.seq_id = __builtin_amdgcn_readfirstlane(next_lds[3]);
          const uint32_t lo = __builtin_amdgcn_readfirstlane(next_lds[4]), hi = __builtin_amdgcn_readfirstlane(next_lds[5]);
          next_tile.carry_base = (int64_t)(((uint64_t)hi << 32) | lo);
        }
      }
      // ---- phase B of block s-1: dZ = dzl - sigma * (C below the lane's keys) ---------------------------------
      if (has_b) {
        const int kb_ = s - 1;
        const int qb = kChRows * (nb - kb_ - 1) + col;
        const float* tl_ = tot_lds + (kb_ & 1) * 128;
        float below = 0.f;
        if (J > 0) {                                         // validated before the barrier that ended the previous slot
          const uint32_t cin_bits = cin[0];
          below = (qb < L) ? __builtin_bit_cast(float, cin_bits) : 0.f;
        }
        if (g > 0) below += tl_[col];
        if (g > 1) below += tl_[32 + col];
        if (g > 2) below += tl_[64 + col];
        const float fixup = below + fix_half;
        uint32_t dzk[8];
#pragma unroll
        for (int R = 0; R < 16; R += 2) dzk[R >> 1] = pack2<T>(dzl[R] - beta[R] * fixup, dzl[R + 1] - beta[R + 1] * fixup);
        T* dz_lds = reinterpret_cast<T*>(lds_raw + ChLds::kDz + (kb_ & 1) * ChLds::kStage);
        u32x4* dd = reinterpret_cast<u32x4*>(dz_lds + col * kRowStride + 32 * g + 16 * half);
        dd[0] = u32x4{dzk[0], dzk[1], dzk[2], dzk[3]};
        dd[1] = u32x4{dzk[4], dzk[5], dzk[6], dzk[7]};
        if (g == 3 && half == 0 && qb < L) {
          // C below the next tile, tagged, in one 8-byte store.  Issued as inline assembly so that the compiler's count of this wave's outstanding loads
          // stays what it is: a store it knew of would turn every wait for a prefetched load into a wait for all.
          const float cnext = below + tot_own;
          const u32x2 cv = {__builtin_bit_cast(uint32_t, cnext), (uint32_t)(J + 1)};
          uint32_t* dst = cbase + 2 * qb;
          asm volatile("global_store_dwordx2 %0, %1, off" :: "v"(dst), "v"(cv) : "memory");
        }
      }
      // ---- phase A of block s, with the MFMAs of block s+1 (or of nothing: the last block's go unused) --------
      if (has_item) {
        const float drem = (float)drem_raw;
        if (J > 0)        // C below this tile for block s: needed in the next slot
          cin = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(crs, qi * 8, 0, kAuxSc1));
        const bool diag = unseen || (jb + 31) > (q0 - 1 + ac) || w_last >= L;
        uint32_t pk[8];
        auto fused = [&](auto diag_tag) {
          constexpr bool kDiag = decltype(diag_tag)::value;
          // The group solver is greedy and sensitive to these counts: with most other values it puts half of the MFMAs
          // back to back.  These give one MFMA per 13 (9) vector-ALU instructions through the whole block in both
          // copies of the slot; check the generated code after changing the math.
#ifndef SBA_CH_LEAD
#define SBA_CH_LEAD 24
#define SBA_CH_GAP_D 13
#define SBA_CH_GAP_N 9
#endif
#ifndef SBA_CH_LEAD_N
#define SBA_CH_LEAD_N 8
#endif
          constexpr int kLead = kDiag ? SBA_CH_LEAD : SBA_CH_LEAD_N;
          constexpr int kGap = kDiag ? SBA_CH_GAP_D : SBA_CH_GAP_N;   // (block of ~225 / ~193 vector-ALU instructions)
          constexpr int kAlu = 0x402;                        // vector ALU including transcendentals
          const T* q_lds = reinterpret_cast<const T*>(lds_raw + ChLds::kQ + mq * ChLds::kStage);
          const T* do_lds = reinterpret_cast<const T*>(lds_raw + ChLds::kDo + md * ChLds::kStage);
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
          chain_math_a<T, kDiag>(s_cur, dp_cur, p.scale_log2, lim, half, drem, prod_in, pk, beta, dzl, tot_own, fix_half);
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
        if (diag) fused(std::true_type{}); else fused(std::false_type{});
        if (s + 1 < n) advance();                            // (the last block's MFMAs ran on a stage that is not a new block)
        // [row][key] tile: this lane's 16 consecutive keys start at column 32*g + 16*half of row `col`.
        T* p_lds = reinterpret_cast<T*>(lds_raw + ChLds::kP + (s & 1) * ChLds::kStage);
        u32x4* pp = reinterpret_cast<u32x4*>(p_lds + col * kRowStride + 32 * g + 16 * half);
        pp[0] = u32x4{pk[0], pk[1], pk[2], pk[3]};
        pp[1] = u32x4{pk[4], pk[5], pk[6], pk[7]};
        if (half == 0) tot_lds[(s & 1) * 128 + 32 * g + col] = tot_own;
        // C below this tile for block s must have arrived (tag J) before this slot's barrier: after that barrier wave 3
        // replaces it with C below the next tile, and all four waves of the tile read the same slot.
        if (J > 0) {
          bool ok = !row_ok || (cin[1] == (uint32_t)J);
          if (!aborted && !__all(ok)) {       // the tile below has not got this far yet
            int spins = 0;
            while (true) {
              cin = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(crs, qi * 8, 0, kAuxSc1));
              ok = !row_ok || (cin[1] == (uint32_t)J);
              if (__all(ok)) break;
              if (++spins > kChSpinLimit || ((spins & 255) == 0 && ch_load_flag(p.status) != 0)) { give_up(); break; }
              __builtin_amdgcn_s_sleep(1);
            }
          }
        }
      }
      // K/V of the next tile into the same registers, once they have fed their last MFMAs of this tile; the next
      // tile's first scores in the last slot, then the next tile becomes the current one.
      const int kv_slot = n > a_slot + 3 ? n : a_slot + 3;
      if (s == kv_slot && have_next) load_kv(next_tile);
      if (s == S - 1) {
        if (have_next) {
          scores(s_next, dp_next);
          tile = next_tile;
          enter_tile(tile);
          have_next = false;
          s = 0;
        } else {
          done = true;
        }
      } else {
        ++s;
      }
    };
    while (true) {
      slot_fn(s_a, dp_a, s_b, dp_b);
      if (done) break;
      slot_fn(s_b, dp_b, s_a, dp_a);
      if (done) break;
    }
    lds_barrier();                                           // the consumers' last slot
  } else {
    // =====================================================================================================
    // Consumer wave c: output `out` (0: dV = P^T dO, 1: dK = dZ^T Q), columns 64*cp .. +63, all 128 keys; and columns
    // 32*c .. +31 of dQ^T.
    const int c = wave, out = c >> 1, cp = c & 1;
    // The consumer waves are the critical path of a slot (the producers wait for them at the slot barrier 30 % of the
    // time) and share each SIMD with a producer wave: raised issue priority for them is worth 2-3 % of the kernel
    // (priority 1, 2 or 3, or giving the consumers the lower wave ids instead: all the same, and not additive).
    __builtin_amdgcn_s_setprio(2);
    f32x16 acc[4][2];
    vec8 kstat[kSteps];                                      // K^T of the tile for columns 32c..: A operand of dQ^T = K^T dZ^T
    int cq_stage = 0, cd_stage = 0;                          // stages of the blocks to contract (Q: 2 behind, dO: 1 behind)
    auto bump = [](int& st, int n_st) { st = st == n_st - 1 ? 0 : st + 1; };
    // Row requests.  This wave brings in rows 8c .. 8c+7 of a block with direct-to-LDS loads of 16 bytes per lane (no
    // staging registers, no LDS write instructions).  Such a load writes the lanes' 16-byte pieces back to back, and
    // the rows are padded in LDS (19 pieces of which 16 hold data), so the lanes are laid over the padded rows: lane
    // i of load k covers piece 64k + i of the wave's 152; a lane over padding asks for an address outside the
    // buffer and leaves zeros there.  The requests run three slots ahead of the math, beyond the end of the tile the
    // wave contracts, so they keep their own descriptors: the rows of the sequence being requested from, the next
    // block, and how many blocks of that tile are left.
    __amdgpu_buffer_rsrc_t rq_q, rq_do;
    int rq_qsb = 0, rq_dosb = 0, rq_block = 0, rq_left = 0;
    int rq_qst = 0, rq_dst = 0;                              // stages of the next row block to request
    auto request_from = [&](const Tile& tl) {
      const Facts ft = facts_of(tl);
      const T* qb = (const T*)p.q.ptr + tl.seq_id * p.q.sb + head * p.q.sh + (int64_t)tl.seq_start * p.q.st;
      const T* dob = (const T*)p.d_o.ptr + tl.seq_id * p.d_o.sb + head * p.d_o.sh + (int64_t)tl.seq_start * p.d_o.st;
      const RowSource<T> qs = make_row_source<T, true>(qb, p.q.st, ft.L, DH), ds = make_row_source<T, true>(dob, p.d_o.st, ft.L, DH);
      rq_q = qs.rsrc; rq_do = ds.rsrc; rq_qsb = qs.stride_bytes; rq_dosb = ds.stride_bytes;
      rq_block = ft.nb - 1; rq_left = ft.n;
    };
    auto request_rows = [&]() {
      lds_u8* qd = (lds_u8*)lds_raw + ChLds::kQ + rq_qst * ChLds::kStage + 8 * c * ChLds::kRowBytes;
      lds_u8* dd = (lds_u8*)lds_raw + ChLds::kDo + rq_dst * ChLds::kStage + 8 * c * ChLds::kRowBytes;
      const int qo = (kChRows * rq_block + 8 * c) * rq_qsb, dob_ = (kChRows * rq_block + 8 * c) * rq_dosb;
      constexpr int kPieces = 8 * ChLds::kRowBytes / 16;     // 152
      constexpr int kOutside = 0x7ffffff0;                   // past every buffer: reads as zero
#pragma unroll
      for (int k = 0; k < 3; k++) {                          // rows beyond the sequence read as zero
        const int piece = 64 * k + lane;
        const int row = (piece * 27) >> 9, cc = piece - 19 * row;           // piece / 19 for piece < 152
        const int vq = cc < 16 ? row * rq_qsb + 16 * cc : kOutside, vd = cc < 16 ? row * rq_dosb + 16 * cc : kOutside;
        if (64 * k + 64 <= kPieces || piece < kPieces) {
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rq_q, (lds_void*)(qd + 1024 * k), 16, vq, qo, 0, 0);
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rq_do, (lds_void*)(dd + 1024 * k), 16, vd, dob_, 0, 0);
        }
      }
      bump(rq_qst, kChQStages); bump(rq_dst, kChDoStages);
      --rq_block; --rq_left;
    };
    request_from(tile);
    for (int k = 0; k < 3 && rq_left > 0; k++) request_rows();
    __builtin_amdgcn_s_waitcnt(0x0F70);
    lds_barrier();
    // Lane-constant parts of the operand addresses (bytes).
    const int s16 = lane & 15;
    const int tr_off = ((8 * half + (s16 >> 2)) * kRowStride + ((lane >> 4) & 1) * 16 + 4 * (s16 & 3)) * 2;
    const int rw_off = (col * kRowStride + 8 * half) * 2;
    bool pending = false;                                    // results of the previous tile still in the accumulators
    Tile done_tile = tile;
    int32_t* pub_flag = nullptr;                             // chain flag to publish once this wave's stores have completed
    int pub_count = 0;
    int claim_v = 0;
    uint32_t rec_w = 0;
    auto store_results = [&](const Tile& tl) {
      const int tl_len = tl.seq_len, tl_j0 = tl.origin;
      const int64_t tl_tok0 = tl.seq_start;
      T* outb = out ? (T*)p.dk.ptr + tl.seq_id * p.dk.sb + head * p.dk.sh + tl_tok0 * p.dk.st
                    : (T*)p.dv.ptr + tl.seq_id * p.dv.sb + head * p.dv.sh + tl_tok0 * p.dv.st;
      const int64_t out_st = out ? p.dk.st : p.dv.st;
      const RowSink<T> sink = make_row_sink<T>(outb, out_st, tl_len, DH);
      const float scale = out ? p.logit_scale : 1.f;
      T* scratch = reinterpret_cast<T*>(lds_raw + ChLds::kScratch + c * ChLds::kScratchWave);
#pragma unroll
      for (int m = 0; m < 4; m++)
#pragma unroll
        for (int nn = 0; nn < 2; nn++)
          store_acc_tile_wide<T>(sink, acc[m][nn], scale, tl_j0 + 32 * m, 32 * (2 * cp + nn), half, col, lane, scratch);
    };
    bool have_tile = true;
    Tile next_tile = tile;
    while (have_tile) {
      const Facts f = facts_of(tile);
      const int L = f.L, J = f.J, n = f.n, S = f.S;
      bool have_next = false;
      bool rq_next = false;                                  // the requests have moved on to the next tile (a tile of one or
                                                             // two row blocks is fully requested before this one ends)
      int32_t* const my_flag = p.chain_flags + ((int64_t)head * p.chain_tile_cap + slot_idx) * 8 + c;
      const int32_t* const pred_flag = my_flag - 8;
      int flag_seen = 0;                                     // the tile below's count for this wave's columns, as last read
      int flag_late = 0;                                     // the same count, requested at the end of a slot for the next one
      bool late_pending = false;
      // dQ partial sums of this sequence's rows (fp32, [row][128]) and the dq output, addressed per sequence.
      const __amdgpu_buffer_rsrc_t dqc_rs = __builtin_amdgcn_make_buffer_rsrc(
          (void*)(p.chain_dq + ((int64_t)head * p.chain_rows + f.crow) * DH), 0, L * DH * 4, 0x00020000);
      const uint64_t dqc_addr = (uint64_t)(p.chain_dq + ((int64_t)head * p.chain_rows + f.crow) * DH);
      const u32x4 dqc_desc = {(uint32_t)dqc_addr, (uint32_t)(dqc_addr >> 32) & 0xffffu, (uint32_t)(L * DH * 4), 0x00020000u};
      const RowSink<T> dq_sink = make_row_sink<T>((T*)p.dq.ptr + tile.seq_id * p.dq.sb + head * p.dq.sh + f.tok0 * p.dq.st, p.dq.st, L, DH);
      const int dqc_voff = col * (DH * 4) + (32 * c + 4 * half) * 4;
      const int dq_voff = col * dq_sink.stride_bytes + (32 * c + 4 * half) * 2;

      for (int s = 0; s < S; ++s) {
        // ---- first slot of a tile: the previous tile's results leave, the tile's K^T is set up --------------------
        if (s == 0) {
          // K^T of this tile for the dQ contraction, through the wave's scratch: [32 keys][32 columns] at a time,
          // gathered down the keys by the transpose read.  The previous tile's results leave first (same scratch).
          const T* kb = (const T*)p.k.ptr + tile.seq_id * p.k.sb + head * p.k.sh + f.tok0 * p.k.st;
          const RowSource<T> ksrc = make_row_source<T, true>(kb, p.k.st, L, DH);
          u32x4 kr[8];
#pragma unroll
          for (int q = 0; q < 4; q++)
#pragma unroll
            for (int h2 = 0; h2 < 2; h2++)
              kr[2 * q + h2] = __builtin_amdgcn_raw_buffer_load_b128(
                  ksrc.rsrc, (f.j0 + 32 * q + (lane >> 1)) * ksrc.stride_bytes + (32 * c + 16 * (lane & 1) + 8 * h2) * 2, 0, 0);
          if (pending) store_results(done_tile);
          pending = false;
#pragma unroll
          for (int m = 0; m < 4; m++)
#pragma unroll
            for (int nn = 0; nn < 2; nn++)
#pragma unroll
              for (int r = 0; r < 16; r++) acc[m][nn][r] = 0.f;
          T* scratch = reinterpret_cast<T*>(lds_raw + ChLds::kScratch + c * ChLds::kScratchWave);
          constexpr int kSS = lds_stride<32>();
#pragma unroll
          for (int q = 0; q < 4; q++) {
            *reinterpret_cast<u32x4*>(scratch + (lane >> 1) * kSS + 16 * (lane & 1)) = kr[2 * q];
            *reinterpret_cast<u32x4*>(scratch + (lane >> 1) * kSS + 16 * (lane & 1) + 8) = kr[2 * q + 1];
            kstat[2 * q] = lds_col8<T>(scratch, kSS, 8 * half, 0, lane);
            kstat[2 * q + 1] = lds_col8<T>(scratch, kSS, 16 + 8 * half, 0, lane);
            __builtin_amdgcn_s_waitcnt(0xC07F);              // lgkmcnt(0): the reads are done before the scratch is rewritten
          }
        }
        // ---- the chain: this wave's 32 columns of the rows of block s-2, as the tile below left them -----------
        const int kz = s - 2;                                // block whose dZ is contracted in this slot
        const bool has_z = kz >= 0 && kz < n;
        const int qz0 = kChRows * (f.nb - 1 - kz);
        const bool final_rows = kz >= n - 4;                 // rows of the tile's own 128-row block: dq leaves
        const bool chain_in = has_z && J > 0;
        // The partial dQ of the tiles below is requested here and added behind this slot's dQ MFMAs.  The tile below must
        // have published the block for this wave's columns first: its count is known from earlier readings, or polled.
        const bool do_dq = has_z;
        const bool take_in = do_dq && chain_in;
        u32x4 cin[4];
        int flag_v = 0;
        if (take_in) {
          // The count that came with the previous slot's partial sums is a slot old by now, and in half of the slots too
          // old to cover this block although the tile below has published it since.  A second request, issued just
          // before the previous slot's four stores (so that waiting for it is not waiting for them), is looked at first:
          // a poll costs a full round trip, and more than one as a rule.
          if (!aborted && flag_seen < kz + 1 && late_pending) {
            ch_vm_wait<4>();
            asm volatile("" : "+v"(flag_late) :: "memory");
            flag_seen = max(flag_seen, __builtin_amdgcn_readfirstlane(flag_late));
          }
          if (!aborted && flag_seen < kz + 1) {
            int spins = 0;
            while (true) {
              flag_seen = ch_load_flag(pred_flag);
              if (flag_seen >= kz + 1) break;
              if (++spins > kChSpinLimit || ((spins & 255) == 0 && ch_load_flag(p.status) != 0)) { give_up(); break; }
              __builtin_amdgcn_s_sleep(1);
            }
          }
          // (the loads that follow are issued after the count has been seen: the hardware issues this wave's loads in
          // program order)  The count for the slots to come travels with the partial sums.
          const int soff = qz0 * (DH * 4);
          ch_chain_load<0>(cin[0], dqc_voff, dqc_desc, soff); ch_chain_load<32>(cin[1], dqc_voff, dqc_desc, soff);
          ch_chain_load<64>(cin[2], dqc_voff, dqc_desc, soff); ch_chain_load<96>(cin[3], dqc_voff, dqc_desc, soff);
          ch_flag_request(flag_v, pred_flag);
        }
        late_pending = false;
        // ---- dV += P^T dO of block s-1, or dK += dZ^T Q of block s-2 -------------------------------------------
        const bool has_w = out ? has_z : (s >= 1 && s - 1 < n);
        const int kw = out ? kz : s - 1;
        if (has_w) {
          const int w_base = (out ? ChLds::kDz : ChLds::kP) + (kw & 1) * ChLds::kStage + tr_off;
          const int r_base = (out ? ChLds::kQ + cq_stage * ChLds::kStage : ChLds::kDo + cd_stage * ChLds::kStage) + tr_off + 128 * cp;
          constexpr int kC1 = 16 * ChLds::kRowBytes;
          u32x2 a_lo[2][4], a_hi[2][4], b_lo[2][2], b_hi[2][2];
          ch_tr_read<0>(a_lo[0][0], a_hi[0][0], w_base); ch_tr_read<64>(a_lo[0][1], a_hi[0][1], w_base);
          ch_tr_read<128>(a_lo[0][2], a_hi[0][2], w_base); ch_tr_read<192>(a_lo[0][3], a_hi[0][3], w_base);
          ch_tr_read<0>(b_lo[0][0], b_hi[0][0], r_base); ch_tr_read<64>(b_lo[0][1], b_hi[0][1], r_base);
          ch_tr_read<kC1>(a_lo[1][0], a_hi[1][0], w_base); ch_tr_read<kC1 + 64>(a_lo[1][1], a_hi[1][1], w_base);
          ch_tr_read<kC1 + 128>(a_lo[1][2], a_hi[1][2], w_base); ch_tr_read<kC1 + 192>(a_lo[1][3], a_hi[1][3], w_base);
          ch_tr_read<kC1>(b_lo[1][0], b_hi[1][0], r_base); ch_tr_read<kC1 + 64>(b_lo[1][1], b_hi[1][1], r_base);
          ch_landed6<12>(a_lo[0], a_hi[0], b_lo[0], b_hi[0]);
#pragma unroll
          for (int m = 0; m < 4; m++)
#pragma unroll
            for (int nn = 0; nn < 2; nn++)
              acc[m][nn] = Elem<T>::mfma(as_vec8<T>(ch_join(a_lo[0][m], a_hi[0][m])), as_vec8<T>(ch_join(b_lo[0][nn], b_hi[0][nn])), acc[m][nn]);
          ch_landed6<0>(a_lo[1], a_hi[1], b_lo[1], b_hi[1]);
#pragma unroll
          for (int m = 0; m < 4; m++)
#pragma unroll
            for (int nn = 0; nn < 2; nn++)
              acc[m][nn] = Elem<T>::mfma(as_vec8<T>(ch_join(a_lo[1][m], a_hi[1][m])), as_vec8<T>(ch_join(b_lo[1][nn], b_hi[1][nn])), acc[m][nn]);
        }
        // ---- everything this wave had in flight has landed by now (the rows requested and the partial dQ stored in the
        // previous slot, the partial sums just loaded): the previous slot's rows are published, and only then are the
        // rows three slots ahead requested, so that no wait of this slot is a wait for them ---------------------
        if (take_in) ch_vm_wait<5>(); else ch_vm_wait<0>();     // all but the five loads of the chain just issued
        if (pub_flag) {
          if (lane == 0) __hip_atomic_store(pub_flag, pub_count, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
          pub_flag = nullptr;
        }
        bool requested = false;
        // The next tile is claimed late and in three slots: the cursor, then the tile record, then LDS.  (Here, where
        // nothing is in flight, so that the claim's own memory operations cost the other slots no wait.)
        if (c == 3) {
          if (s == f.a) { if (lane == 0) claim_v = atomicAdd(p.head_queue + head, 1); }
          else if (s == f.a + 1) {
            claim_v = __builtin_amdgcn_readfirstlane(claim_v);
            if (claim_v < n_tiles && lane < 6) rec_w = reinterpret_cast<const uint32_t*>(p.k_tiles + claim_v)[lane];
          } else if (s == f.a + 2) {
            if (lane < 6) next_lds[lane] = (int)rec_w;
            if (lane == 0) next_lds[8] = claim_v;
          }
        }
        if (s == f.a + 3) {
          const int ns = __builtin_amdgcn_readfirstlane(next_lds[8]);
          have_next = ns < n_tiles;
          if (have_next) {
            next_tile.seq_start = __builtin_amdgcn_readfirstlane(next_lds[0]);
            next_tile.seq_len = __builtin_amdgcn_readfirstlane(next_lds[1]);
            next_tile.origin = __builtin_amdgcn_readfirstlane(next_lds[2]);
            next_tile.seq_id = __builtin_amdgcn_readfirstlane(next_lds[3]);
            const uint32_t lo = __builtin_amdgcn_readfirstlane(next_lds[4]), hi = __builtin_amdgcn_readfirstlane(next_lds[5]);
            next_tile.carry_base = (int64_t)(((uint64_t)hi << 32) | lo);
            slot_idx = ns;                                   // used for the flags of the next tile (read at its start)
          }
        }
        if (!rq_next && rq_left == 0 && have_next && s + 3 >= S) { request_from(next_tile); rq_next = true; }
        if (rq_left > 0 && (s + 3 < n || s + 3 >= S)) { request_rows(); requested = true; }
        // ---- dQ^T (32 columns x 32 rows) += K^T dZ^T over the tile's 128 keys ---------------------------------
        if (do_dq) {
          const int z_base = ChLds::kDz + (kz & 1) * ChLds::kStage + rw_off;
          u32x4 zb[8];
          ch_row_read<0>(zb[0], z_base); ch_row_read<32>(zb[1], z_base); ch_row_read<64>(zb[2], z_base); ch_row_read<96>(zb[3], z_base);
          ch_row_read<128>(zb[4], z_base); ch_row_read<160>(zb[5], z_base); ch_row_read<192>(zb[6], z_base); ch_row_read<224>(zb[7], z_base);
          ch_landed4<4>(zb[0], zb[1], zb[2], zb[3]);
          f32x16 dq0;
#pragma unroll
          for (int r = 0; r < 16; r++) dq0[r] = 0.f;
#pragma unroll
          for (int kk = 0; kk < 4; kk++) dq0 = Elem<T>::mfma(kstat[kk], as_vec8<T>(zb[kk]), dq0);
          ch_landed4<0>(zb[4], zb[5], zb[6], zb[7]);
#pragma unroll
          for (int kk = 4; kk < 8; kk++) dq0 = Elem<T>::mfma(kstat[kk], as_vec8<T>(zb[kk]), dq0);
          // The partial sums of the tiles below join here.  Younger than their loads are only the row requests (6, when
          // any) and, in three slots of a tile, a memory operation of the claim (the wait is then stricter than needed).
          // (Whole-vector bit casts: a bit cast of one element of a vector reads element 0.)
          if (take_in) {
            if (requested) ch_vm_wait<6>(); else ch_vm_wait<0>();
            ch_chain_landed(cin, flag_v);
            flag_seen = max(flag_seen, __builtin_amdgcn_readfirstlane(flag_v));
#pragma unroll
            for (int a4 = 0; a4 < 4; a4++) {
              const f32x4 v = __builtin_bit_cast(f32x4, cin[a4]);
#pragma unroll
              for (int b = 0; b < 4; b++) dq0[4 * a4 + b] += v[b];
            }
          }
          if (J > 0 && kz + 1 < n && !aborted) { ch_flag_request(flag_late, pred_flag); late_pending = true; }
          // dq0[4a + b]: row qz0 + col, column 32c + 8a + 4*half + b.
          if (final_rows) {
#pragma unroll
            for (int a4 = 0; a4 < 4; a4++) {
              const u32x2 o2 = {pack2<T>(dq0[4 * a4] * p.logit_scale, dq0[4 * a4 + 1] * p.logit_scale),
                                pack2<T>(dq0[4 * a4 + 2] * p.logit_scale, dq0[4 * a4 + 3] * p.logit_scale)};
              __builtin_amdgcn_raw_buffer_store_b64(o2, dq_sink.rsrc, dq_voff + 16 * a4, qz0 * dq_sink.stride_bytes, 0);
            }
          } else {
#pragma unroll
            for (int a4 = 0; a4 < 4; a4++) {
              const f32x4 v = {dq0[4 * a4], dq0[4 * a4 + 1], dq0[4 * a4 + 2], dq0[4 * a4 + 3]};
              __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), dqc_rs, dqc_voff + 32 * a4, qz0 * (DH * 4), 0);
            }
          }
        }
        if (out == 0 && s >= 1 && s - 1 < n) bump(cd_stage, kChDoStages);
        if (do_dq) {
          if (!final_rows) { pub_flag = my_flag; pub_count = kz + 1; }
        }
        if (has_z) bump(cq_stage, kChQStages);
        lds_barrier();
      }
      pending = true;
      done_tile = tile;
      have_tile = have_next;
      tile = next_tile;
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);
    if (pub_flag && lane == 0) __hip_atomic_store(pub_flag, pub_count, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    if (pending) store_results(done_tile);
  }
}


template <typename T>
static hipError_t launch_chain_t(const BwdParams& p_in, int max_tiles, hipStream_t stream) {
  const size_t lds_bytes = ChLds::kBytes;
  static std::atomic<uint64_t> lds_done{0};
  int dev = 0, cus = 0;
  hipError_t e = device_cus(&dev, &cus);
  if (e != hipSuccess) return e;
  if ((e = raise_lds_limit(&bwd_chain_kernel<T>, lds_done, dev, lds_bytes)) != hipSuccess) return e;
  BwdParams p = p_in;
  p.wgs_per_head = cus / p.num_heads;
  if (p.wgs_per_head > max_tiles) p.wgs_per_head = max_tiles;
  const dim3 grid((unsigned)(p.wgs_per_head * p.num_heads)), block(kChThreads);
  hipLaunchKernelGGL((bwd_chain_kernel<T>), grid, block, lds_bytes, stream, p);
  return hipGetLastError();
}

// Whether the one-kernel backward can run these parameters: head_dim 128 with 16-byte addressable rows, a head
// count that puts all workgroups of a head on one XCD, at least one workgroup per head, and no fused remainder term.
bool chain_supported(const BwdParams& p) {
  int dev = 0, cus = 0;
  if (device_cus(&dev, &cus) != hipSuccess) return false;
  return p.vec_ok && p.head_dim == 128 && (p.num_heads & 7) == 0 && cus / p.num_heads >= 1 && !p.add_rem;
}

hipError_t launch_bwd_chain(const BwdParams& p, int dtype_is_f16, int max_tiles, hipStream_t stream) {
  return dtype_is_f16 ? launch_chain_t<_Float16>(p, max_tiles, stream) : launch_chain_t<__bf16>(p, max_tiles, stream);
}

}  // namespace sba
