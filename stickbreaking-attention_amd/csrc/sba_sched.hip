// cu_seqlens -> tile scheduler.
//
// The reference pads every sequence to the longest one: its grid is (num_seqs, H/2, max_len/64 + 1) programs,
// most of which exit idle on a ragged batch (stickbreaking_attention/sb_varlen/sb_varlen_fwd.py:475-479, :294).
// Here a single small kernel reads cu_seqlens on the device (no host synchronisation) and enumerates exactly the
// tiles that exist, so the one launch that follows fills the chip without padding.  Order: sequences longest
// first, and inside a sequence the heaviest tile first (the last query tile / the first key tile).  The tiles of
// one (head, sequence) are therefore resident together and sweep the same K/V (or Q/dO) rows a step or two apart,
// which keeps those rows in the XCD's L2 instead of re-fetching them from HBM, and the launch still ends with
// the cheap tiles of the short sequences.  It also lays out the per-(row, 32-key sub-tile) carries per sequence.
#include "sba_device.hpp"
#include "sba_params.hpp"

namespace sba {

constexpr int kBins = 4096;          // sequence length classes (query tiles per sequence, saturating)
constexpr int kSchedThreads = 1024;

// Returns false for an unusable cu_seqlens entry (see seq_span); the span is then empty.
__device__ __forceinline__ bool seq_bounds(const SchedParams& p, int s, int* start, int* len) {
  if (p.cu == nullptr) { *start = 0; *len = p.fixed_len; return true; }
  return seq_span(p.cu, p.cu_is_int64, p.cu_has_leading_zero, s, p.total_tokens, start, len);
}

// Exclusive prefix sum over bins taken from the heaviest bin downwards; bins[] becomes the start offsets.
__device__ void descending_offsets(int* bins, int* scratch) {
  constexpr int kPer = kBins / kSchedThreads;
  const int t = threadIdx.x;
  // thread t owns bins (kBins-1 - kPer*t) down to (kBins-1 - kPer*t - kPer + 1)
  int local[kPer], sum = 0;
#pragma unroll
  for (int i = 0; i < kPer; i++) { local[i] = bins[kBins - 1 - (kPer * t + i)]; sum += local[i]; }
  scratch[t] = sum;
  __syncthreads();
  for (int d = 1; d < kSchedThreads; d <<= 1) {
    const int v = (t >= d) ? scratch[t - d] : 0;
    __syncthreads();
    scratch[t] += v;
    __syncthreads();
  }
  int base = scratch[t] - sum;
#pragma unroll
  for (int i = 0; i < kPer; i++) { bins[kBins - 1 - (kPer * t + i)] = base; base += local[i]; }
  __syncthreads();
}

__global__ __launch_bounds__(kSchedThreads) void sched_kernel(SchedParams p) {
  if (blockIdx.x > 0) {      // helper workgroups: clear the region the launch was asked to clear
    const int64_t n16 = p.zero_bytes / 16, per = (n16 + gridDim.x - 2) / (gridDim.x - 1);
    const int64_t a = per * (blockIdx.x - 1), b = a + per < n16 ? a + per : n16;
    u32x4* z = reinterpret_cast<u32x4*>(p.zero_fill);
    for (int64_t i = a + threadIdx.x; i < b; i += kSchedThreads) z[i] = u32x4{0u, 0u, 0u, 0u};
    return;
  }
  __shared__ int qbins[kBins];
  __shared__ int kbins[kBins];
  __shared__ int scratch[kSchedThreads];
  __shared__ long long carry_run;
  __shared__ int status;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = kSchedThreads / 64;
  for (int i = threadIdx.x; i < kBins; i += kSchedThreads) { qbins[i] = 0; kbins[i] = 0; }
  if (threadIdx.x == 0) { carry_run = 0; status = kSchedOk; }
  __syncthreads();

  // Pass 1: tiles per length class (class = number of query tiles of the sequence, saturating).  Every entry of
  // cu_seqlens is checked here; the checks are local (each end against its predecessor and the token count), and
  // together they bound the tile counts and carry slots by what the caller's buffers were sized for.
  for (int s = threadIdx.x; s < p.num_seqs; s += kSchedThreads) {
    int start, len;
    if (!seq_bounds(p, s, &start, &len)) status = kSchedBadCu;
    const int nq = (len + kBlockQ - 1) / kBlockQ, nk = (len + p.key_tile - 1) / p.key_tile;
    const int cls = min(nq, kBins - 1);
    if (nq) atomicAdd(&qbins[cls], nq);
    if (nk && p.want_key_tiles) atomicAdd(&kbins[cls], nk);
  }
  __syncthreads();
  if (status != kSchedOk) {      // uniform: nothing is scheduled, every output row is zero-filled as uncovered
    if (threadIdx.x == 0) { p.counts[kCountQ] = 0; p.counts[kCountK] = 0; p.counts[kCountStatus] = status; p.counts[kCountCovered] = 0; }
    if (p.want_key_tiles)
      for (int h = threadIdx.x; h < p.num_heads; h += kSchedThreads) p.head_queue[h] = 0;
    return;
  }
  descending_offsets(qbins, scratch);
  if (p.want_key_tiles) descending_offsets(kbins, scratch);

  // Carry layout: exclusive prefix sum of carry_slots(M_s) over sequences (block-wide, chunked).
  if (p.want_carry_base) {
    for (int s0 = 0; s0 < p.num_seqs; s0 += kSchedThreads) {
      const int s = s0 + threadIdx.x;
      int start = 0, len = 0;
      if (s < p.num_seqs) seq_bounds(p, s, &start, &len);
      const long long mine = carry_slots((len + kBlockQ - 1) / kBlockQ);
      // inclusive scan of `mine` through 64-bit shuffles would need two passes; sequences per chunk are
      // few enough for a shared-memory Hillis-Steele scan on the low/high words kept as long long.
      __shared__ long long sc[kSchedThreads];
      sc[threadIdx.x] = mine;
      __syncthreads();
      for (int d = 1; d < kSchedThreads; d <<= 1) {
        const long long v = (threadIdx.x >= d) ? sc[threadIdx.x - d] : 0;
        __syncthreads();
        sc[threadIdx.x] += v;
        __syncthreads();
      }
      const long long base = carry_run;
      if (s < p.num_seqs) p.carry_base[s] = base + sc[threadIdx.x] - mine;
      __syncthreads();
      if (threadIdx.x == kSchedThreads - 1) carry_run = base + sc[threadIdx.x];
      __syncthreads();
    }
    if (carry_run > p.carry_capacity) {      // uniform: the caller's max_seqlen (or slot count) was too small
      if (threadIdx.x == 0) { p.counts[kCountQ] = 0; p.counts[kCountK] = 0; p.counts[kCountStatus] = kSchedCarryOverflow; p.counts[kCountCovered] = 0; }
      if (p.want_key_tiles)
        for (int h = threadIdx.x; h < p.num_heads; h += kSchedThreads) p.head_queue[h] = 0;
      return;
    }
  }
  __syncthreads();

  // Pass 2: each sequence takes a contiguous range of slots in its class; one wave per sequence.
  for (int s = wave; s < p.num_seqs; s += nwaves) {
    int start, len;
    seq_bounds(p, s, &start, &len);
    const int nq = (len + kBlockQ - 1) / kBlockQ, nk = (len + p.key_tile - 1) / p.key_tile;
    const int cls = min(nq, kBins - 1);
    int qbase = 0, kbase = 0;
    if (lane == 0) {
      if (nq) qbase = atomicAdd(&qbins[cls], nq);
      if (nk && p.want_key_tiles) kbase = atomicAdd(&kbins[cls], nk);
    }
    qbase = __shfl(qbase, 0);
    kbase = __shfl(kbase, 0);
    const int64_t cbase = p.want_carry_base ? p.carry_base[s] : 0;      // written above by this workgroup
    for (int t = lane; t < nq; t += 64) {        // heaviest query tile (the last one) first
      Tile d; d.seq_start = start; d.seq_len = len; d.origin = (nq - 1 - t) * kBlockQ; d.seq_id = s; d.carry_base = cbase;
      p.q_tiles[qbase + t] = d;
    }
    if (p.want_key_tiles) {
      for (int t = lane; t < nk; t += 64) {      // heaviest key tile (the first one) first
        Tile d; d.seq_start = start; d.seq_len = len; d.origin = t * p.key_tile; d.seq_id = s; d.carry_base = cbase;
        p.k_tiles[kbase + t] = d;
      }
    }
  }
  __syncthreads();
  // After the scatter, the lightest bin (work 0) ends at the total count.
  if (threadIdx.x == 0) {
    p.counts[kCountQ] = qbins[0];
    p.counts[kCountK] = p.want_key_tiles ? kbins[0] : 0;
    p.counts[kCountStatus] = kSchedOk;
    int start = 0, len = (int)p.total_tokens;      // fixed-length mode: every row belongs to a sequence
    if (p.cu != nullptr) seq_bounds(p, p.num_seqs - 1, &start, &len);
    p.counts[kCountCovered] = start + len;
  }
  if (p.want_key_tiles)
    for (int h = threadIdx.x; h < p.num_heads; h += kSchedThreads) p.head_queue[h] = 0;

}

hipError_t launch_sched(const SchedParams& p, hipStream_t stream) {
  // One workgroup schedules; with a region to clear, one more per 256 KiB of it (at most 64) clears alongside.
  int helpers = 0;
  if (p.zero_fill && p.zero_bytes > 0) {
    helpers = (int)((p.zero_bytes + (256 << 10) - 1) / (256 << 10));
    if (helpers > 64) helpers = 64;
  }
  hipLaunchKernelGGL(sched_kernel, dim3(1 + helpers), dim3(kSchedThreads), 0, stream, p);
  return hipGetLastError();
}

}  // namespace sba
