/*
 * libsba — stick-breaking attention for AMD MI355X (gfx950), C ABI.
 *
 * The reference library (speedcell4/stickbreaking-attention) has no FFI: its boundary is a Python
 * operator API whose inner ops are out-parameter functions that launch device kernels on the
 * caller's current stream and return nothing.  Each entry point below replaces one of those inner
 * ops; the Python `torch.autograd.Function`s that sit above them keep the reference's names and
 * signatures.
 *
 * Conventions
 *   - The caller owns every buffer, including the workspace.  The library never allocates, never
 *     synchronises and never throws: work is enqueued on `stream` and the call returns 0 or a
 *     negative SbaStatus.  `sba_strerror` turns a status into text.
 *   - All pointers are device pointers except the SbaArgs struct itself.
 *   - q, k, v, o, do, dq, dk, dv are [batch,] head, token, head_dim tensors addressed through
 *     element strides; the head_dim stride must be 1 (the reference makes the same assumption:
 *     stickbreaking_attention/sb_varlen/sb_varlen_fwd.py:235).
 *   - Packed (varlen) mode: cu_seqlens != NULL, tensors are (H, T, D), batch stride ignored.
 *     Fixed-length mode: cu_seqlens == NULL, tensors are (B, H, L, D) with num_seqs = B and
 *     total_tokens = L.
 *   - Re-entrant and stream-ordered.  The only process-wide state is a per-device cache of device
 *     attributes (compute-unit count, the kernels' LDS limits), filled on first use.  Calls that
 *     share a workspace must be ordered on one stream.
 *   - cu_seqlens is read on the device, so a bad one cannot be reported by the return value.  The
 *     scheduler checks every entry (non-decreasing, within [0, total_tokens], a leading entry equal
 *     to 0) and that the carry buffer is large enough for the actual lengths; on failure it schedules
 *     nothing, all outputs of the call are zero-filled, and the int32 at SBA_STATUS_OFFSET of the
 *     workspace holds SBA_SCHED_BAD_CU_SEQLENS or SBA_SCHED_CARRY_TOO_SMALL (0 otherwise) once the
 *     stream has run.  Rows of the packed token axis at or beyond the last cu_seqlens entry belong to
 *     no sequence; their outputs and gradients are zero-filled.
 */
#ifndef SBA_H
#define SBA_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SBA_VERSION 5

/* Scheduler status word: int32 at this byte offset of the workspace, valid after the stream has run. */
#define SBA_STATUS_OFFSET 8
#define SBA_SCHED_OK 0
#define SBA_SCHED_BAD_CU_SEQLENS 1
#define SBA_SCHED_CARRY_TOO_SMALL 2
#define SBA_CHAIN_TIMEOUT 3        /* one-kernel backward: a workgroup gave up waiting for the key tile below its own */
#define SBA_CHAIN_XCD_MISMATCH 4   /* one-kernel backward: the workgroups of a head did not share an XCD */

/* Size of the static device scratch behind sba_fwd_static. */
#define SBA_STATIC_SCRATCH_BYTES ((size_t)1 << 20)

typedef enum SbaDtype { SBA_BF16 = 0, SBA_F32 = 1, SBA_F16 = 2 } SbaDtype;

typedef enum SbaStatus {
  SBA_OK = 0,
  SBA_ERR_NULL = -1,        /* a required pointer is NULL */
  SBA_ERR_DTYPE = -2,       /* dtype not supported by this build */
  SBA_ERR_HEAD_DIM = -3,    /* head_dim outside 1..128 */
  SBA_ERR_STRIDE = -4,      /* a negative stride (any non-negative head/token/batch stride is accepted; strides and
                               base pointers that are multiples of 16 bytes select the fast kernels) */
  SBA_ERR_ALIGN = -5,       /* a tensor base pointer is not aligned to its element size */
  SBA_ERR_SHAPE = -6,       /* non-positive sizes, total_tokens > 2^30, a negative carry_slots or a flag outside {0, 1} */
  SBA_ERR_WORKSPACE = -7,   /* workspace missing, not 256-byte aligned, or too small (sba_bwd: smaller than one head needs) */
  SBA_ERR_LAUNCH = -8,      /* the HIP runtime rejected a launch (hipGetLastError) */
  SBA_ERR_TOO_LARGE = -9    /* sba_fwd_static: the tile schedule does not fit the library's static scratch */
} SbaStatus;

/* One strided [batch,] head, token, head_dim tensor (strides in elements; head_dim stride is 1). */
typedef struct SbaTensor {
  void* ptr;
  int64_t stride_batch;   /* fixed-length mode only */
  int64_t stride_head;
  int64_t stride_token;
} SbaTensor;

/* One strided [batch,] head, token vector (strides in elements). */
typedef struct SbaVector {
  void* ptr;
  int64_t stride_batch;
  int64_t stride_head;
  int64_t stride_token;
} SbaVector;

typedef struct SbaArgs {
  int32_t dtype;               /* SbaDtype of q, k, v, o, do, dq, dk, dv, rem, drem */
  int32_t head_dim;            /* D, 1..128 */
  int32_t num_heads;           /* H */
  int32_t num_seqs;            /* number of sequences (varlen) or batch size B (fixed) */
  int64_t total_tokens;        /* T (varlen) or L (fixed) */
  int64_t max_seqlen;          /* upper bound on the longest sequence; <= 0 means "unknown" (T is assumed) */
  float logit_scale;           /* z = logit_scale * q.k  (the operator's inv_temp) */
  int32_t attend_current;      /* 0: keys j < i are visible; 1: keys j <= i */

  const void* cu_seqlens;      /* device; cumulative sequence ends; NULL selects fixed-length mode */
  int32_t cu_is_int64;         /* element width of cu_seqlens: 0 = int32, 1 = int64 */
  int32_t cu_has_leading_zero; /* 1: cu_seqlens has num_seqs + 1 entries starting with 0 */

  SbaTensor q, k, v;           /* inputs */
  SbaTensor o;                 /* forward output, dtype of q */
  SbaVector rem;               /* forward output, dtype of q: 1 - sum_j A_ij */
  float* row_stat;             /* forward output, fp32, contiguous (H, T) / (B, H, L): log2(rem).  -inf (never NaN) for a
                                  row whose remainder underflows fp32 -- a few hundred saturated keys do that -- where
                                  the reference keeps a finite neg_log_acc (sb_varlen_fwd.py:156-181); rem is 0 or denormal in both,
                                  and the backward here does not read row_stat except with add_remainder, where only
                                  exp2(row_stat) = rem enters. */
  float* carry;                /* forward output (optional, NULL when no backward will follow) and backward input:
                                  for every row and every 32-key sub-tile the row sweeps, the product of (1 - sigma)
                                  over the keys between that sub-tile and the row.  sba_workspace_bytes sizes it. */

  SbaTensor d_o;               /* backward input: gradient of o */
  SbaVector d_rem;             /* backward input: gradient of rem (ptr may be NULL = zeros) */
  SbaTensor dq, dk, dv;        /* backward outputs */

  void* workspace;             /* device scratch, 256-byte aligned */
  size_t workspace_bytes;
  void* stream;                /* hipStream_t */
  void** trace_events;         /* optional (NULL = off): hipEvent_t handles the library records on `stream` so a
                                  caller can time the kernels separately.  sba_fwd records [0] before and [1] after
                                  the attention kernel (the scheduler kernel runs before [0]); sba_bwd records [0]
                                  before the dQ kernel, [1] between the dQ and dK/dV kernels and [2] after. */
  int32_t add_remainder;       /* 1: the forward writes o + rem * v instead of o, the step every caller of the
                                  reference applies to its outputs (tests/test_varlen.py:103, tests/test_attn.py:67).
                                  The backward then takes d_o as the gradient of that sum and d_rem as the
                                  gradient that reaches rem directly, needs row_stat (as the forward wrote it) as an
                                  input, and returns dv including rem * d_o. */
  int32_t recompute_carry;     /* 0 or 1.  1: the backward does not take `carry` from the forward (which may then be run
                                  with carry = NULL) but rebuilds it in its own workspace from q and k, with the forward
                                  kernel stripped of everything else: the state kept between the passes is then O(tokens)
                                  as in the reference (q, k, v and, with add_remainder, row_stat), at the price of one more
                                  kernel in the backward.  Must be the same in sba_workspace_bytes and sba_bwd.  16-bit
                                  dtypes only.  In sba_fwd (with carry = NULL) it makes the forward's scheduler check the
                                  carry capacity exactly as the backward's will, so that an understated max_seqlen or
                                  carry_slots voids both passes and not the backward alone. */
  int64_t carry_slots;         /* fp32 slots of `carry` (and of the backward's prefix plane) per head.  0: sized from
                                  the bound total_tokens * max_seqlen / 64 (packed mode), which is several times the
                                  need of a ragged batch; a caller that knows the lengths on the host passes
                                  SbaPlan.carry_slots from sba_plan_host for the exact size.  Must be the same in the
                                  forward, the backward and sba_workspace_bytes.  Ignored in fixed-length mode, whose
                                  exact count follows from the shape. */
  int32_t backward_kernels;    /* How sba_bwd computes dq, dk, dv.  1: a dQ kernel and a dK/dV kernel.  2: where it applies
                                  (head_dim 128, 16-bit, 16-byte aligned rows, a head count that is a multiple of 8, no
                                  add_remainder) ONE kernel in which the key tiles of a sequence hand the row prefix
                                  sums and the partial dQ to each other through the L2; the two kernels otherwise.
                                  0: the one kernel where it applies AND was measured to be the faster one: no
                                  sequence longer than 256 tokens, or at most 32 heads with (total_tokens / num_seqs) *
                                  num_heads >= 32768 and max_seqlen * num_heads <= 131072 (in packed mode an overstated
                                  max_seqlen only costs the faster choice).  A head count above 8 that is not a multiple
                                  of 8 is then split where that pays (long sequences): the largest multiple of 8 through
                                  the one kernel, the remaining heads through the two, one pass after the other (with
                                  trace_events, [1] and [2] then bracket the last pass's kernels only).  Must be the
                                  same in sba_workspace_bytes and sba_bwd. */
  int32_t reserved0;
} SbaArgs;

/* What the device scheduler will derive from cu_seqlens, computed on the host from a host copy. */
typedef struct SbaPlan {
  int32_t status;              /* SBA_SCHED_OK or SBA_SCHED_BAD_CU_SEQLENS, as the device scheduler would decide */
  int32_t longest;             /* longest sequence */
  int64_t covered_tokens;      /* tokens that belong to a sequence (the last cu_seqlens entry) */
  int64_t query_tiles;         /* 128-row query tiles over all sequences */
  int64_t key_tiles;           /* 64-key tiles over all sequences */
  int64_t carry_slots;         /* exact fp32 slots per head of the carry buffer: sum over sequences of
                                  256 M (M + 1), M = ceil(length / 128) */
  int64_t pairs;               /* visible (query, key) pairs per head */
} SbaPlan;

/* ABI version of this header (SBA_VERSION) the library was built against. */
int sba_version(void);

/* Text for a status code.  Never NULL. */
const char* sba_strerror(int status);

/*
 * Buffer sizes in bytes: the forward's workspace (tile schedule), the backward's workspace (tile
 * schedules plus the per-(row, key tile) prefix sums that let its two lock-free kernels agree) and the
 * `carry` buffer that travels from the forward to the backward.  Any output pointer may be NULL.
 * Uses dtype, head_dim, num_heads, num_seqs, total_tokens, max_seqlen and cu_seqlens (NULL or not).
 */
int sba_workspace_bytes(const SbaArgs* args, size_t* fwd_bytes, size_t* bwd_bytes, size_t* carry_bytes);

/*
 * Host mirror of the device scheduler's reading of cu_seqlens (same code): validates a HOST copy of
 * cu_seqlens (element width and leading zero as args->cu_is_int64 / cu_has_leading_zero say; num_seqs,
 * total_tokens, attend_current from args) and reports the exact sizes.  Touches no device.  For callers
 * that have the lengths on the host anyway and want exact buffer sizes, and for validating cu_seqlens
 * before a launch.  In fixed-length mode (cu_seqlens_host == NULL) the plan is that of num_seqs
 * sequences of total_tokens.  The reference has no counterpart (its grid is padded to max_seqlens:
 * sb_varlen_fwd.py:475-479, and cu_seqlens is not validated: sb_varlen_fwd.py:283-288).
 */
int sba_plan_host(const SbaArgs* args, const void* cu_seqlens_host, SbaPlan* plan);

/*
 * Forward: fills o, rem, row_stat (and carry when given).
 * Replaces `_compileable_forward` (stickbreaking_attention/sb_varlen/sb_varlen_fwd.py:453-521,
 * custom op "varlen_fwd") and `_compileable_fwd` (stickbreaking_attention/sb_attn/sb_fwd.py:175-251,
 * custom op "attn_fwd"), including the cu_seqlens -> program mapping of `_forward`
 * (sb_varlen_fwd.py:280-294).
 */
int sba_fwd(const SbaArgs* args);

/*
 * The forward for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): the same kernels and results as sba_fwd, with the tile schedule
 * kept in a static device array of the library (SBA_STATIC_SCRATCH_BYTES = 1 MiB per GPU, held until the
 * process ends) instead of a caller workspace.  args->workspace and args->workspace_bytes are ignored; all
 * other buffers (inputs, o, rem, row_stat and, when a backward will follow, carry) are still the caller's.
 * The call allocates nothing and frees nothing.  It returns SBA_ERR_TOO_LARGE when the forward workspace that
 * sba_workspace_bytes reports exceeds the array (roughly total_tokens / 128 + num_seqs > 32000 query tiles).
 * Every call on one GPU shares that GPU's array and rewrites all of it that it reads, so calls need not clear
 * it, but two calls that overlap in time on one GPU (different streams or threads) race: order them.
 * The scheduler status word is not readable by the caller here.
 * No counterpart in the reference, whose launcher allocates its outputs and lock buffers on every call
 * (sb_varlen_fwd.py:417-424, sb_varlen_bwd.py:569-572).
 */
int sba_fwd_static(const SbaArgs* args);

/*
 * Backward: fills dq, dk, dv from q, k, v, carry, d_o, d_rem (and row_stat when add_remainder is set).
 * 16-bit dtypes: every element of dq, dk, dv is written exactly once (no zero-fill needed, no atomics,
 * no locks; bit-reproducible).  SBA_F32: dk and dv are zero-filled by the call and summed with fp32
 * atomics, so their last bits depend on the execution order.
 * Replaces `_compileable_backward` (stickbreaking_attention/sb_varlen/sb_varlen_bwd.py:541-640,
 * custom op "varlen_bwd") and (stickbreaking_attention/sb_attn/sb_bwd.py:207-296, custom op
 * "attn_bwd"), and the `locked_add` accumulation (sb_varlen_bwd.py:11-53).
 * Workspace: bwd_bytes of sba_workspace_bytes runs all heads in one pass.  A smaller workspace is taken as a memory
 * limit: the heads are independent, so the call takes them through in groups of as many as fit, one group after
 * the other on the stream (bit-identical results as long as every pass takes the same form of the backward as
 * the single pass would -- see backward_kernels; equal to rounding otherwise).  The minimum is bwd_bytes of the
 * same arguments with num_heads = 1; below that the call returns SBA_ERR_WORKSPACE before launching anything.
 * With several groups trace_events
 * bracket the whole call but only the last group's dQ / dK/dV split.
 */
int sba_bwd(const SbaArgs* args);

/*
 * How many attention kernels sba_bwd runs for these arguments on the current device when the workspace holds all
 * heads: 1 (the chained kernel, see SbaArgs.backward_kernels) or 2 (dQ, then dK/dV; also for a call whose heads are
 * split between the two forms); a negative SBA_ERR_* for arguments sba_bwd would refuse.  Launches nothing.  For callers that attribute the time between trace_events.
 * No counterpart in the reference (it always runs one kernel with atomics and locks, sb_varlen_bwd.py:541-640).
 */
int sba_bwd_kernels(const SbaArgs* args);

#ifdef __cplusplus
}
#endif
#endif /* SBA_H */
