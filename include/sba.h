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
 *   - Re-entrant and stream-ordered; no global mutable state.  Calls that share a workspace must
 *     be ordered on one stream.
 */
#ifndef SBA_H
#define SBA_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SBA_VERSION 2

typedef enum SbaDtype { SBA_BF16 = 0, SBA_F32 = 1, SBA_F16 = 2 } SbaDtype;

typedef enum SbaStatus {
  SBA_OK = 0,
  SBA_ERR_NULL = -1,        /* a required pointer is NULL */
  SBA_ERR_DTYPE = -2,       /* dtype not supported by this build */
  SBA_ERR_HEAD_DIM = -3,    /* head_dim outside 1..128 */
  SBA_ERR_STRIDE = -4,      /* a row (token) or head stride is not a multiple of the vector width, or negative */
  SBA_ERR_ALIGN = -5,       /* a tensor base pointer is not 16-byte aligned */
  SBA_ERR_SHAPE = -6,       /* non-positive sizes */
  SBA_ERR_WORKSPACE = -7,   /* workspace missing or smaller than sba_workspace_bytes reports */
  SBA_ERR_LAUNCH = -8       /* the HIP runtime rejected a launch (hipGetLastError) */
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
  float* row_stat;             /* forward output, fp32, contiguous (H, T) / (B, H, L): log2(rem) */
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
  int32_t reserved0;           /* must be 0 */
} SbaArgs;

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
 * Forward: fills o, rem, row_stat (and carry when given).
 * Replaces `_compileable_forward` (stickbreaking_attention/sb_varlen/sb_varlen_fwd.py:453-521,
 * custom op "varlen_fwd") and `_compileable_fwd` (stickbreaking_attention/sb_attn/sb_fwd.py:175-251,
 * custom op "attn_fwd"), including the cu_seqlens -> program mapping of `_forward`
 * (sb_varlen_fwd.py:280-294).
 */
int sba_fwd(const SbaArgs* args);

/*
 * Backward: fills dq, dk, dv from q, k, v, carry, d_o, d_rem (and row_stat when add_remainder is set).  Every element of dq, dk, dv is written
 * exactly once (no zero-fill needed, no atomics, no locks).
 * Replaces `_compileable_backward` (stickbreaking_attention/sb_varlen/sb_varlen_bwd.py:541-640,
 * custom op "varlen_bwd") and (stickbreaking_attention/sb_attn/sb_bwd.py:207-296, custom op
 * "attn_bwd"), and the `locked_add` accumulation (sb_varlen_bwd.py:11-53).
 */
int sba_bwd(const SbaArgs* args);

#ifdef __cplusplus
}
#endif
#endif /* SBA_H */
