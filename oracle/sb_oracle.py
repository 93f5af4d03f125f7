"""CPU oracle for stick-breaking attention.  TEST INFRASTRUCTURE ONLY.

Nothing that ships may import this module: only ``tests/``, ``__graft_entry__.smoke()`` and
the ``cpu_baseline`` leg of ``bench.py`` use it, and only as the checker or as the timed CPU
baseline -- never as a compute path of the product.

What it restates (citations are into the reference repository):

* ``dense_stickbreaking``      -- stickbreaking_attention/sb_ref.py:8-25 (the definition: logits,
  logsigmoid(z) masked to -1e5, logsigmoid(-z) masked to 0, the L x L ``cum_weight`` contraction,
  exp, ``att @ v`` and ``1 - att.sum(-1)``).
* ``causal_operands``          -- tests/test_varlen.py:14-15 and tests/test_attn.py:13-17 (how the
  callers build ``mask`` = triu(0) / triu(1) for attend_current, and ``cum_weight`` = tril(-1)).
* ``varlen_dense``             -- tests/test_varlen.py:11-28 (packed (H, T, D) tensor split per
  sequence, one dense call each, results concatenated) and
  stickbreaking_attention/sb_varlen/__init__.py:70-77 (``zero_start`` strips a leading 0 of
  ``cu_seqlens``; the default scale is 1/sqrt(D)).
* ``stream_forward`` / ``stream_backward`` -- the same operator written without the O(L^3)
  contraction: a reversed cumulative sum of log(1-sigmoid(z)) along the key axis gives
  log A_ij = log sigmoid(z_ij) + sum_{j<k<i} log(1-sigmoid(z_ik)); the backward is the analytic
  form dz_ij = g_ij - sigmoid(z_ij) * sum_{j'<=j} g_ij', g_ij = A_ij (do_i.v_j - drem_i), which is
  what stickbreaking_attention/sb_varlen/sb_varlen_bwd.py:438-452 evaluates tile by tile.

* ``stream_rowblocked``        -- the streaming form a block of query rows at a time (for 64K-token sequences).
* ``rounding_floor``           -- the streaming form evaluated in float64 with exactly two kinds of rounding
  put back: the weights P and the logit gradient dZ are rounded to the 16-bit input type before they are
  contracted (the reference rounds at the same points: sb_varlen_fwd.py:193 ``p.to(v.dtype)``,
  sb_varlen_bwd.py:449-450 ``dqk.to(k.dtype)``), and the five results are rounded to the 16-bit output type.
  It is the error no implementation with 16-bit matrix operands and 16-bit outputs can avoid; the GPU tests
  compare the kernels' error with it on the same inputs.

Parity status: every function here is pinned by tests/test_oracle_pins.py against checks that do
not retype its formula -- an O(L^3) scalar-loop evaluation of the product form
A_ij = s_ij * prod_{j<k<i}(1 - s_ik) in float64, the q = 0 closed form (A_ij = 2^-(i-j),
rem_i = 2^-i), saturated logits, the identity sum_j A_ij + rem_i = 1, first-row and length-1
behaviour, central finite differences and torch.autograd.gradcheck for the gradients, and
varlen == concatenation of per-sequence calls.  No function is "parity unpinned".  The reference
ships no golden vectors or fixtures for this path (its tests compare live against sb_ref.py), and
sb_ref.py itself was read, not executed.
"""
from __future__ import annotations

import math
from typing import Optional, Sequence, Tuple

import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------------------------
# Dense restatement of the definition (O(L^2) memory, O(L^3) flops through the L x L contraction)
# --------------------------------------------------------------------------------------------
def causal_operands(length: int, attend_current: bool = False, device="cpu", dtype=torch.float32):
    """``mask`` (True = key not visible) and ``cum_weight`` exactly as the reference's callers build
    them: tests/test_varlen.py:14-15, tests/test_attn.py:13-17."""
    ones = torch.ones(length, length, device=device)
    mask = ones.triu(1 if attend_current else 0).bool()
    cum_weight = ones.tril(-1).to(dtype)
    return mask, cum_weight


def dense_stickbreaking(q, k, v, mask, cum_weight, scale: Optional[float] = None):
    """Restatement of sb_ref.py:8-25.  ``q, k, v``: (..., L, D).  Returns ``(att @ v, 1 - sum att)``.

    ``scale`` generalises the reference's hard-coded 1/sqrt(D) (sb_ref.py:12) so that the operator's
    ``inv_temp`` argument (sb_varlen/__init__.py:74-75) can be checked as well."""
    if scale is None:
        scale = 1.0 / math.sqrt(q.shape[-1])
    z = torch.matmul(q, k.transpose(-1, -2)) * scale
    in_dtype = z.dtype
    z = z.float() if z.dtype != torch.float64 else z
    log_take = F.logsigmoid(z).masked_fill(mask, -1e5).to(in_dtype)      # log sigma(z); hidden keys -> exp() == 0
    log_skip = F.logsigmoid(-z).masked_fill(mask, 0).to(in_dtype)        # log(1 - sigma(z)); hidden keys -> factor 1
    # skipped[i, k] = sum_{j > k} log_skip[i, j]   (cum_weight[j, k] = 1 for j > k)
    skipped = torch.einsum("...ij,jk->...ik", log_skip, cum_weight.to(log_skip.dtype))
    att = (log_take + skipped).exp()
    return torch.matmul(att, v), 1 - att.sum(dim=-1)


def _normalise_cu(cu_seqlens, zero_start: bool) -> list:
    cu = [int(x) for x in (cu_seqlens.tolist() if torch.is_tensor(cu_seqlens) else cu_seqlens)]
    if zero_start:
        assert cu[0] == 0, "zero_start=True requires cu_seqlens[0] == 0"   # sb_varlen/__init__.py:71-73
        cu = cu[1:]
    return cu


def varlen_dense(q, k, v, cu_seqlens, scale=None, zero_start=False, attend_current=False):
    """Packed ``(H, T, D)`` inputs; one dense call per sequence as tests/test_varlen.py:11-28 does.
    Returns ``o`` (H, T, D) and ``rem`` (H, T)."""
    ends = _normalise_cu(cu_seqlens, zero_start)
    outs, rems, start = [], [], 0
    for end in ends:
        n = end - start
        mask, cw = causal_operands(n, attend_current, device=q.device, dtype=q.dtype)
        o, r = dense_stickbreaking(q[None, :, start:end], k[None, :, start:end], v[None, :, start:end], mask, cw, scale)
        outs.append(o[0])
        rems.append(r[0])
        start = end
    return torch.cat(outs, 1), torch.cat(rems, 1)


def fixed_dense(q, k, v, scale=None, attend_current=False):
    """Fixed-length ``(B, H, L, D)`` call as tests/test_attn.py:12-20 does."""
    mask, cw = causal_operands(q.shape[-2], attend_current, device=q.device, dtype=q.dtype)
    return dense_stickbreaking(q, k, v, mask, cw, scale)


# --------------------------------------------------------------------------------------------
# Streaming form: no L x L x L contraction, closed-form backward.  (..., L, D) operands.
# --------------------------------------------------------------------------------------------
def _visible(length: int, attend_current: bool, device) -> torch.Tensor:
    i = torch.arange(length, device=device)
    return (i[None, :] <= i[:, None]) if attend_current else (i[None, :] < i[:, None])


def stream_forward(q, k, v, scale=None, attend_current=False, want_att=False):
    """o, rem (and optionally A, sigma) for one (..., L, D) problem in the dtype of the inputs
    (use float64 for a tight check)."""
    if scale is None:
        scale = 1.0 / math.sqrt(q.shape[-1])
    L = q.shape[-2]
    vis = _visible(L, attend_current, q.device)
    z = torch.matmul(q, k.transpose(-1, -2)) * scale
    log_skip = torch.where(vis, -F.softplus(z), torch.zeros_like(z))
    # suffix[i, j] = sum_{k > j} log_skip[i, k]  (hidden keys contribute 0, so k runs to the diagonal)
    suffix = log_skip.flip(-1).cumsum(-1).flip(-1) - log_skip
    log_a = F.logsigmoid(z) + suffix
    att = torch.where(vis, log_a.exp(), torch.zeros_like(z))
    o = torch.matmul(att, v)
    rem = log_skip.sum(-1).exp()          # prod_j (1 - sigma_ij): equals 1 - sum_j A_ij
    if want_att:
        return o, rem, att, torch.sigmoid(z)
    return o, rem


def stream_backward(q, k, v, do, drem, scale=None, attend_current=False):
    """Analytic gradients of ``sum(o * do) + sum(rem * drem)`` w.r.t. q, k, v."""
    if scale is None:
        scale = 1.0 / math.sqrt(q.shape[-1])
    _, _, att, beta = stream_forward(q, k, v, scale, attend_current, want_att=True)
    d_att = torch.matmul(do, v.transpose(-1, -2)) - drem[..., None]       # rem = 1 - sum A  =>  dA -= drem
    g = att * d_att
    dz = g - beta * g.cumsum(-1)
    dz = torch.where(_visible(q.shape[-2], attend_current, q.device), dz, torch.zeros_like(dz))
    dq = torch.matmul(dz, k) * scale
    dk = torch.matmul(dz.transpose(-1, -2), q) * scale
    dv = torch.matmul(att.transpose(-1, -2), do)
    return dq, dk, dv


def stream_rowblocked(q, k, v, do=None, drem=None, scale=None, attend_current=False, block=2048, dtype=torch.float32,
                      rows: Optional[Tuple[int, int]] = None):
    """``stream_forward`` / ``stream_backward`` of ONE (L, D) problem evaluated a block of query rows at a time, so that
    a 64K-token sequence needs (block x L) matrices instead of (L x L): rows are independent in o, rem and dq, and
    dk, dv are sums over row blocks.  Same formulas, same results to rounding (pinned against the unblocked form).
    ``rows = (r0, r1)`` evaluates only those query rows: o, rem, dq are then complete for them (and zero elsewhere),
    dk and dv hold only those rows' contributions."""
    if scale is None:
        scale = 1.0 / math.sqrt(q.shape[-1])
    L, D = q.shape
    q, k, v = (t.to(dtype) for t in (q, k, v))
    o = torch.zeros(L, D, dtype=dtype)
    rem = torch.zeros(L, dtype=dtype)
    grads = None
    if do is not None:
        do = do.to(dtype)
        drem = torch.zeros(L, dtype=dtype) if drem is None else drem.to(dtype)
        grads = [torch.zeros(L, D, dtype=dtype) for _ in range(3)]
    first, last = (0, L) if rows is None else rows
    for r0 in range(first, last, block):
        r1 = min(r0 + block, last)
        nk = min(r1 if attend_current else r1 - 1, L)          # keys any row of the block can see
        if nk <= 0:
            rem[r0:r1] = 1
            continue
        i = torch.arange(r0, r1)[:, None]
        j = torch.arange(nk)[None, :]
        vis = (j <= i) if attend_current else (j < i)
        z = torch.matmul(q[r0:r1], k[:nk].T) * scale
        log_skip = torch.where(vis, -F.softplus(z), torch.zeros_like(z))
        suffix = log_skip.flip(-1).cumsum(-1).flip(-1) - log_skip
        att = torch.where(vis, (F.logsigmoid(z) + suffix).exp(), torch.zeros_like(z))
        o[r0:r1] = torch.matmul(att, v[:nk])
        rem[r0:r1] = log_skip.sum(-1).exp()
        if grads is not None:
            g = att * (torch.matmul(do[r0:r1], v[:nk].T) - drem[r0:r1, None])
            dz = torch.where(vis, g - torch.sigmoid(z) * g.cumsum(-1), torch.zeros_like(z))
            grads[0][r0:r1] = torch.matmul(dz, k[:nk]) * scale
            grads[1][:nk] += torch.matmul(dz.T, q[r0:r1]) * scale
            grads[2][:nk] += torch.matmul(att.T, do[r0:r1])
    if grads is None:
        return o, rem
    return (o, rem, *grads)


def varlen_stream(q, k, v, cu_seqlens, scale=None, zero_start=False, attend_current=False,
                  do=None, drem=None, dtype=torch.float32, heads: Optional[Sequence[int]] = None):
    """Packed (H, T, D) evaluation with the streaming form, one (head, sequence) slice at a time so
    that 16K-token sequences fit in memory.  Inputs are upcast to ``dtype`` (the bf16-rounded values
    are what both sides consume).  Returns (o, rem) or (o, rem, dq, dk, dv), all in ``dtype``.
    ``heads`` restricts the evaluation to a subset of heads (other heads are returned as zeros)."""
    ends = _normalise_cu(cu_seqlens, zero_start)
    H, T, D = q.shape
    heads = range(H) if heads is None else heads
    o = torch.zeros(H, T, D, dtype=dtype)
    rem = torch.zeros(H, T, dtype=dtype)
    grads = None
    if do is not None:
        grads = [torch.zeros(H, T, D, dtype=dtype) for _ in range(3)]
        if drem is None:
            drem = torch.zeros(H, T, dtype=do.dtype)
    for h in heads:
        start = 0
        for end in ends:
            sl = slice(start, end)
            qs, ks, vs = (t[h, sl].to(dtype) for t in (q, k, v))
            os_, rs = stream_forward(qs, ks, vs, scale, attend_current)
            o[h, sl], rem[h, sl] = os_, rs
            if do is not None:
                gq, gk, gv = stream_backward(qs, ks, vs, do[h, sl].to(dtype), drem[h, sl].to(dtype), scale, attend_current)
                grads[0][h, sl], grads[1][h, sl], grads[2][h, sl] = gq, gk, gv
            start = end
    if grads is None:
        return o, rem
    return (o, rem, *grads)


def fixed_stream(q, k, v, scale=None, attend_current=False, do=None, drem=None, dtype=torch.float32):
    """(B, H, L, D) evaluation with the streaming form, one (batch, head) slice at a time."""
    B, H, L, D = q.shape
    o = torch.zeros(B, H, L, D, dtype=dtype)
    rem = torch.zeros(B, H, L, dtype=dtype)
    grads = [torch.zeros(B, H, L, D, dtype=dtype) for _ in range(3)] if do is not None else None
    if do is not None and drem is None:
        drem = torch.zeros(B, H, L, dtype=do.dtype)
    for b in range(B):
        for h in range(H):
            qs, ks, vs = (t[b, h].to(dtype) for t in (q, k, v))
            o[b, h], rem[b, h] = stream_forward(qs, ks, vs, scale, attend_current)
            if do is not None:
                gq, gk, gv = stream_backward(qs, ks, vs, do[b, h].to(dtype), drem[b, h].to(dtype), scale, attend_current)
                grads[0][b, h], grads[1][b, h], grads[2][b, h] = gq, gk, gv
    if grads is None:
        return o, rem
    return (o, rem, *grads)


def dense_backward_autograd(q, k, v, cu_seqlens, do, drem, scale=None, zero_start=False, attend_current=False):
    """Gradients of the dense restatement by autograd, the way tests/test_varlen.py:31-43 obtains
    the reference gradients (``output.backward(do)``), extended with an explicit ``drem``."""
    q, k, v = (t.detach().clone().requires_grad_() for t in (q, k, v))
    o, rem = varlen_dense(q, k, v, cu_seqlens, scale, zero_start, attend_current)
    torch.autograd.backward([o, rem], [do, drem])
    return o.detach(), rem.detach(), q.grad, k.grad, v.grad


def rounding_floor(q, k, v, do, drem, scale=None, attend_current=False, low=torch.bfloat16, with_exact=False):
    """(o, rem, dq, dk, dv) of one (L, D) problem as an implementation would return them that computes everything
    exactly (float64 here) except that P and dZ are rounded to ``low`` before their contractions and the outputs are
    rounded to ``low``.  Inputs are the ``low``-rounded values both sides consume.  ``with_exact`` also returns the
    unrounded float64 results from the same intermediates (what ``stream_forward`` / ``stream_backward`` give)."""
    q, k, v, do, drem = (t.double() for t in (q, k, v, do, drem))
    if scale is None:
        scale = 1.0 / math.sqrt(q.shape[-1])
    rnd = lambda t: t.to(low).double()
    o, rem, att, beta = stream_forward(q, k, v, scale, attend_current, want_att=True)
    g = torch.matmul(do, v.transpose(-1, -2))
    g -= drem[..., None]
    g *= att
    dz = g.cumsum(-1)
    dz *= beta
    del beta
    torch.sub(g, dz, out=dz)
    del g
    dz.masked_fill_(~_visible(q.shape[-2], attend_current, q.device), 0)
    exact = (o, rem, scale * torch.matmul(dz, k), scale * torch.matmul(dz.transpose(-1, -2), q),
             torch.matmul(att.transpose(-1, -2), do)) if with_exact else None
    p16, dz16 = rnd(att), rnd(dz)
    del att, dz
    floor = (rnd(torch.matmul(p16, v)), rnd(rem), rnd(scale * torch.matmul(dz16, k)),
             rnd(scale * torch.matmul(dz16.transpose(-1, -2), q)), rnd(torch.matmul(p16.transpose(-1, -2), do)))
    return (floor, exact) if with_exact else floor


def varlen_rounding_floor(q, k, v, cu_seqlens, do, drem, scale=None, zero_start=False, attend_current=False,
                          heads: Optional[Sequence[int]] = None, low=torch.bfloat16):
    """``rounding_floor`` over a packed (H, T, D) batch, one (head, sequence) slice at a time.  Returns
    ``(floor, exact)``: two (o, rem, dq, dk, dv) tuples in float64 (heads outside ``heads`` are zeros)."""
    ends = _normalise_cu(cu_seqlens, zero_start)
    H, T, D = q.shape
    heads = range(H) if heads is None else heads
    make = lambda: [torch.zeros(H, T, D, dtype=torch.float64), torch.zeros(H, T, dtype=torch.float64)] + \
                   [torch.zeros(H, T, D, dtype=torch.float64) for _ in range(3)]
    floor, exact = make(), make()
    for h in heads:
        start = 0
        for end in ends:
            sl = slice(start, end)
            f, e = rounding_floor(q[h, sl], k[h, sl], v[h, sl], do[h, sl], drem[h, sl], scale, attend_current, low, with_exact=True)
            for dst, src in zip(floor + exact, f + e):
                dst[h, sl] = src
            start = end
    return tuple(floor), tuple(exact)


def with_remainder(outputs, v, do=None):
    """The step callers of the reference apply to its outputs, ``o + rem[..., None] * v``
    (tests/test_varlen.py:103, tests/test_attn.py:67), applied to an (o, rem[, dq, dk, dv]) tuple that was
    evaluated for the gradients ``(do, drem + (do * v).sum(-1))``: y = o + rem v has
    d/d(o) = do, d/d(rem) = drem + do . v, and dv gains rem * do."""
    o, rem = outputs[0], outputs[1]
    vf = v.to(o.dtype)
    y = o + rem[..., None] * vf
    if len(outputs) == 2:
        return y, rem
    dq, dk, dv = outputs[2:]
    return y, rem, dq, dk, dv + rem[..., None] * do.to(o.dtype)


def remainder_drem(do, drem, v):
    """Gradient that reaches ``rem`` when the output is ``o + rem[..., None] * v``."""
    extra = (do.double() * v.double()).sum(-1)
    return extra if drem is None else drem.double() + extra


# --------------------------------------------------------------------------------------------
# Work accounting shared by tests and the benchmark
# --------------------------------------------------------------------------------------------
def visible_pairs(lengths: Sequence[int], heads: int, attend_current: bool = False) -> int:
    """Number of (query, key) pairs the operator touches: H * sum_s L_s (L_s - 1) / 2, plus
    sum_s L_s when the current token is visible."""
    per_head = sum(n * (n - 1) // 2 + (n if attend_current else 0) for n in lengths)
    return heads * per_head
