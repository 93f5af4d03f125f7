"""Packed variable-length stick-breaking attention.

Same call surface as the reference's stickbreaking_attention/sb_varlen/__init__.py:23-81:
``sb_attn_varlen(q, k, v, cu_seqlens, max_seqlens, inv_temp=None, zero_start=True, attend_current=False)``
returns ``(o, rem)`` for ``q, k, v`` of shape (num_heads, total_tokens, head_dim).  ``max_seqlens`` may be
omitted (the reference's README calls the function without it); it only bounds scratch memory here, the
tile schedule is derived from ``cu_seqlens`` on the device.
"""
import math

import torch

from .. import _native


class StickBreakingAttention(torch.autograd.Function):
    """Counterpart of sb_varlen/__init__.py:23-67.  ``cu_seqlens`` here still carries its leading zero when
    ``zero_start`` was requested; the scheduler kernel skips it instead of the host slicing the tensor."""

    @staticmethod
    def forward(ctx, q, k, v, cu_seqlens, max_seqlens, inv_temp, attend_current, leading_zero=False, add_remainder=False):
        need_grad = any(ctx.needs_input_grad[:3])
        o, rem, row_stat, carry = _native.forward(q, k, v, cu_seqlens, leading_zero, max_seqlens, inv_temp,
                                                 attend_current, want_carry=need_grad, add_remainder=add_remainder)
        ctx.save_for_backward(q, k, v, carry, cu_seqlens, row_stat if add_remainder else None)
        ctx.add_remainder = add_remainder
        ctx.logit_scale = inv_temp
        ctx.max_seqlens = max_seqlens
        ctx.attend_current = attend_current
        ctx.leading_zero = leading_zero
        return o, rem

    @staticmethod
    def backward(ctx, do, drem):
        q, k, v, carry, cu_seqlens, row_stat = ctx.saved_tensors
        dq, dk, dv = _native.backward(do, drem, q, k, v, carry, cu_seqlens, ctx.leading_zero,
                                      ctx.max_seqlens, ctx.logit_scale, ctx.attend_current,
                                      row_stat=row_stat, add_remainder=ctx.add_remainder)
        return dq, dk, dv, None, None, None, None, None, None


def sb_attn_varlen(q, k, v, cu_seqlens, max_seqlens=None, inv_temp=None, zero_start=True, attend_current=False,
                   add_remainder=False):
    """``add_remainder=True`` returns ``(o + rem[..., None] * v, rem)``: the combination every caller of the
    reference forms from its outputs (tests/test_varlen.py:103), fused into the kernels' epilogues."""
    cu_seqlens = _native.prepare_cu_seqlens(cu_seqlens, q.device)
    if zero_start:
        assert cu_seqlens[0] == 0          # same check (and host sync) as sb_varlen/__init__.py:71-73
    _native._require_gpu(q, k, v)
    if inv_temp is None:
        inv_temp = 1 / math.sqrt(q.size(-1))
    return StickBreakingAttention.apply(q, k, v, cu_seqlens, max_seqlens, inv_temp, attend_current, bool(zero_start),
                                        bool(add_remainder))


def sb_attn_varlen_(q, k, v, inv_temp, cu_seqlens, max_seqlens, attend_current):
    """Positional form of sb_varlen/__init__.py:80-81: ``cu_seqlens`` holds sequence ends, no leading zero."""
    cu_seqlens = _native.prepare_cu_seqlens(cu_seqlens, q.device)
    return StickBreakingAttention.apply(q, k, v, cu_seqlens, max_seqlens, inv_temp, attend_current, False)
