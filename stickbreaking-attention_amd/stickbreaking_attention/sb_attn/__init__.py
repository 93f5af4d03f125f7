"""Fixed-length stick-breaking attention.

Same call surface as the reference's stickbreaking_attention/sb_attn/__init__.py:15-63:
``sb_attn(q, k, v, inv_temp=None, zero_start=True, attend_current=False)`` returns ``(o, rem)`` for
``q, k, v`` of shape (batch, num_heads, seq_len, head_dim).  ``zero_start`` is accepted and ignored, as in
the reference (sb_attn/__init__.py:56).
"""
import math

import torch

from .. import _native


class StickBreakingAttention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, inv_temp, attend_current=False, add_remainder=False, save_carry=True):
        need_grad = any(ctx.needs_input_grad[:3]) and (save_carry or q.dtype == torch.float32)   # fp32 always keeps them
        o, rem, row_stat, carry = _native.forward(q, k, v, None, False, q.size(2), inv_temp, attend_current,
                                                 want_carry=need_grad, add_remainder=add_remainder)
        ctx.save_for_backward(q, k, v, carry, row_stat if add_remainder else None)
        ctx.add_remainder = add_remainder
        ctx.logit_scale = inv_temp
        ctx.attend_current = attend_current
        return o, rem

    @staticmethod
    def backward(ctx, do, drem):
        q, k, v, carry, row_stat = ctx.saved_tensors
        dq, dk, dv = _native.backward(do, drem, q, k, v, carry, None, False, q.size(2),
                                      ctx.logit_scale, ctx.attend_current, row_stat=row_stat, add_remainder=ctx.add_remainder)
        return dq, dk, dv, None, None, None, None


def sb_attn(q, k, v, inv_temp=None, zero_start=True, attend_current=False, add_remainder=False, save_carry=True):
    """``add_remainder=True`` returns ``(o + rem[..., None] * v, rem)`` (what tests/test_attn.py:67 forms from the
    reference's outputs), fused into the kernels' epilogues.  ``save_carry=False`` keeps only q, k, v for the backward,
    which then rebuilds the forward's per-(row, sub-tile) products itself."""
    if inv_temp is None:
        inv_temp = 1 / math.sqrt(q.size(-1))
    return sb_attn_(q, k, v, inv_temp, attend_current=attend_current, add_remainder=add_remainder, save_carry=save_carry)


def sb_attn_(q, k, v, inv_temp, attend_current, add_remainder=False, save_carry=True):
    return StickBreakingAttention.apply(q, k, v, inv_temp, attend_current, bool(add_remainder), bool(save_carry))
