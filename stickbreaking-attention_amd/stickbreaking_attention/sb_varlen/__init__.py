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
    def forward(ctx, q, k, v, cu_seqlens, max_seqlens, inv_temp, attend_current, leading_zero=False, add_remainder=False,
                carry_slots=0, save_carry=True):
        need_grad = any(ctx.needs_input_grad[:3]) and (save_carry or q.dtype == torch.float32)   # fp32 always keeps them
        o, rem, row_stat, carry = _native.forward(q, k, v, cu_seqlens, leading_zero, max_seqlens, inv_temp,
                                                 attend_current, want_carry=need_grad, add_remainder=add_remainder,
                                                 carry_slots=carry_slots)
        ctx.carry_slots = carry_slots
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
                                      row_stat=row_stat, add_remainder=ctx.add_remainder, carry_slots=ctx.carry_slots)
        return dq, dk, dv, None, None, None, None, None, None, None, None


def sb_attn_varlen(q, k, v, cu_seqlens, max_seqlens=None, inv_temp=None, zero_start=True, attend_current=False,
                   add_remainder=False, save_carry=True):
    """``add_remainder=True`` returns ``(o + rem[..., None] * v, rem)``: the combination every caller of the
    reference forms from its outputs (tests/test_varlen.py:103), fused into the kernels' epilogues.
    ``save_carry=False`` keeps only q, k, v between the forward and the backward, as the reference does, instead of
    the per-(row, 32-key sub-tile) products (L^2 / 16 bytes per head and sequence); the backward rebuilds them with one
    more kernel.  Gradients are bit-identical either way.

    A ``cu_seqlens`` that exists only on the device (a GPU tensor with ``zero_start=False``, or any call under
    ``torch.compile``) cannot be validated on the host.  The scheduler kernel validates it instead, and also checks
    that the sequences fit the scratch sized from ``max_seqlens``; when either check fails it schedules NOTHING:
    ``o``, ``rem`` and all gradients come back as zeros and no error is raised (the reference reads the same entries
    unchecked and would run out of bounds, sb_varlen_fwd.py:283-288).  Set ``SBA_DEBUG_CHECK=1`` to have every launch
    followed by a read of the scheduler's status word (one synchronisation per call) and a ``ValueError`` that says
    which check failed; never understate ``max_seqlens``."""
    # The lengths are on the host when cu_seqlens was given as a CPU tensor, or after the one device-to-host copy that
    # stands in for the reference's `assert cu_seqlens[0] == 0` (sb_varlen/__init__.py:71-73, the same host sync).
    # They are then validated there and the carry buffer is sized exactly; a device-only cu_seqlens is validated by
    # the scheduler kernel and the buffer is sized from the bound total_tokens * max_seqlens / 64.
    cu_host = cu_seqlens if cu_seqlens.device.type == "cpu" else None
    if zero_start:
        if cu_host is None and not torch.compiler.is_compiling():
            cu_host = cu_seqlens.cpu()
        assert (cu_host if cu_host is not None else cu_seqlens)[0] == 0
    _native._require_gpu(q, k, v)
    carry_slots = 0
    if cu_host is not None:
        plan = _native.plan_host(cu_host, bool(zero_start), q.size(1))
        if plan.status != 0:
            raise ValueError("cu_seqlens must be non-decreasing sequence ends within [0, total_tokens]")
        carry_slots = int(plan.carry_slots)
    cu_seqlens = _native.prepare_cu_seqlens(cu_seqlens, q.device)
    if inv_temp is None:
        inv_temp = 1 / math.sqrt(q.size(-1))
    return StickBreakingAttention.apply(q, k, v, cu_seqlens, max_seqlens, inv_temp, attend_current, bool(zero_start),
                                        bool(add_remainder), carry_slots, bool(save_carry))


def sb_attn_varlen_(q, k, v, inv_temp, cu_seqlens, max_seqlens, attend_current):
    """Positional form of sb_varlen/__init__.py:80-81: ``cu_seqlens`` holds sequence ends, no leading zero."""
    cu_seqlens = _native.prepare_cu_seqlens(cu_seqlens, q.device)
    return StickBreakingAttention.apply(q, k, v, cu_seqlens, max_seqlens, inv_temp, attend_current, False)
