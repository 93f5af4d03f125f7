"""The device-side void path, through the C ABI: a `cu_seqlens` that exists only on the device and is not a
non-decreasing sequence of ends within [0, total_tokens], or sequences that do not fit the carry capacity derived
from an understated max_seqlen / carry_slots.  The scheduler kernel then schedules nothing: the call returns 0, the
int32 at SBA_STATUS_OFFSET of the workspace says why, and every output of the call is zero-filled (instead of tiles
addressed from bad offsets).  Forward and backward, bf16 and fp32, and the chained backward.
"""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

BAD_CU, CARRY_TOO_SMALL = 1, 2


def _forward(native, q, k, v, cu, max_len, carry_slots, want_carry, recompute=False):
    lib = native.lib()
    H, T, D = q.shape
    o = torch.full_like(q, 7.0)
    rem = torch.full((H, T), 7.0, dtype=q.dtype, device=q.device)
    stat = torch.full((H, T), 7.0, dtype=torch.float32, device=q.device)
    a = native._base_args(q, cu, False, max_len, D ** -0.5, False, carry_slots)
    a.q, a.k, a.v, a.o = (native._tensor(t, False) for t in (q, k, v, o))
    a.rem = native._vector(rem, False)
    a.row_stat = stat.data_ptr()
    a.recompute_carry = 1 if recompute else 0
    need, need_carry = ctypes.c_size_t(0), ctypes.c_size_t(0)
    assert lib.sba_workspace_bytes(ctypes.byref(a), ctypes.byref(need), None, ctypes.byref(need_carry)) == 0
    carry = torch.full((need_carry.value // 4 if want_carry else 0,), float("nan"), dtype=torch.float32, device=q.device)
    if want_carry:
        a.carry = carry.data_ptr()
    ws = torch.full((need.value,), 0xFF, dtype=torch.uint8, device=q.device)
    a.workspace, a.workspace_bytes = ws.data_ptr(), need.value
    ret = lib.sba_fwd(ctypes.byref(a))
    torch.cuda.synchronize()
    status = int(ws[native.STATUS_OFFSET:native.STATUS_OFFSET + 4].view(torch.int32).item())
    return ret, status, (o, rem, stat), carry


def _backward(native, q, k, v, cu, max_len, carry_slots, carry, backward_kernels):
    lib = native.lib()
    H, T, D = q.shape
    do = torch.ones_like(q)
    drem = torch.ones((H, T), dtype=q.dtype, device=q.device)
    grads = [torch.full_like(q, 7.0) for _ in range(3)]
    saved = native.BACKWARD_KERNELS
    native.BACKWARD_KERNELS = backward_kernels
    try:
        a = native._base_args(q, cu, False, max_len, D ** -0.5, False, carry_slots)
    finally:
        native.BACKWARD_KERNELS = saved
    a.q, a.k, a.v, a.d_o, a.dq, a.dk, a.dv = (native._tensor(t, False) for t in (q, k, v, do, *grads))
    a.d_rem = native._vector(drem, False)
    if carry is None:
        a.recompute_carry = 1
    else:
        a.carry = carry.data_ptr()
    need = ctypes.c_size_t(0)
    assert lib.sba_workspace_bytes(ctypes.byref(a), None, ctypes.byref(need), None) == 0
    ws = torch.full((need.value,), 0xFF, dtype=torch.uint8, device=q.device)
    a.workspace, a.workspace_bytes = ws.data_ptr(), need.value
    ret = lib.sba_bwd(ctypes.byref(a))
    torch.cuda.synchronize()
    status = int(ws[native.STATUS_OFFSET:native.STATUS_OFFSET + 4].view(torch.int32).item())
    return ret, status, grads


def _inputs(H, T, D, dtype, device):
    g = torch.Generator().manual_seed(71)
    return [torch.randn(H, T, D, generator=g).to(dtype).to(device) for _ in range(3)]


@pytest.mark.parametrize("dtype,H,D,kernels", [(torch.bfloat16, 2, 64, 1), (torch.float32, 2, 64, 1), (torch.bfloat16, 8, 128, 2)],
                         ids=["bf16", "f32", "bf16-chained"])
@pytest.mark.parametrize("ends", [[200, 100, 300], [200, 400], [-5, 300]], ids=["decreasing", "beyond-total", "negative"])
def test_bad_device_cu_seqlens_voids_the_call(gpu_device, dtype, H, D, kernels, ends):
    from stickbreaking_attention import _native as native

    T = 300
    q, k, v = _inputs(H, T, D, dtype, gpu_device)
    cu = torch.tensor(ends, dtype=torch.int32, device=gpu_device)
    ret, status, outs, carry = _forward(native, q, k, v, cu, T, 0, want_carry=True)
    assert ret == 0 and status == BAD_CU
    for name, t in zip(("o", "rem", "row_stat"), outs):
        assert (t == 0).all(), f"forward {name} is not zero-filled"
    ret, status, grads = _backward(native, q, k, v, cu, T, 0, carry, kernels)
    assert ret == 0 and status == BAD_CU
    for name, t in zip(("dq", "dk", "dv"), grads):
        assert (t == 0).all(), f"backward {name} is not zero-filled"


@pytest.mark.parametrize("dtype,H,D,kernels", [(torch.bfloat16, 2, 64, 1), (torch.float32, 2, 64, 1), (torch.bfloat16, 8, 128, 2)],
                         ids=["bf16", "f32", "bf16-chained"])
@pytest.mark.parametrize("how", ["max_seqlen", "carry_slots"])
def test_understated_capacity_voids_the_call(gpu_device, dtype, H, D, kernels, how):
    from stickbreaking_attention import _native as native

    # one sequence of 4000 tokens among short ones: needs 256 * 32 * 33 carry slots per head for that sequence alone
    lengths = [4000, 50, 46]
    T = sum(lengths)
    q, k, v = _inputs(H, T, D, dtype, gpu_device)
    cu = torch.tensor([4000, 4050, 4096], dtype=torch.int32, device=gpu_device)
    max_len, slots = (64, 0) if how == "max_seqlen" else (4000, 1024)      # bound T * 64 / 64 + 6 T + 512 B, or 1024 slots
    ret, status, outs, carry = _forward(native, q, k, v, cu, max_len, slots, want_carry=True)
    assert ret == 0 and status == CARRY_TOO_SMALL
    for name, t in zip(("o", "rem", "row_stat"), outs):
        assert (t == 0).all(), f"forward {name} is not zero-filled"
    ret, status, grads = _backward(native, q, k, v, cu, max_len, slots, carry, kernels)
    assert ret == 0 and status == CARRY_TOO_SMALL
    for name, t in zip(("dq", "dk", "dv"), grads):
        assert (t == 0).all(), f"backward {name} is not zero-filled"
    if dtype != torch.float32:
        # nothing kept between the passes: the forward (told that the backward will rebuild the products) and the
        # backward make the same check, so both are void -- not a correct forward followed by zero gradients
        ret, status, outs, _ = _forward(native, q, k, v, cu, max_len, slots, want_carry=False, recompute=True)
        assert ret == 0 and status == CARRY_TOO_SMALL and all((t == 0).all() for t in outs)
        ret, status, grads = _backward(native, q, k, v, cu, max_len, slots, None, kernels)
        assert ret == 0 and status == CARRY_TOO_SMALL and all((t == 0).all() for t in grads)
    # the same call with honest figures stands
    ret, status, outs, _ = _forward(native, q, k, v, cu, 4000, 0, want_carry=True)
    assert ret == 0 and status == 0 and not (outs[1] == 0).all()


def test_python_operators_raise_on_a_void_schedule(gpu_device):
    """With SBA_DEBUG_CHECK (on in these tests) the operators read the status word back and raise."""
    from stickbreaking_attention import _native as native, sb_attn_varlen

    assert native.DEBUG_CHECK
    q, k, v = _inputs(2, 300, 64, torch.bfloat16, gpu_device)
    cu = torch.tensor([200, 100, 300], dtype=torch.int32, device=gpu_device)
    with pytest.raises(ValueError, match="cu_seqlens"):
        sb_attn_varlen(q, k, v, cu, 300, zero_start=False)
    cu = torch.tensor([4000, 4050, 4096], dtype=torch.int32, device=gpu_device)
    q, k, v = (t.requires_grad_() for t in _inputs(2, 4096, 64, torch.bfloat16, gpu_device))
    with pytest.raises(ValueError, match="carry"):
        sb_attn_varlen(q, k, v, cu, 64, zero_start=False, save_carry=False)      # void in the forward already
