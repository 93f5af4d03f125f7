"""sba_fwd_static -- the forward entry point that allocates nothing (its tile schedule lives in a static device array
of the library) -- against sba_fwd, through the C ABI: bit-identical o, rem, row_stat and carry on two calls in a
row, the second on a smaller input (the array keeps the first call's contents), then the size limit."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _call(native, entry, q, k, v, cu, max_len, want_carry, with_workspace):
    """One forward through `entry` (sba_fwd or sba_fwd_static) on preallocated outputs; returns them."""
    lib = native.lib()
    fn = getattr(lib, entry)
    H, T, D = q.shape
    o = torch.full_like(q, 7.0)
    rem = torch.full((H, T), 7.0, dtype=q.dtype, device=q.device)
    stat = torch.full((H, T), 7.0, dtype=torch.float32, device=q.device)
    a = native._base_args(q, cu, False, max_len, D ** -0.5, False)
    a.q, a.k, a.v, a.o = (native._tensor(t, False) for t in (q, k, v, o))
    a.rem = native._vector(rem, False)
    a.row_stat = stat.data_ptr()
    need, need_carry = ctypes.c_size_t(0), ctypes.c_size_t(0)
    assert lib.sba_workspace_bytes(ctypes.byref(a), ctypes.byref(need), None, ctypes.byref(need_carry)) == 0
    carry = torch.full((need_carry.value // 4 if want_carry else 0,), float("nan"), dtype=torch.float32, device=q.device)
    if want_carry:
        a.carry = carry.data_ptr()
    ws = None
    if with_workspace:
        ws = torch.empty(need.value, dtype=torch.uint8, device=q.device)
        a.workspace, a.workspace_bytes = ws.data_ptr(), need.value
    status = fn(ctypes.byref(a))
    torch.cuda.synchronize()
    return status, (o, rem, stat, carry), need.value


def _case(lengths, H, D, seed, device):
    g = torch.Generator().manual_seed(seed)
    T = sum(lengths)
    q, k, v = (torch.randn(H, T, D, generator=g).bfloat16().to(device) for _ in range(3))
    cu = torch.tensor(np.cumsum(lengths), dtype=torch.int32, device=device)
    return q, k, v, cu


def test_static_scratch_forward_matches_workspace_forward(gpu_device):
    from stickbreaking_attention import _native as native

    # the larger problem first, then a smaller one whose schedule overwrites only the head of the array
    for lengths, H, D, seed in (([700, 1, 129, 64, 300, 5], 4, 128, 51), ([90, 33], 2, 64, 52)):
        q, k, v, cu = _case(lengths, H, D, seed, gpu_device)
        for want_carry in (True, False):
            st_ws, ref, _ = _call(native, "sba_fwd", q, k, v, cu, max(lengths), want_carry, True)
            st_static, got, _ = _call(native, "sba_fwd_static", q, k, v, cu, max(lengths), want_carry, False)
            assert st_ws == 0 and st_static == 0
            for name, a, b in zip(("o", "rem", "row_stat", "carry"), got, ref):
                assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), f"{name} differs (lengths {lengths})"
            assert not (got[0] == 7).any() and not torch.isnan(got[2]).any()      # every row was written


def test_static_scratch_rejects_what_does_not_fit(gpu_device):
    from stickbreaking_attention import _native as native

    # 40000 single-token sequences: a schedule of ~40000 query tiles (32 bytes each) exceeds the 1 MiB array
    lengths = [1] * 40000
    q, k, v, cu = _case(lengths, 1, 8, 53, gpu_device)
    status, outs, need = _call(native, "sba_fwd_static", q, k, v, cu, 1, False, False)
    assert need > (1 << 20) and status == -9
    assert native.lib().sba_strerror(-9) not in (b"ok", b"unknown status")
    assert (outs[0] == 7).all()                      # nothing was launched
    status, outs, _ = _call(native, "sba_fwd", q, k, v, cu, 1, False, True)
    assert status == 0 and (outs[0] == 0).all() and (outs[1] == 1).all()
