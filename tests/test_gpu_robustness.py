"""GPU regression tests around the edges of the hot path: buffers that arrive uninitialised, kernel variants chosen
independently by the forward and the backward, token rows no sequence covers, producer layouts, torch.compile.
Everything goes through the C ABI (via the Python operators) and is compared with the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import sb_oracle as orc
from test_gpu_parity import NAMES, run_varlen, small_case, tol_check

pytestmark = pytest.mark.gpu


@pytest.fixture
def poisoned(monkeypatch):
    """Carry buffer and workspaces filled with NaN bit patterns before every launch: a slot that is read before it
    is written turns into NaN in the outputs instead of passing on whatever the allocator returned."""
    from stickbreaking_attention import _native

    monkeypatch.setattr(_native, "POISON", True)


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("attend_current", [False, True])
def test_poisoned_buffers_lengths_one_past_a_sub_tile(gpu_device, poisoned, D, attend_current):
    # L - 1 a multiple of 32 but not of 128: the last key opens a 32-key sub-tile that only rows beyond the
    # sequence's end would sweep; its per-row scalars are never recorded and must never be used.
    lengths = [33, 65, 97, 161, 193, 225, 289, 34, 1, 96, 128, 129]
    host, dev, cu = small_case(2, D, lengths, torch.bfloat16, seed=41)
    ref = orc.varlen_stream(*host[:3], cu, attend_current=attend_current, do=host[3], drem=host[4], dtype=torch.float64)
    got = run_varlen(*dev[:3], cu.to(gpu_device), lengths, False, attend_current, dev[3], dev[4])
    for n, a, b in zip(NAMES, got, ref):
        tol_check(n, a, b, torch.bfloat16, f"poisoned D={D}")


@pytest.mark.parametrize("which", ["do", "q"])
def test_poisoned_buffers_forward_and_backward_on_different_kernel_variants(gpu_device, poisoned, which):
    # head_dim 128: a tensor at an 8-byte offset sends one pass to the generic 64-key kernels while the other runs the
    # aligned 32-key kernels; the recorded products must serve both.
    lengths = [74, 33, 200, 1, 161]
    host, dev, cu = small_case(2, 128, lengths, torch.bfloat16, seed=42)
    ref = orc.varlen_stream(*host[:3], cu, do=host[3], drem=host[4], dtype=torch.float64)

    def misaligned(t):
        buf = torch.empty(t.numel() + 4, dtype=t.dtype, device=t.device)
        view = buf[4:].view(t.shape)
        view.copy_(t)
        assert view.data_ptr() % 16 == 8
        return view

    q, k, v, do, drem = dev
    if which == "do":
        do = misaligned(do)          # forward aligned, backward generic
        got = run_varlen(q, k, v, cu.to(gpu_device), lengths, False, False, do, drem)
    else:
        from stickbreaking_attention import _native

        # forward generic (q misaligned), backward aligned: drive the two launches directly
        scale = 128 ** -0.5
        cu_d = cu.to(gpu_device)
        o, rem, stat, carry = _native.forward(misaligned(q), k, v, cu_d, False, max(lengths), scale, False, want_carry=True)
        got = [o, rem, *_native.backward(do, drem, q, k, v, carry, cu_d, False, max(lengths), scale, False)]
        torch.cuda.synchronize()
    for n, a, b in zip(NAMES, got, ref):
        tol_check(n, a, b, torch.bfloat16, f"mixed variants ({which} misaligned)")


@pytest.mark.parametrize("dtype,D", [(torch.bfloat16, 128), (torch.bfloat16, 64), (torch.bfloat16, 50), (torch.float32, 64)])
def test_rows_no_sequence_covers_are_zero(gpu_device, poisoned, dtype, D):
    # total_tokens beyond the last cu_seqlens entry (trailing padding of a packed batch): the reference returns zero
    # gradients and rem there (zeros_like: sb_varlen_bwd.py:506-508, sb_varlen_fwd.py:418); so must this.
    lengths = [150, 1, 300]
    pad = 333
    host, dev, cu = small_case(2, D, lengths + [pad], dtype, seed=43)
    cu = cu[:-1]                                  # the last `pad` rows belong to no sequence
    T = sum(lengths)
    ref = orc.varlen_stream(*(t[:, :T] for t in host[:3]), cu, do=host[3][:, :T], drem=host[4][:, :T], dtype=torch.float64)
    got = run_varlen(*dev[:3], cu.to(gpu_device), lengths, False, False, dev[3], dev[4])
    for n, a, b in zip(NAMES, got, ref):
        tol_check(n, a[:, :T], b, dtype, f"covered rows {dtype} D={D}")
        assert (a[:, T:] == 0).all(), f"{n}: rows beyond the last sequence are not zero"


def test_exact_carry_size_from_host_lengths(gpu_device, poisoned):
    # cu_seqlens on the host (or zero_start=True, which copies it once): the carry buffer is sized exactly from the
    # lengths instead of the total_tokens * max_seqlens / 64 bound; results are bit-identical
    from stickbreaking_attention import _native, sb_attn_varlen

    lengths = [1, 700, 64, 3, 129]
    host, dev, cu = small_case(2, 128, lengths, torch.bfloat16, seed=44)
    a = run_varlen(*dev[:3], cu.to(gpu_device), lengths, False, False, dev[3], dev[4])          # device cu: bound
    b = run_varlen(*dev[:3], cu, lengths, False, False, dev[3], dev[4])                          # host cu: exact
    cu0 = torch.cat([torch.zeros(1, dtype=cu.dtype), cu]).to(gpu_device)
    c = run_varlen(*dev[:3], cu0, lengths, True, False, dev[3], dev[4])                          # zero_start: exact
    for x, y, z in zip(a, b, c):
        assert torch.equal(x, y) and torch.equal(x, z)
    plan = _native.plan_host(cu, False, sum(lengths))
    exact = sum(256 * m * (m + 1) for m in (-(-n // 128) for n in lengths))
    assert plan.status == 0 and plan.carry_slots == exact and plan.longest == 700
    assert _native.carry_elems(2, sum(lengths), len(lengths), 700, False, exact) * 4 <= 2 * exact * 4 + 256
    with pytest.raises(ValueError):
        sb_attn_varlen(*dev[:3], torch.tensor([5, 3, 10]), 10, zero_start=False)                # decreasing ends


@pytest.mark.parametrize("dtype,D", [(torch.bfloat16, 128), (torch.float16, 128), (torch.bfloat16, 64), (torch.bfloat16, 72)])
@pytest.mark.parametrize("attend_current", [False, True])
def test_backward_that_rebuilds_the_forward_products(gpu_device, poisoned, dtype, D, attend_current):
    # save_carry=False: nothing but q, k, v is kept between the passes (the reference's saved state, O(L)); the
    # backward rebuilds the per-(row, sub-tile) products in its own workspace.  Same arithmetic, so the same bits,
    # and parity with the oracle like every other path.
    from stickbreaking_attention import sb_attn

    lengths = [33, 500, 1, 129, 257, 64, 97]
    host, dev, cu = small_case(2, D, lengths, dtype, seed=45)
    ref = orc.varlen_stream(*host[:3], cu, attend_current=attend_current, do=host[3], drem=host[4], dtype=torch.float64)
    for cu_arg in (cu.to(gpu_device), cu):                        # carry sized from the bound / exactly
        kept = run_varlen(*dev[:3], cu_arg, lengths, False, attend_current, dev[3], dev[4])
        rebuilt = run_varlen(*dev[:3], cu_arg, lengths, False, attend_current, dev[3], dev[4], save_carry=False)
        for n, a, b, r in zip(NAMES, rebuilt, kept, ref):
            assert torch.equal(a, b), f"{n}: rebuilt products give other bits than kept ones"
            tol_check(n, a, r, dtype, f"rebuilt products {dtype} D={D}")
    # with the remainder term fused, and in the fixed-length operator
    kept = run_varlen(*dev[:3], cu.to(gpu_device), lengths, False, attend_current, dev[3], dev[4], add_remainder=True)
    rebuilt = run_varlen(*dev[:3], cu.to(gpu_device), lengths, False, attend_current, dev[3], dev[4], add_remainder=True,
                         save_carry=False)
    for n, a, b in zip(NAMES, rebuilt, kept):
        assert torch.equal(a, b), f"{n} (fused remainder)"
    g = torch.Generator().manual_seed(46)
    x = [torch.randn(2, 2, 300, D, generator=g).to(dtype).to(gpu_device) for _ in range(4)]
    drem = torch.randn(2, 2, 300, generator=g).to(dtype).to(gpu_device)
    grads = []
    for save in (True, False):
        q, k, v = (t.clone().requires_grad_() for t in x[:3])
        o, rem = sb_attn(q, k, v, attend_current=attend_current, save_carry=save)
        grads.append(torch.autograd.grad([o, rem], [q, k, v], [x[3], drem]))
    torch.cuda.synchronize()
    for a, b in zip(*grads):
        assert torch.equal(a, b)


@pytest.mark.parametrize("dtype,D,save_carry", [(torch.bfloat16, 128, False), (torch.bfloat16, 128, True),
                                                 (torch.bfloat16, 64, False), (torch.float32, 32, True)])
def test_backward_under_a_workspace_limit_goes_head_group_by_head_group(gpu_device, poisoned, dtype, D, save_carry):
    # A backward workspace smaller than the whole call needs: the library processes as many heads at a time as fit.
    # 5 heads under a limit that holds 2: passes of 2, 2 and 1 heads; same bits as the single pass.
    from stickbreaking_attention import _native, sb_attn

    lengths = [200, 33, 1, 385]
    H = 5
    host, dev, cu = small_case(H, D, lengths, dtype, seed=47)
    options = dict(save_carry=save_carry, add_remainder=True)

    def one_head_bytes():
        a = _native._base_args(dev[0][:1], cu.to(gpu_device), False, max(lengths), 1.0, False)
        a.recompute_carry = 0 if (save_carry or dtype == torch.float32) else 1
        import ctypes
        need = ctypes.c_size_t()
        assert _native.lib().sba_workspace_bytes(ctypes.byref(a), None, ctypes.byref(need), None) == 0
        return need.value

    whole = run_varlen(*dev[:3], cu.to(gpu_device), lengths, False, False, dev[3], dev[4], **options)
    g = torch.Generator().manual_seed(48)
    x = [torch.randn(2, H, 300, D, generator=g).to(dtype).to(gpu_device) for _ in range(4)]
    drem = torch.randn(2, H, 300, generator=g).to(dtype).to(gpu_device)

    def fixed_grads():
        q, k, v = (t.clone().requires_grad_() for t in x[:3])
        o, rem = sb_attn(q, k, v, **options)
        out = torch.autograd.grad([o, rem], [q, k, v], [x[3], drem])
        torch.cuda.synchronize()
        return out

    whole_fixed = fixed_grads()
    try:
        _native.set_backward_workspace_limit(int(2.5 * one_head_bytes()))
        limited = run_varlen(*dev[:3], cu.to(gpu_device), lengths, False, False, dev[3], dev[4], **options)
        _native.set_backward_workspace_limit(1)                  # below one head: raised to the minimum, one head per pass
        limited_fixed = fixed_grads()
    finally:
        _native.set_backward_workspace_limit(None)
    for n, a, b in zip(NAMES, limited, whole):
        if dtype == torch.float32 and n in ("dk", "dv"):          # summed with fp32 atomics on this path
            assert torch.allclose(a, b, rtol=1e-5, atol=1e-5), n
        else:
            assert torch.equal(a, b), f"{n}: head groups give other bits than one pass"
    for n, a, b in zip(NAMES[2:], limited_fixed, whole_fixed):
        if dtype == torch.float32 and n in ("dk", "dv"):
            assert torch.allclose(a, b, rtol=1e-5, atol=1e-5), n
        else:
            assert torch.equal(a, b), f"{n} (fixed length)"
    ref = orc.varlen_stream(*host[:3], cu, do=host[3], drem=orc.remainder_drem(host[3], host[4], host[2]).float(),
                            dtype=torch.float32)
    for n, a, b in zip(NAMES, limited, orc.with_remainder(ref, host[2], host[3])):
        tol_check(n, a, b, dtype, "head groups")


@pytest.mark.parametrize("attend_current", [False, True])
def test_token_major_producer_layouts_against_oracle(gpu_device, attend_current):
    """(T, H, D) packed and (B, L, H, D) fixed-length tensors permuted to the operators' layouts, as the reference's
    benchmarks hand them over (benchmarks/varlen.py:44-46, benchmarks/attn.py:14-16): checked against the oracle,
    and o keeps q's strides."""
    from stickbreaking_attention import sb_attn

    lengths = [150, 90, 1, 270]
    host, dev, cu = small_case(4, 128, lengths, torch.bfloat16, seed=45)
    ref = orc.varlen_stream(*host[:3], cu, attend_current=attend_current, do=host[3], drem=host[4], dtype=torch.float64)
    thd = [t.transpose(0, 1).contiguous().transpose(0, 1) for t in dev[:4]]          # (T, H, D) storage
    got = run_varlen(*thd[:3], cu.to(gpu_device), lengths, False, attend_current, thd[3], dev[4])
    assert got[0].stride() == thd[0].stride() and not got[0].is_contiguous()
    for n, a, b in zip(NAMES, got, ref):
        tol_check(n, a, b, torch.bfloat16, "(T,H,D) layout")

    B, L, H, D = 2, 300, 3, 64
    g = torch.Generator().manual_seed(46)
    blhd = [torch.randn(B, L, H, D, generator=g).bfloat16() for _ in range(4)]        # (B, L, H, D) storage
    drem = torch.randn(B, H, L, generator=g).bfloat16()
    q, k, v, do = (t.permute(0, 2, 1, 3) for t in blhd)                                # (B, H, L, D) views
    ref = orc.fixed_stream(q, k, v, attend_current=attend_current, do=do, drem=drem, dtype=torch.float64)
    qd, kd, vd = (t.to(gpu_device).permute(0, 2, 1, 3).requires_grad_() for t in blhd[:3])
    assert not qd.is_contiguous() and qd.stride(-1) == 1
    o, rem = sb_attn(qd, kd, vd, attend_current=attend_current)
    grads = torch.autograd.grad([o, rem], [qd, kd, vd], [blhd[3].to(gpu_device).permute(0, 2, 1, 3), drem.to(gpu_device)])
    assert o.stride() == qd.stride()
    for n, a, b in zip(NAMES, [o, rem, *grads], ref):
        tol_check(n, a, b, torch.bfloat16, "(B,L,H,D) layout")


@pytest.mark.parametrize("backend", ["aot_eager", "inductor"])
def test_torch_compile_against_oracle(gpu_device, backend):
    """The compiled graph (launchers as stickbreaking_attention::* operators, mirroring utils.py:20-40) against the
    ORACLE, not only against eager; `inductor` is the default torch.compile backend."""
    from stickbreaking_attention import sb_attn, sb_attn_varlen

    lengths = [200, 1, 77, 130]
    host, dev, cu = small_case(2, 128, lengths, torch.bfloat16, seed=47)
    cu_d = cu.to(gpu_device)
    ref = orc.varlen_stream(*host[:3], cu, do=host[3], drem=host[4], dtype=torch.float64)

    def varlen_fn(q, k, v, do, drem):
        o, rem = sb_attn_varlen(q, k, v, cu_d, max(lengths), zero_start=False)
        return ((o.float() * do.float()).sum() + (rem.float() * drem.float()).sum()), o, rem

    try:
        compiled = torch.compile(varlen_fn, backend=backend)
        q, k, v = (t.detach().clone().requires_grad_() for t in dev[:3])
        loss, o, rem = compiled(q, k, v, dev[3], dev[4])
        loss.backward()
        torch.cuda.synchronize()
    except Exception as e:       # code generation needs a working compiler toolchain on the box
        if backend == "inductor":
            pytest.skip(f"inductor backend unavailable here: {type(e).__name__}: {str(e)[:200]}")
        raise
    for n, a, b in zip(NAMES, (o.detach(), rem.detach(), q.grad, k.grad, v.grad), ref):
        tol_check(n, a, b, torch.bfloat16, f"compiled ({backend})")

    B, H, L, D = 2, 2, 102, 128
    g = torch.Generator().manual_seed(48)
    qf, kf, vf, dof = (torch.randn(B, H, L, D, generator=g).bfloat16() for _ in range(4))
    dremf = torch.randn(B, H, L, generator=g).bfloat16()
    ref = orc.fixed_stream(qf, kf, vf, do=dof, drem=dremf, dtype=torch.float64)

    def fixed_fn(q, k, v, do, drem):
        o, rem = sb_attn(q, k, v)
        return ((o.float() * do.float()).sum() + (rem.float() * drem.float()).sum()), o, rem

    q, k, v = (t.to(gpu_device).requires_grad_() for t in (qf, kf, vf))
    loss, o, rem = torch.compile(fixed_fn, backend=backend)(q, k, v, dof.to(gpu_device), dremf.to(gpu_device))
    loss.backward()
    torch.cuda.synchronize()
    for n, a, b in zip(NAMES, (o.detach(), rem.detach(), q.grad, k.grad, v.grad), ref):
        tol_check(n, a, b, torch.bfloat16, f"compiled fixed ({backend})")


def test_single_sequence_of_64k_tokens(gpu_device, poisoned):
    """One 65536-token sequence, one head: the length at which the per-(row, 32-key sub-tile) planes the backward works
    from (L^2 / 16 bytes per head each) are the largest buffers in play, sized exactly from the host lengths.  o, rem
    and dq are checked against the row-blocked oracle on the first, a middle and the last 2048 rows (rows are
    independent in those three), dk and dv against it on the last 2048 keys (which only the last 2048 rows see); dk and
    dv as a whole, which sum over all rows, against the library's fp32 vector-ALU path on the same values -- a separate implementation pinned by its own oracle tests -- and the forward outputs against it too."""
    from stickbreaking_attention import _native

    L, D = 65536, 128
    g = torch.Generator().manual_seed(61)
    q, k, v, do = (torch.randn(1, L, D, generator=g).bfloat16() for _ in range(4))
    drem = torch.randn(1, L, generator=g).bfloat16()
    cu = torch.tensor([L], dtype=torch.int32)
    plan = _native.plan_host(cu, False, L)
    assert plan.carry_slots == 256 * 512 * 513 and plan.pairs == L * (L - 1) // 2
    dev = [t.to(gpu_device) for t in (q, k, v, do, drem)]
    got = run_varlen(*dev[:3], cu, [L], False, False, dev[3], dev[4])          # host cu_seqlens: exact buffer sizes
    for t in got:
        assert torch.isfinite(t.float()).all()
    for r0 in (0, 31744, L - 2048):
        ref = orc.stream_rowblocked(q[0], k[0], v[0], do[0], drem[0], rows=(r0, r0 + 2048))
        for n, a, b in zip(NAMES[:3], got[:3], ref[:3]):
            tol_check(n, a[0, r0:r0 + 2048], b[r0:r0 + 2048], torch.bfloat16, f"64k rows {r0}..{r0 + 2047}")
        if r0 == L - 2048:
            # the last 2048 keys are seen by the last 2048 rows only, so this row block's dk and dv are complete for them
            for n, a, b in zip(NAMES[3:], got[3:], ref[3:]):
                tol_check(n, a[0, r0:], b[r0:], torch.bfloat16, f"64k keys {r0}..{L - 1}")
    f32 = run_varlen(*(t.float() for t in dev[:3]), cu, [L], False, False, dev[3].float(), dev[4].float())
    for n, a, b in zip(NAMES, got, f32):
        tol_check(n, a, b.double().cpu(), torch.bfloat16, "64k vs fp32 path")


def test_64k_tokens_four_heads_with_bounded_backward_memory(gpu_device, poisoned):
    """The long-context configuration of the operator: nothing but q, k, v kept between the passes (save_carry=False)
    and the backward's workspace capped at 600 MB, which holds the two per-(row, sub-tile) planes of ONE head at 65536
    tokens (2 x 269 MB) -- the heads go through one at a time.  Same bits as the default mode, which holds 8 planes
    (4 saved by the forward, 4 in the workspace) for the same call."""
    from stickbreaking_attention import _native

    L, D, H = 65536, 128, 4
    g = torch.Generator().manual_seed(62)
    q, k, v, do = (torch.randn(H, L, D, generator=g).bfloat16().to(gpu_device) for _ in range(4))
    drem = torch.randn(H, L, generator=g).bfloat16().to(gpu_device)
    cu = torch.tensor([L], dtype=torch.int32)
    default = run_varlen(q, k, v, cu, [L], False, False, do, drem)
    torch.cuda.empty_cache()
    torch.cuda.reset_peak_memory_stats()
    before = torch.cuda.memory_allocated()
    try:
        _native.set_backward_workspace_limit(600 << 20)
        bounded = run_varlen(q, k, v, cu, [L], False, False, do, drem, save_carry=False)
    finally:
        _native.set_backward_workspace_limit(None)
    peak = torch.cuda.max_memory_allocated() - before
    for n, a, b in zip(NAMES, bounded, default):
        assert torch.equal(a, b), n
    # inputs' clones, outputs, gradients (about 0.45 GB) + the 600 MB workspace; the default mode needs 2.1 GB of planes
    assert peak < 1200 << 20, f"peak {peak >> 20} MiB"
