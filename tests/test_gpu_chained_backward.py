"""GPU tests of the one-kernel ("chained") backward: `SbaArgs.backward_kernels = 2`, reached through the Python
operators and the C ABI.

The chained kernel must give what the two-kernel backward gives up to the rounding of a different summation order
(dq is summed over key tiles in fp32 in both, but the chained kernel carries the partial sums through memory), and
both must meet the oracle to the bar of test_gpu_parity.py: max-abs error <= 2e-2, or one ulp of the 16-bit output
type where |reference| is large.  The status word of the workspace is read back after every launch (a wait that
ran out, or workgroups of a head on different XCDs, would show there and raise).
"""
import ctypes

import numpy as np
import pytest
import torch

from oracle import sb_oracle as orc
from test_gpu_parity import error_bound, small_case, tol_check

pytestmark = pytest.mark.gpu


@pytest.fixture()
def native_checked():
    from stickbreaking_attention import _native

    saved = (_native.DEBUG_CHECK, _native.BACKWARD_KERNELS)
    _native.DEBUG_CHECK = True
    yield _native
    _native.DEBUG_CHECK, _native.BACKWARD_KERNELS = saved


def grads_varlen(native, mode, dev_t, cu, lengths, attend_current):
    from stickbreaking_attention import sb_attn_varlen

    native.BACKWARD_KERNELS = mode
    q, k, v, do, drem = dev_t
    q, k, v = (t.detach().clone().requires_grad_() for t in (q, k, v))
    o, rem = sb_attn_varlen(q, k, v, cu.to(q.device), max(lengths), zero_start=False, attend_current=attend_current)
    g = torch.autograd.grad([o, rem], [q, k, v], [do, drem])
    torch.cuda.synchronize()
    return [t.detach() for t in g]


CASES = [
    # label, H, lengths
    ("one-row", 8, [1]),
    ("one-block", 8, [32]),
    ("block-plus-one", 8, [33]),
    ("one-tile", 8, [128]),
    ("tile-plus-one", 8, [129]),
    ("ragged", 8, [200, 1, 77, 130]),
    ("two-chains", 8, [1000, 333]),
    ("sixteen-tiles", 8, [2048]),
    ("many-heads", 32, [700, 64, 300]),
    ("long-and-short", 16, [4096, 64, 700]),
    # more key tiles than workgroups of a head, among them tiles of one or two row blocks taken as a workgroup's
    # second or later tile
    ("several-tiles-per-workgroup", 32, [300] * 12),
    ("short-last-tiles", 32, [290, 130, 161, 257, 420, 129, 385, 33, 1, 513, 140, 260, 200, 100, 390]),
]


@pytest.mark.parametrize("label,H,lengths", CASES, ids=[c[0] for c in CASES])
@pytest.mark.parametrize("attend_current", [False, True], ids=["strict", "attend-current"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
def test_chained_backward_matches_oracle_and_two_kernels(gpu_device, native_checked, label, H, lengths, attend_current, dtype):
    if dtype == torch.float16 and sum(lengths) > 1500:
        pytest.skip("fp16 is covered on the short cases")
    host, dev_t, cu = small_case(H, 128, lengths, dtype, seed=len(lengths) + H)
    two = grads_varlen(native_checked, 1, dev_t, cu, lengths, attend_current)
    one = grads_varlen(native_checked, 2, dev_t, cu, lengths, attend_current)
    again = grads_varlen(native_checked, 2, dev_t, cu, lengths, attend_current)
    q, k, v, do, drem = host
    ref = orc.varlen_stream(q, k, v, cu, do=do, drem=drem, dtype=torch.float64, attend_current=attend_current)
    for name, a, b, c, r in zip(("dq", "dk", "dv"), one, two, again, ref[2:]):
        tol_check(name, a, r, dtype, f"chained {label}")
        # no atomics anywhere: a second run gives the same bits
        assert torch.equal(a, c), f"{label}: {name} differs between two runs of the chained kernel"
        # against the two-kernel backward: both within the bound of the oracle, so within twice the bound of each other
        diff = (a.double().cpu() - b.double().cpu()).abs()
        assert (diff <= 2 * error_bound(r.double(), dtype)).all(), f"{label}: {name} chained vs two kernels {diff.max().item():.3e}"


EDGE_LENGTHS = [1, 2, 31, 32, 33, 63, 64, 65, 96, 97, 127, 128, 129, 160, 161, 191, 192, 193, 255, 256, 257, 300, 385, 511, 513, 640,
                769, 1025]


def draw_chained_case(seed):
    rng = np.random.default_rng(9000 + seed)
    n_seq = int(rng.integers(1, 9))
    return dict(
        seed=seed, dtype=[torch.bfloat16, torch.bfloat16, torch.float16][rng.integers(0, 3)], H=int(rng.choice([8, 8, 16, 24])),
        lengths=[int(rng.choice(EDGE_LENGTHS)) if rng.random() < 0.7 else int(rng.integers(1, 1400)) for _ in range(n_seq)],
        attend_current=bool(rng.integers(0, 2)), zero_start=bool(rng.integers(0, 2)), host_cu=bool(rng.integers(0, 2)),
        save_carry=bool(rng.integers(0, 3) > 0), token_major=bool(rng.integers(0, 3) == 0), pad=int(rng.choice([0, 0, 1, 130])),
        qk_std=float(rng.choice([1.0, 1.0, 2.0])), int64_cu=bool(rng.integers(0, 2)),
    )


@pytest.mark.parametrize("seed", range(24))
def test_random_chained_case_against_oracle(gpu_device, native_checked, seed):
    """The seeded sweep of test_gpu_random_sweep.py on the shapes the one-kernel backward applies to (head_dim 128, 8 / 16 / 24
    heads), with that backward forced: ragged lengths around the block and tile edges, attend_current, a leading zero in
    cu_seqlens, cu_seqlens on the host or the device, rebuilt products, token-major strides, rows no sequence covers."""
    from stickbreaking_attention import sb_attn_varlen

    c = draw_chained_case(seed)
    print({k: (str(v) if k == "dtype" else v) for k, v in c.items()}, flush=True)
    dtype, H, lengths, pad = c["dtype"], c["H"], c["lengths"], c["pad"]
    T = sum(lengths)
    g = torch.Generator().manual_seed(9500 + seed)
    q, k, v, do = (torch.randn(H, T + pad, 128, generator=g) for _ in range(4))
    drem = torch.randn(H, T + pad, generator=g)
    q, k = q * c["qk_std"], k * c["qk_std"]
    host = [t.to(dtype) for t in (q, k, v, do, drem)]
    ends = torch.tensor(np.cumsum(lengths), dtype=torch.int64 if c["int64_cu"] else torch.int32)
    cu = torch.cat([torch.zeros(1, dtype=ends.dtype), ends]) if c["zero_start"] else ends

    def to_gpu(t):
        if c["token_major"] and t.dim() == 3:                      # (T, H, D) storage viewed as (H, T, D)
            return t.transpose(0, 1).contiguous().to(gpu_device).transpose(0, 1)
        return t.to(gpu_device)

    native_checked.BACKWARD_KERNELS = 2
    qd, kd, vd = (to_gpu(t).requires_grad_() for t in host[:3])
    o, rem = sb_attn_varlen(qd, kd, vd, cu if c["host_cu"] else cu.to(gpu_device), max(lengths), zero_start=c["zero_start"],
                            attend_current=c["attend_current"], save_carry=c["save_carry"])
    grads = torch.autograd.grad([o, rem], [qd, kd, vd], [to_gpu(host[3]), host[4].to(gpu_device)])
    torch.cuda.synchronize()
    cov = [t[:, :T] for t in host]
    ref = orc.varlen_stream(*cov[:3], ends, attend_current=c["attend_current"], do=cov[3], drem=cov[4], dtype=torch.float64)
    for name, a, b in zip(("o", "rem", "dq", "dk", "dv"), (o, rem, *grads), ref):
        tol_check(name, a[:, :T], b, dtype, f"chained sweep {seed}")
        if pad:
            assert (a[:, T:] == 0).all(), f"{name}: rows no sequence covers must be zero"


def test_chained_backward_fixed_length(gpu_device, native_checked):
    """`sb_attn` (batch, head, token, head_dim): the chain buffers are addressed per batch element."""
    from stickbreaking_attention import sb_attn

    B, H, L, D = 3, 8, 300, 128
    g = torch.Generator().manual_seed(5)
    q, k, v, do = (torch.randn(B, H, L, D, generator=g).bfloat16() for _ in range(4))
    drem = torch.randn(B, H, L, generator=g).bfloat16()
    out = {}
    for mode in (1, 2):
        native_checked.BACKWARD_KERNELS = mode
        qd, kd, vd = (t.to(gpu_device).requires_grad_() for t in (q, k, v))
        o, rem = sb_attn(qd, kd, vd)
        out[mode] = torch.autograd.grad([o, rem], [qd, kd, vd], [do.to(gpu_device), drem.to(gpu_device)])
        torch.cuda.synchronize()
    for b in range(B):
        cu = torch.tensor([L], dtype=torch.int32)
        ref = orc.varlen_stream(q[b], k[b], v[b], cu, do=do[b], drem=drem[b], dtype=torch.float64)
        for name, a, r in zip(("dq", "dk", "dv"), out[2], ref[2:]):
            tol_check(name, a[b], r, torch.bfloat16, f"chained fixed-length batch {b}")


def test_chained_backward_in_head_groups(gpu_device, native_checked):
    """A backward workspace too small for all heads: the heads go through in groups, each group a chained launch of its
    own (its own flags, tags and XCD map); same bits as the single launch."""
    lengths, H = [1500, 700], 16
    host, dev_t, cu = small_case(H, 128, lengths, torch.bfloat16, seed=77)
    whole = grads_varlen(native_checked, 2, dev_t, cu, lengths, False)
    q = dev_t[0]
    a = native_checked._base_args(q, cu.to(q.device), False, max(lengths), 1.0, False)
    for f in ("q", "k", "v", "d_o", "dq", "dk", "dv"):
        setattr(a, f, native_checked._tensor(q, False))
    need = native_checked._workspace_bytes(a)[1]
    try:
        native_checked.set_backward_workspace_limit(int(need * 0.6))          # two groups of 8 heads
        grouped = grads_varlen(native_checked, 2, dev_t, cu, lengths, False)
    finally:
        native_checked.set_backward_workspace_limit(None)
    for name, x, y in zip(("dq", "dk", "dv"), grouped, whole):
        assert torch.equal(x, y), name


def test_head_count_not_a_multiple_of_eight_is_split(gpu_device, native_checked):
    """12 heads (the reference's benchmark shape), left to the library: the first 8 go through the one-kernel backward,
    the other 4 through the two kernels, one pass after the other -- the same bits as the two parts run on their own."""
    lengths, H = [12288], 12                 # long enough for the split to pay (and so to be chosen)
    host, dev_t, cu = small_case(H, 128, lengths, torch.bfloat16, seed=78)
    auto = grads_varlen(native_checked, 0, dev_t, cu, lengths, False)
    first = grads_varlen(native_checked, 2, [t[:8] for t in dev_t], cu, lengths, False)
    rest = grads_varlen(native_checked, 1, [t[8:] for t in dev_t], cu, lengths, False)
    two = grads_varlen(native_checked, 1, dev_t, cu, lengths, False)
    for name, a, b, c, d in zip(("dq", "dk", "dv"), auto, first, rest, two):
        assert torch.equal(a[:8], b), f"{name}: heads 0..7 differ from the chained backward on those heads"
        assert torch.equal(a[8:], c), f"{name}: heads 8..11 differ from the two-kernel backward on those heads"
        assert not torch.equal(a[:8], d[:8]) or name == "dv"       # (the split really took the other kernel for them)


def test_benchmark_shape_all_heads_agree_with_two_kernels_and_repeat(gpu_device, native_checked):
    """The benchmark configuration (32 heads, 32768 tokens, 25 sequences) through both backwards on ALL heads -- every
    workgroup of every XCD, several tiles per workgroup, where the oracle of test_gpu_parity.py covers six heads: two
    independent orders of summation must agree to twice the bound each has against the oracle, and the one-kernel
    backward must repeat its own bits."""
    import bench

    inp = bench.make_inputs("c3", gpu_device)
    lengths = inp["lengths"]
    dev_t = [inp[n] for n in ("q", "k", "v", "do", "drem")]
    cu = inp["cu"].cpu()
    assert not inp["zero_start"]
    two = grads_varlen(native_checked, 1, dev_t, cu, lengths, False)
    one = grads_varlen(native_checked, 2, dev_t, cu, lengths, False)
    again = grads_varlen(native_checked, 2, dev_t, cu, lengths, False)
    for name, a, b, c in zip(("dq", "dk", "dv"), one, two, again):
        assert torch.isfinite(a.float()).all(), name
        assert torch.equal(a, c), f"{name} differs between two runs of the chained kernel"
        worst = -float("inf")
        for h in range(0, a.shape[0], 8):                     # in slices, to bound the fp32 temporaries
            x, y = a[h:h + 8].float(), b[h:h + 8].float()
            excess = (x - y).abs() - 2 * torch.maximum(torch.full_like(y, 2e-2), y.abs() * 2.0 ** -7)
            worst = max(worst, excess.max().item())
        print(f"c3 all heads, chained vs two kernels, {name}: largest excess over twice the bound {worst:.3e}", flush=True)
        assert worst <= 0.0, f"{name}: chained and two-kernel backward differ by {worst:.3e} beyond twice the bound"


def _bwd_kernels(native, q, lengths, backward_kernels, add_remainder=False, max_seqlen=None):
    """`sba_bwd_kernels` for a packed call on tensors shaped like `q` (nothing is launched)."""
    cu = torch.tensor(np.cumsum(lengths), dtype=torch.int32, device=q.device)
    native.BACKWARD_KERNELS = backward_kernels
    a = native._base_args(q, cu, False, max_seqlen or max(lengths), 1.0, False)
    a.add_remainder = 1 if add_remainder else 0
    for f in ("q", "k", "v", "d_o", "dq", "dk", "dv"):
        setattr(a, f, native._tensor(q, False))
    return native.lib().sba_bwd_kernels(ctypes.byref(a))


def test_which_backward_runs(gpu_device, native_checked):
    """The one-kernel backward runs only where it applies; left to the library (0) only where it is the faster one."""
    n = native_checked
    q = torch.zeros(8, 4096, 128, dtype=torch.bfloat16, device=gpu_device)
    assert _bwd_kernels(n, q, [4096], 2) == 1
    assert _bwd_kernels(n, q, [4096], 1) == 2
    assert _bwd_kernels(n, q, [4096], 0) == 1                                        # mean x heads = 32768, longest x heads <= 131072
    assert _bwd_kernels(n, q, [1024] * 4, 0) == 2                                    # short sequences: two kernels
    assert _bwd_kernels(n, q, [1024] * 4, 2) == 1
    assert _bwd_kernels(n, q, [128] * 32, 0) == 1                                    # nothing to hand over: one kernel
    assert _bwd_kernels(n, q, [4096], 2, add_remainder=True) == 2
    assert _bwd_kernels(n, q[:7], [4096], 2) == 2                                    # 7 heads
    assert _bwd_kernels(n, q[..., :64], [4096], 2) == 2                              # head_dim 64
    assert _bwd_kernels(n, q.float(), [4096], 2) == 2                                # fp32
    big = torch.zeros(32, 8192, 128, dtype=torch.bfloat16, device=gpu_device)
    assert _bwd_kernels(n, big, [8192], 0) == 2                                      # 8192 * 32 > 131072
    assert _bwd_kernels(n, big, [4096, 4096], 0) == 1
    assert _bwd_kernels(n, big, [4096, 4096], 0, max_seqlen=8192) == 2               # an overstated bound decides
    assert _bwd_kernels(n, big, [8192], 2) == 1
    wide = torch.zeros(64, 2048, 128, dtype=torch.bfloat16, device=gpu_device)
    assert _bwd_kernels(n, wide, [2048], 0) == 2                                     # more than 32 heads
    assert _bwd_kernels(n, wide, [128] * 16, 0) == 1
