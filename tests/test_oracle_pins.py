"""Pins for the CPU oracle: every check here is independent of the oracle's own formulas
(scalar product-form loops, closed forms, invariants, finite differences)."""
import math

import numpy as np
import pytest
import torch

from oracle import sb_oracle as orc


def _sigmoid(x):
    return 1.0 / (1.0 + math.exp(-x))


def brute_force(q, k, v, scale, attend_current):
    """A_ij = s_ij * prod_{j<k<i (or <=i)} (1 - s_ik) with plain Python floats (float64), O(L^3)."""
    L, D = q.shape
    A = np.zeros((L, L))
    for i in range(L):
        hi = i + 1 if attend_current else i          # visible keys: j < hi
        for j in range(hi):
            s = _sigmoid(scale * float(np.dot(q[i], k[j])))
            prod = 1.0
            for kk in range(j + 1, hi):
                prod *= 1.0 - _sigmoid(scale * float(np.dot(q[i], k[kk])))
            A[i, j] = s * prod
    o = A @ v
    rem = 1.0 - A.sum(-1)
    return A, o, rem


def brute_loss(q, k, v, do, drem, scale, attend_current):
    _, o, rem = brute_force(q, k, v, scale, attend_current)
    return float((o * do).sum() + (rem * drem).sum())


@pytest.mark.parametrize("attend_current", [False, True])
@pytest.mark.parametrize("L,D", [(1, 4), (2, 4), (7, 8), (13, 16)])
def test_forward_matches_product_form(L, D, attend_current):
    rng = np.random.default_rng(L * 100 + D)
    q, k, v = (rng.standard_normal((L, D)) * 1.5 for _ in range(3))
    scale = 0.37
    A, o, rem = brute_force(q, k, v, scale, attend_current)
    tq, tk, tv = (torch.tensor(x, dtype=torch.float64) for x in (q, k, v))
    mask, cw = orc.causal_operands(L, attend_current, dtype=torch.float64)
    od, rd = orc.dense_stickbreaking(tq, tk, tv, mask, cw, scale)
    os_, rs, att, _ = orc.stream_forward(tq, tk, tv, scale, attend_current, want_att=True)
    np.testing.assert_allclose(od.numpy(), o, atol=1e-12)
    np.testing.assert_allclose(rd.numpy(), rem, atol=1e-12)
    np.testing.assert_allclose(os_.numpy(), o, atol=1e-12)
    np.testing.assert_allclose(rs.numpy(), rem, atol=1e-12)
    np.testing.assert_allclose(att.numpy(), A, atol=1e-12)


def test_default_scale_is_inverse_sqrt_d():
    # sb_ref.py:12 divides by sqrt(D); a wrong default (e.g. 1/D) must fail here.
    rng = np.random.default_rng(3)
    L, D = 6, 16
    q, k, v = (rng.standard_normal((L, D)) for _ in range(3))
    _, o, rem = brute_force(q, k, v, 1 / math.sqrt(D), False)
    tq, tk, tv = (torch.tensor(x) for x in (q, k, v))
    mask, cw = orc.causal_operands(L, dtype=torch.float64)
    od, rd = orc.dense_stickbreaking(tq, tk, tv, mask, cw)
    os_, rs = orc.stream_forward(tq, tk, tv)
    np.testing.assert_allclose(od.numpy(), o, atol=1e-12)
    np.testing.assert_allclose(os_.numpy(), o, atol=1e-12)
    np.testing.assert_allclose(rd.numpy(), rem, atol=1e-12)
    np.testing.assert_allclose(rs.numpy(), rem, atol=1e-12)


@pytest.mark.parametrize("attend_current", [False, True])
def test_zero_query_closed_form(attend_current):
    # q = 0  =>  sigma = 1/2 everywhere: A_ij = 2^-(i-j) (2^-(i-j+1) with the current token), rem_i = 2^-i (2^-(i+1)).
    L, D = 20, 8
    torch.manual_seed(0)
    k = torch.randn(L, D, dtype=torch.float64)
    v = torch.randn(L, D, dtype=torch.float64)
    q = torch.zeros(L, D, dtype=torch.float64)
    i = torch.arange(L, dtype=torch.float64)
    shift = 1 if attend_current else 0
    expect_rem = 2.0 ** -(i + shift)
    expect_o = torch.zeros(L, D, dtype=torch.float64)
    for a in range(L):
        for b in range(a + shift):
            expect_o[a] += 2.0 ** -(a - b + shift) * v[b]
    for fn in ("dense", "stream"):
        if fn == "dense":
            mask, cw = orc.causal_operands(L, attend_current, dtype=torch.float64)
            o, rem = orc.dense_stickbreaking(q, k, v, mask, cw)
        else:
            o, rem = orc.stream_forward(q, k, v, attend_current=attend_current)
        torch.testing.assert_close(rem, expect_rem, atol=1e-13, rtol=0)
        torch.testing.assert_close(o, expect_o, atol=1e-13, rtol=0)


def test_saturated_logits():
    # z -> +inf: all mass on the previous token (o_i = v_{i-1}, rem -> 0); z -> -inf: no mass (o = 0, rem = 1).
    L, D = 9, 4
    v = torch.arange(L * D, dtype=torch.float32).reshape(L, D)
    ones = torch.ones(L, D)
    o, rem = orc.stream_forward(ones, 40 * ones, v, scale=1.0)
    assert torch.equal(o[0], torch.zeros(D)) and rem[0] == 1
    torch.testing.assert_close(o[1:], v[:-1], atol=1e-6, rtol=0)
    assert rem[1:].abs().max() < 1e-30
    o, rem = orc.stream_forward(ones, -40 * ones, v, scale=1.0)
    assert o.abs().max() < 1e-30 * v.max() * L + 1e-20
    torch.testing.assert_close(rem, torch.ones(L), atol=1e-6, rtol=0)
    mask, cw = orc.causal_operands(L)
    od, rd = orc.dense_stickbreaking(ones, 40 * ones, v, mask, cw, 1.0)
    torch.testing.assert_close(od[1:], v[:-1], atol=1e-5, rtol=0)
    assert rd[0] == 1


@pytest.mark.parametrize("attend_current", [False, True])
def test_mass_conservation_and_first_row(attend_current):
    torch.manual_seed(1)
    L, D = 65, 16
    q, k, v = (torch.randn(3, L, D, dtype=torch.float64) for _ in range(3))
    o, rem, att, beta = orc.stream_forward(q, k, v, attend_current=attend_current, want_att=True)
    torch.testing.assert_close(att.sum(-1) + rem, torch.ones(3, L, dtype=torch.float64), atol=1e-12, rtol=0)
    assert (att >= 0).all() and (rem >= 0).all()
    assert (att.triu(1 if attend_current else 0) == 0).all()
    if attend_current:
        torch.testing.assert_close(att[:, 0, 0], beta[:, 0, 0])
        torch.testing.assert_close(rem[:, 0], 1 - beta[:, 0, 0])
    else:
        assert (o[:, 0] == 0).all() and (rem[:, 0] == 1).all()


@pytest.mark.parametrize("attend_current", [False, True])
def test_gradients_finite_differences(attend_current):
    # central differences on the scalar product-form loops pin dq, dk, dv of the analytic backward
    rng = np.random.default_rng(7)
    L, D, scale = 6, 3, 0.8
    q, k, v, do = (rng.standard_normal((L, D)) for _ in range(4))
    drem = rng.standard_normal(L)
    tq, tk, tv, tdo, tdr = (torch.tensor(x) for x in (q, k, v, do, drem))
    dq, dk, dv = orc.stream_backward(tq, tk, tv, tdo, tdr, scale, attend_current)
    eps = 1e-6
    for name, arr, grad in (("q", q, dq), ("k", k, dk), ("v", v, dv)):
        num = np.zeros_like(arr)
        for idx in np.ndindex(*arr.shape):
            orig = arr[idx]
            arr[idx] = orig + eps
            up = brute_loss(q, k, v, do, drem, scale, attend_current)
            arr[idx] = orig - eps
            dn = brute_loss(q, k, v, do, drem, scale, attend_current)
            arr[idx] = orig
            num[idx] = (up - dn) / (2 * eps)
        np.testing.assert_allclose(grad.numpy(), num, atol=2e-8, err_msg=name)


@pytest.mark.parametrize("attend_current", [False, True])
def test_analytic_backward_matches_autograd_of_dense(attend_current):
    torch.manual_seed(2)
    H, D = 2, 8
    cu = [5, 6, 30]
    T = cu[-1]
    q, k, v, do = (torch.randn(H, T, D, dtype=torch.float64) for _ in range(4))
    drem = torch.randn(H, T, dtype=torch.float64)
    o1, r1, dq1, dk1, dv1 = orc.dense_backward_autograd(q, k, v, cu, do, drem, 0.5, False, attend_current)
    o2, r2, dq2, dk2, dv2 = orc.varlen_stream(q, k, v, cu, 0.5, False, attend_current, do, drem, dtype=torch.float64)
    for a, b in ((o1, o2), (r1, r2), (dq1, dq2), (dk1, dk2), (dv1, dv2)):
        torch.testing.assert_close(a, b, atol=1e-11, rtol=0)


def test_gradcheck_dense():
    torch.manual_seed(4)
    L, D = 5, 3
    q, k, v = (torch.randn(1, L, D, dtype=torch.float64, requires_grad=True) for _ in range(3))
    mask, cw = orc.causal_operands(L, dtype=torch.float64)
    assert torch.autograd.gradcheck(lambda a, b, c: orc.dense_stickbreaking(a, b, c, mask, cw, 0.7), (q, k, v))


def test_row_total_identity():
    # sum_j g_ij = do_i . o_i - drem_i (1 - rem_i): used by the device backward as its prefix-sum anchor
    torch.manual_seed(5)
    L, D = 33, 8
    q, k, v, do = (torch.randn(L, D, dtype=torch.float64) for _ in range(4))
    drem = torch.randn(L, dtype=torch.float64)
    o, rem, att, _ = orc.stream_forward(q, k, v, want_att=True)
    g = att * (do @ v.T - drem[:, None])
    torch.testing.assert_close(g.sum(-1), (do * o).sum(-1) - drem * (1 - rem), atol=1e-12, rtol=0)


def test_varlen_is_concatenation_and_zero_start_forms_agree():
    torch.manual_seed(6)
    H, D = 3, 8
    lengths = [1, 5, 33, 1, 17]
    cu = np.cumsum(lengths).tolist()
    T = cu[-1]
    q, k, v = (torch.randn(H, T, D) for _ in range(3))
    o, rem = orc.varlen_dense(q, k, v, cu)
    o0, rem0 = orc.varlen_dense(q, k, v, [0] + cu, zero_start=True)
    assert torch.equal(o, o0) and torch.equal(rem, rem0)
    os_, rs = orc.varlen_stream(q, k, v, torch.tensor(cu))
    torch.testing.assert_close(os_, o, atol=2e-6, rtol=0)
    torch.testing.assert_close(rs, rem, atol=2e-6, rtol=0)
    start = 0
    for n in lengths:
        of, rf = orc.fixed_dense(q[None, :, start:start + n], k[None, :, start:start + n], v[None, :, start:start + n])
        assert torch.equal(of[0], o[:, start:start + n]) and torch.equal(rf[0], rem[:, start:start + n])
        # length-1 sequences / first tokens: nothing visible
        assert (o[:, start] == 0).all() and (rem[:, start] == 1).all()
        start += n
    with pytest.raises(AssertionError):
        orc.varlen_dense(q, k, v, cu, zero_start=True)     # cu[0] != 0


def test_mask_fill_quirks_fp32():
    # sb_ref.py:17 fills hidden log sigma with -1e5: exp() must be exactly 0 in fp32 (no leakage into o or rem)
    torch.manual_seed(8)
    L, D = 40, 8
    q, k = torch.randn(L, D), torch.randn(L, D)
    v = torch.full((L, D), 1e30)
    mask, cw = orc.causal_operands(L)
    o, rem = orc.dense_stickbreaking(q, k, v, mask, cw)
    assert torch.isfinite(o).all() and (o[0] == 0).all() and rem[0] == 1


def test_fp32_dense_vs_fp64_stream_config1():
    # configuration C1 shape: fp32, H=4, D=64, lengths [128, 256, 64]; fp32 dense restatement stays within 1e-5 of fp64
    g = torch.Generator().manual_seed(0)
    H, D, cu = 4, 64, [128, 384, 448]
    q, k, v, do = (torch.randn(H, 448, D, generator=g) for _ in range(4))
    drem = torch.randn(H, 448, generator=g)
    o, rem, dq, dk, dv = orc.dense_backward_autograd(q, k, v, cu, do, drem)
    ref = orc.varlen_stream(q, k, v, cu, do=do, drem=drem, dtype=torch.float64)
    for a, b in zip((o, rem, dq, dk, dv), ref):
        assert (a.double() - b).abs().max() < 2e-5


def test_visible_pairs():
    assert orc.visible_pairs([4096] * 8, 32) == 8 * 32 * 4096 * 4095 // 2
    assert orc.visible_pairs([1, 2, 3], 2, attend_current=True) == 2 * (0 + 1 + 3 + 6)


def test_remainder_term_gradients_match_autograd():
    """y = o + rem v: the hand-derived backward (do unchanged, drem + do.v into rem, rem*do added to dv) against
    autograd through the dense restatement of sb_ref.py followed by the callers' own combination."""
    g = torch.Generator().manual_seed(5)
    H, D, lengths = 2, 8, [7, 1, 12]
    T = sum(lengths)
    q, k, v, dy = (torch.randn(H, T, D, generator=g, dtype=torch.float64) for _ in range(4))
    drem = torch.randn(H, T, generator=g, dtype=torch.float64)
    cu = torch.tensor(lengths).cumsum(0)
    qa, ka, va = (t.clone().requires_grad_() for t in (q, k, v))
    o, rem = orc.varlen_dense(qa, ka, va, cu)
    y = o + rem[..., None] * va
    torch.autograd.backward([y, rem], [dy, drem])
    got = orc.with_remainder(orc.varlen_stream(q, k, v, cu, do=dy, drem=orc.remainder_drem(dy, drem, v).double(),
                                               dtype=torch.float64), v, dy)
    for name, a, b in zip(("y", "rem", "dq", "dk", "dv"), got, (y.detach(), rem.detach(), qa.grad, ka.grad, va.grad)):
        assert torch.allclose(a, b, atol=1e-10, rtol=1e-9), name


@pytest.mark.parametrize("attend_current", [False, True])
def test_fixed_stream_matches_brute_force_and_packed_view(attend_current):
    """`fixed_stream` is the checker of every fixed-length GPU test: its (B, H, L, D) slicing is pinned against the
    scalar product-form loops on a tiny case (forward) with finite differences of those loops (gradients), and on a
    larger case against `varlen_stream` on the same data packed as B sequences, and against autograd through the
    dense restatement.  A transposed batch/head index, a dropped drem or a wrong scale default fails one of them."""
    rng = np.random.default_rng(11)
    B, H, L, D = 2, 2, 5, 4
    q, k, v, do = (rng.standard_normal((B, H, L, D)) for _ in range(4))
    drem = rng.standard_normal((B, H, L))
    tq, tk, tv, tdo, tdr = (torch.tensor(x) for x in (q, k, v, do, drem))
    o, rem, dq, dk, dv = orc.fixed_stream(tq, tk, tv, attend_current=attend_current, do=tdo, drem=tdr, dtype=torch.float64)
    scale = 1 / math.sqrt(D)
    eps = 1e-6
    for b in range(B):
        for h in range(H):
            _, ob, rb = brute_force(q[b, h], k[b, h], v[b, h], scale, attend_current)
            np.testing.assert_allclose(o[b, h].numpy(), ob, atol=1e-12)
            np.testing.assert_allclose(rem[b, h].numpy(), rb, atol=1e-12)
            for arr, grad in ((q, dq), (k, dk), (v, dv)):
                for idx in ((0, 1), (L - 1, D - 1), (2, 0)):
                    full = (b, h) + idx
                    orig = arr[full]
                    arr[full] = orig + eps
                    up = brute_loss(q[b, h], k[b, h], v[b, h], do[b, h], drem[b, h], scale, attend_current)
                    arr[full] = orig - eps
                    dn = brute_loss(q[b, h], k[b, h], v[b, h], do[b, h], drem[b, h], scale, attend_current)
                    arr[full] = orig
                    assert abs(grad[full].item() - (up - dn) / (2 * eps)) < 5e-8
    # larger case: the packed view through varlen_stream, and autograd through the dense restatement
    torch.manual_seed(12)
    B, H, L, D = 3, 2, 37, 8
    q, k, v, do = (torch.randn(B, H, L, D, dtype=torch.float64) for _ in range(4))
    drem = torch.randn(B, H, L, dtype=torch.float64)
    got = orc.fixed_stream(q, k, v, scale=0.4, attend_current=attend_current, do=do, drem=drem, dtype=torch.float64)
    pack = lambda t: t.transpose(0, 1).reshape(H, B * L, *t.shape[3:])
    cu = [L * (b + 1) for b in range(B)]
    ref = orc.varlen_stream(pack(q), pack(k), pack(v), cu, 0.4, False, attend_current, pack(do), pack(drem), dtype=torch.float64)
    dense = orc.dense_backward_autograd(pack(q), pack(k), pack(v), cu, pack(do), pack(drem), 0.4, False, attend_current)
    for a, b_, c in zip(got, ref, dense):
        assert torch.equal(pack(a), b_)
        torch.testing.assert_close(pack(a), c, atol=1e-11, rtol=0)
    # forward-only form and the default drem
    o2, rem2 = orc.fixed_stream(q, k, v, scale=0.4, attend_current=attend_current, dtype=torch.float64)
    assert torch.equal(o2, got[0]) and torch.equal(rem2, got[1])
    nodrem = orc.fixed_stream(q, k, v, scale=0.4, attend_current=attend_current, do=do, dtype=torch.float64)
    zero = orc.fixed_stream(q, k, v, scale=0.4, attend_current=attend_current, do=do, drem=torch.zeros_like(drem), dtype=torch.float64)
    for a, b_ in zip(nodrem, zero):
        assert torch.equal(a, b_)


def _bound16(ref):
    return torch.maximum(torch.full_like(ref, 2e-2), ref.abs() * 2.0 ** -7)


def test_rounding_floor_is_the_exact_result_when_nothing_is_rounded():
    """With a 64-bit "low" type the emulation rounds nothing and must reproduce the streaming forward and the analytic
    backward exactly; with bf16 every result is a bf16 value and P / dZ enter their contractions rounded (checked on
    one element by redoing the contraction by hand)."""
    torch.manual_seed(21)
    L, D = 70, 16
    q, k, v, do = (torch.randn(L, D, dtype=torch.float64) for _ in range(4))
    drem = torch.randn(L, dtype=torch.float64)
    exact = orc.rounding_floor(q, k, v, do, drem, low=torch.float64)
    o, rem = orc.stream_forward(q, k, v)
    grads = orc.stream_backward(q, k, v, do, drem)
    for a, b in zip(exact, (o, rem, *grads)):
        torch.testing.assert_close(a, b, atol=1e-13, rtol=0)
    low = orc.rounding_floor(q, k, v, do, drem)
    for t in low:
        assert torch.equal(t, t.bfloat16().double())
    _, _, att, _ = orc.stream_forward(q, k, v, want_att=True)
    by_hand = (att[:, 3].bfloat16().double() * do[:, 5]).sum()          # dv[3, 5] = sum_i bf16(A_i3) do_i5
    assert low[4][3, 5] == by_hand.bfloat16().double()


def test_rounding_floor_of_saturating_logits_sits_at_the_parity_bound():
    """The adversarial configuration (q, k ~ N(0, 9), short sequences): exact arithmetic with bf16 matrix operands and
    bf16 outputs lands dq / dk within a few thousandths of max(2e-2, 2^-7 |ref|) -- inside on this sample, a few
    elements outside on others -- because |dZ| reaches 8..16 there and its bf16 rounding error (2^-9 relative) is
    contracted against |k| ~ 3.  The GPU test of that configuration therefore measures this floor on its own inputs
    and allows the kernels the floor's excess; nothing is fitted."""
    import bench

    inp = bench.make_inputs("c5", "cpu", heads=1)
    n_seq = 400
    lengths = inp["lengths"][:n_seq]
    T = sum(lengths)
    cu = np.cumsum(lengths)
    host = [inp[n][:, :T] for n in ("q", "k", "v", "do", "drem")]
    exact = orc.varlen_stream(*host[:3], cu, do=host[3], drem=host[4], dtype=torch.float64)
    floor, exact2 = orc.varlen_rounding_floor(*host[:3], cu, host[3], host[4])
    for a, b in zip(exact, exact2):          # the emulation's unrounded by-product is the streaming oracle
        torch.testing.assert_close(a, b, atol=1e-12, rtol=0)
    worst = 0.0
    for name, a, b in zip(("o", "rem", "dq", "dk", "dv"), floor, exact):
        excess = ((a - b).abs() - _bound16(b)).max().item()
        print(f"{name}: floor max-abs err {(a - b).abs().max().item():.3e}, excess over the bound {excess:.3e}")
        worst = max(worst, excess)
    assert -6e-3 < worst < 6e-3  # at the bound, on one side or the other ...
    assert max((a - b).abs().max().item() for a, b in zip(floor[2:4], exact[2:4])) > 2e-2      # ... and well above 2e-2 absolute


@pytest.mark.parametrize("attend_current", [False, True])
def test_rowblocked_stream_matches_unblocked(attend_current):
    """`stream_rowblocked` (the checker of the 64K-token GPU test) against the unblocked streaming form, which the tests
    above pin: block sizes that do and do not divide the length, a block larger than the sequence, length 1."""
    torch.manual_seed(31)
    for L, block in ((97, 32), (64, 64), (50, 512), (1, 4), (130, 7)):
        D = 8
        q, k, v, do = (torch.randn(L, D, dtype=torch.float64) for _ in range(4))
        drem = torch.randn(L, dtype=torch.float64)
        o, rem = orc.stream_forward(q, k, v, 0.3, attend_current)
        grads = orc.stream_backward(q, k, v, do, drem, 0.3, attend_current)
        got = orc.stream_rowblocked(q, k, v, do, drem, 0.3, attend_current, block=block, dtype=torch.float64)
        for a, b in zip(got, (o, rem, *grads)):
            torch.testing.assert_close(a, b, atol=1e-12, rtol=0)
        fwd_only = orc.stream_rowblocked(q, k, v, scale=0.3, attend_current=attend_current, block=block, dtype=torch.float64)
        assert torch.equal(fwd_only[0], got[0]) and torch.equal(fwd_only[1], got[1])
        if L > 40:          # a window of rows: o, rem, dq complete inside it, untouched outside
            part = orc.stream_rowblocked(q, k, v, do, drem, 0.3, attend_current, block=block, dtype=torch.float64, rows=(20, 41))
            for a, b in zip(part[:3], (o, rem, grads[0])):
                torch.testing.assert_close(a[20:41], b[20:41], atol=1e-12, rtol=0)
                assert (a[:20] == 0).all() and (a[41:] == 0).all()
