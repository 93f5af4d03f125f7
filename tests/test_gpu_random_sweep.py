"""Seeded random sweep over the operator's options on the GPU, every case against the CPU oracle.

The fixed parity cases pin the benchmark configurations and the reference's own grid; this sweep draws the
combinations nobody thought of: head counts, head dims (fast-path and generic), dtypes, ragged lengths around the
32/64/128 tile edges, attend_current, a leading zero in cu_seqlens, cu_seqlens on the host or on the device, the fused
remainder term, a backward that rebuilds the forward's products, a backward workspace limit (heads in groups), token-major
strides and trailing rows no sequence covers.  The cases are a pure function of the seed, so a failure names its case.
"""
import numpy as np
import pytest
import torch

from oracle import sb_oracle as orc
from test_gpu_parity import NAMES, tol_check

pytestmark = pytest.mark.gpu

EDGE_LENGTHS = [1, 2, 31, 32, 33, 63, 64, 65, 96, 97, 127, 128, 129, 160, 161, 191, 192, 193, 255, 256, 257, 300, 385, 511, 513]


def draw_case(seed):
    rng = np.random.default_rng(1000 + seed)
    dtype = [torch.bfloat16, torch.bfloat16, torch.float16, torch.float32][rng.integers(0, 4)]
    D = int(rng.choice([16, 32, 50, 64, 64, 72, 128, 128, 128]))
    H = int(rng.integers(1, 6))
    n_seq = int(rng.integers(1, 7))
    lengths = [int(rng.choice(EDGE_LENGTHS)) if rng.random() < 0.6 else int(rng.integers(1, 700)) for _ in range(n_seq)]
    if dtype == torch.float32:                       # the fp32 path is the slow vector-ALU one: keep it small
        lengths = [min(n, 200) for n in lengths[:3]]
        H = min(H, 2)
    qk_std = 1.0 if dtype == torch.float32 else float(rng.choice([1.0, 1.0, 2.0]))
    return dict(
        seed=seed, dtype=dtype, D=D, H=H, lengths=lengths,
        attend_current=bool(rng.integers(0, 2)), zero_start=bool(rng.integers(0, 2)), host_cu=bool(rng.integers(0, 2)),
        add_remainder=bool(rng.integers(0, 2)), save_carry=bool(rng.integers(0, 3) > 0),
        limit_heads=bool(rng.integers(0, 3) == 0), token_major=bool(rng.integers(0, 3) == 0),
        pad=int(rng.choice([0, 0, 1, 130])), qk_std=qk_std,
        int64_cu=bool(rng.integers(0, 2)),
    )


@pytest.mark.parametrize("seed", range(48))
def test_random_case_against_oracle(gpu_device, seed):
    from stickbreaking_attention import _native, sb_attn_varlen

    c = draw_case(seed)
    print({k: (str(v) if k == "dtype" else v) for k, v in c.items()}, flush=True)
    dtype, D, H, lengths, pad = c["dtype"], c["D"], c["H"], c["lengths"], c["pad"]
    T = sum(lengths)
    g = torch.Generator().manual_seed(5000 + seed)
    q, k, v, do = (torch.randn(H, T + pad, D, generator=g) for _ in range(4))
    drem = torch.randn(H, T + pad, generator=g)
    q, k = q * c["qk_std"], k * c["qk_std"]
    host = [t.to(dtype) for t in (q, k, v, do, drem)]
    ends = torch.tensor(np.cumsum(lengths), dtype=torch.int64 if c["int64_cu"] else torch.int32)
    cu = torch.cat([torch.zeros(1, dtype=ends.dtype), ends]) if c["zero_start"] else ends

    def to_gpu(t):
        if c["token_major"] and t.dim() == 3:                      # (T, H, D) storage viewed as (H, T, D)
            return t.transpose(0, 1).contiguous().to(gpu_device).transpose(0, 1)
        return t.to(gpu_device)

    dq_, dk_, dv_ = (to_gpu(t).requires_grad_() for t in host[:3])
    cu_arg = cu if c["host_cu"] else cu.to(gpu_device)
    try:
        if c["limit_heads"]:
            _native.set_backward_workspace_limit(1)                 # raised to one head's need: one head per pass
        o, rem = sb_attn_varlen(dq_, dk_, dv_, cu_arg, max(lengths), zero_start=c["zero_start"],
                                attend_current=c["attend_current"], add_remainder=c["add_remainder"],
                                save_carry=c["save_carry"])
        grads = torch.autograd.grad([o, rem], [dq_, dk_, dv_], [to_gpu(host[3]), host[4].to(gpu_device)])
        torch.cuda.synchronize()
    finally:
        _native.set_backward_workspace_limit(None)
    got = [o, rem, *grads]

    cov = [t[:, :T] for t in host]
    if c["add_remainder"]:
        ref = orc.varlen_stream(*cov[:3], ends, attend_current=c["attend_current"], do=cov[3],
                                drem=orc.remainder_drem(cov[3], cov[4], cov[2]).float(), dtype=torch.float64)
        ref = orc.with_remainder(ref, cov[2], cov[3])
    else:
        ref = orc.varlen_stream(*cov[:3], ends, attend_current=c["attend_current"], do=cov[3], drem=cov[4], dtype=torch.float64)
    for n, a, b in zip(NAMES, got, ref):
        tol_check(n, a[:, :T], b, dtype, f"sweep {seed}")
        if pad:
            assert (a[:, T:] == 0).all(), f"{n}: rows no sequence covers must be zero"


@pytest.mark.parametrize("seed", range(16))
def test_random_fixed_length_case_against_oracle(gpu_device, seed):
    """The fixed-length operator on (B, H, L, D) or token-major (B, L, H, D) storage, same options."""
    from stickbreaking_attention import _native, sb_attn

    rng = np.random.default_rng(3000 + seed)
    dtype = [torch.bfloat16, torch.float16, torch.float32][rng.integers(0, 3)]
    D = int(rng.choice([32, 64, 72, 128, 128]))
    B, H = int(rng.integers(1, 4)), int(rng.integers(1, 4))
    L = int(rng.choice(EDGE_LENGTHS)) if dtype != torch.float32 else int(rng.choice([1, 33, 128, 161]))
    opts = dict(attend_current=bool(rng.integers(0, 2)), add_remainder=bool(rng.integers(0, 2)), save_carry=bool(rng.integers(0, 2)))
    token_major, limit = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    print(dict(seed=seed, dtype=str(dtype), D=D, B=B, H=H, L=L, token_major=token_major, limit=limit, **opts), flush=True)
    g = torch.Generator().manual_seed(7000 + seed)
    q, k, v, do = (torch.randn(B, H, L, D, generator=g).to(dtype) for _ in range(4))
    drem = torch.randn(B, H, L, generator=g).to(dtype)

    def to_gpu(t):
        if token_major:
            return t.transpose(1, 2).contiguous().to(gpu_device).transpose(1, 2)
        return t.to(gpu_device)

    qd, kd, vd = (to_gpu(t).requires_grad_() for t in (q, k, v))
    try:
        if limit:
            _native.set_backward_workspace_limit(1)
        o, rem = sb_attn(qd, kd, vd, **opts)
        grads = torch.autograd.grad([o, rem], [qd, kd, vd], [to_gpu(do), drem.to(gpu_device)])
        torch.cuda.synchronize()
    finally:
        _native.set_backward_workspace_limit(None)
    # the oracle per batch entry, as a packed batch of one sequence
    for b in range(B):
        cu = torch.tensor([L], dtype=torch.int32)
        if opts["add_remainder"]:
            ref = orc.varlen_stream(q[b], k[b], v[b], cu, attend_current=opts["attend_current"], do=do[b],
                                    drem=orc.remainder_drem(do[b], drem[b], v[b]).float(), dtype=torch.float64)
            ref = orc.with_remainder(ref, v[b], do[b])
        else:
            ref = orc.varlen_stream(q[b], k[b], v[b], cu, attend_current=opts["attend_current"], do=do[b], drem=drem[b],
                                    dtype=torch.float64)
        for n, a, r in zip(NAMES, [o, rem, *grads], ref):
            tol_check(n, a[b], r, dtype, f"fixed sweep {seed} batch {b}")
