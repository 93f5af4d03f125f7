#!/usr/bin/env python3
"""Benchmark of the stick-breaking attention hot path on one MI355X.

A "step" is one forward + backward of ``sb_attn_varlen`` over one synthetic packed batch, called through the
Python operators (so allocations and the scheduler kernel are inside the timed region), inputs resident in HBM.
Default workload: bf16, 32 heads x head_dim 128, 32768 packed tokens with log-normal sequence lengths.

Prints ONE JSON line: whole-step algorithmic TFLOP/s (14 * D * visible pairs per step), plus
  roofline     -- the slowest attention kernel timed with HIP events recorded by the library on the launch
                  stream, its algorithmic FLOPs and the fraction of the bf16 dense MFMA peak (2.5 PFLOP/s);
  cpu_baseline -- the dense fp32 CPU restatement of the reference algorithm timed on a bounded slice.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import math
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "stickbreaking-attention_amd"))

MFMA_BF16_PEAK = 2.5e15          # MI355X dense bf16 MFMA peak, FLOP/s

# HBM bytes per launch (fetch + write) of each kernel cannot be read from inside this script (hardware counters need
# rocprofv3): they are measured by the two `rocprofv3 --pmc` runs whose summary is profiles/c3_varlen_hbm_traffic_pmc.txt
# and kept, with the commit they were measured at, in the JSON file beside that summary.  `roofline.traffic` reports
# the figure for the dominant kernel of the workload it was measured on, null otherwise.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")


def measured_traffic(workload, kernel):
    try:
        with open(TRAFFIC_FILE) as f:
            rec = json.load(f)
        return rec["bytes_per_launch"][workload][kernel]
    except (OSError, KeyError, ValueError):
        return None


# ----------------------------------------------------------------------------------------------
# Synthetic workloads (the five configurations the baseline names); shared with the tests.
# ----------------------------------------------------------------------------------------------
def lengths_for(name: str):
    rng = np.random.default_rng(0)
    if name == "c1":
        return [128, 256, 64]
    if name == "c2":
        total, out = 16384, []
        while sum(out) < total:
            out.append(int(rng.integers(256, 4097)))
        out[-1] -= sum(out) - total
        return out
    if name == "c3":
        total, out = 32768, []
        while sum(out) < total:
            out.append(int(np.clip(np.rint(rng.lognormal(math.log(1024), 1.0)), 16, 8192)))
        out[-1] -= sum(out) - total
        return out
    if name == "c4":
        return [4096] * 8
    if name == "c5":
        return [int(x) for x in rng.integers(1, 65, 2048)] + [16384]
    raise ValueError(name)


WORKLOADS = {
    #        heads, head_dim, dtype,           qk_std, zero_start, fixed
    "c1": dict(H=4, D=64, dtype=torch.float32, qk_std=1.0, zero_start=False, fixed=False),
    "c2": dict(H=12, D=64, dtype=torch.bfloat16, qk_std=1.0, zero_start=False, fixed=False),
    "c3": dict(H=32, D=128, dtype=torch.bfloat16, qk_std=1.0, zero_start=False, fixed=False),
    "c4": dict(H=32, D=128, dtype=torch.bfloat16, qk_std=1.0, zero_start=False, fixed=True),
    "c5": dict(H=32, D=128, dtype=torch.bfloat16, qk_std=3.0, zero_start=True, fixed=False),
}


def make_inputs(name: str, device, heads=None):
    """q, k, v, grad_o, grad_rem drawn on the CPU from seed 0 (in that order, fp32), cast to the workload dtype.
    Packed layout (H, T, D); the fixed-length workload is the same data viewed as (B, H, L, D)."""
    w = WORKLOADS[name]
    lengths = lengths_for(name)
    H = heads or w["H"]
    T, D = sum(lengths), w["D"]
    g = torch.Generator().manual_seed(0)
    q, k, v, do = (torch.randn(H, T, D, generator=g) for _ in range(4))
    drem = torch.randn(H, T, generator=g)
    q, k = q * w["qk_std"], k * w["qk_std"]
    q, k, v, do, drem = (t.to(w["dtype"]).to(device) for t in (q, k, v, do, drem))
    cu = torch.tensor(np.cumsum(lengths), dtype=torch.int32)
    if w["zero_start"]:
        cu = torch.cat([torch.zeros(1, dtype=torch.int32), cu])
    return dict(q=q, k=k, v=v, do=do, drem=drem, cu=cu.to(device), lengths=lengths, H=H, D=D, T=T, **{k_: w[k_] for k_ in ("zero_start", "fixed", "dtype")})


def visible_pairs(lengths, heads, attend_current=False):
    return heads * sum(n * (n - 1) // 2 + (n if attend_current else 0) for n in lengths)


# ----------------------------------------------------------------------------------------------
class KernelTimer:
    """HIP events handed to the library through SbaArgs.trace_events (recorded on the launch stream)."""

    def __init__(self, native):
        self.hip = native.lib()          # dlsym through libsba.so reaches the HIP runtime it is linked to
        self.hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        self.hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
        self.hip.hipEventSynchronize.argtypes = [ctypes.c_void_p]
        self.hip.hipEventDestroy.argtypes = [ctypes.c_void_p]

    def new_set(self, n=3):
        arr = (ctypes.c_void_p * n)()
        for i in range(n):
            ev = ctypes.c_void_p()
            assert self.hip.hipEventCreate(ctypes.byref(ev)) == 0
            arr[i] = ev
        return arr

    def free(self, arr):
        for ev in arr:
            assert self.hip.hipEventDestroy(ctypes.c_void_p(ev)) == 0

    def elapsed_ms(self, a, b):
        assert self.hip.hipEventSynchronize(b) == 0
        ms = ctypes.c_float()
        assert self.hip.hipEventElapsedTime(ctypes.byref(ms), a, b) == 0
        return ms.value


def time_kernels(inp, native, iters, save_carry=True):
    """Average duration of the forward, dQ and dK/dV kernels through the C ABI (scheduler kernel excluded; without
    saved products the kernel that rebuilds them is timed with the dQ kernel)."""
    timer = KernelTimer(native)
    q, k, v = inp["q"], inp["k"], inp["v"]
    lead0 = inp["zero_start"]
    maxlen = max(inp["lengths"])
    scale = 1 / math.sqrt(inp["D"])
    sums = [0.0, 0.0, 0.0]
    fixed = inp["fixed"]
    if fixed:
        B, L = len(inp["lengths"]), inp["lengths"][0]
        q, k, v, do = (t.view(inp["H"], B, L, inp["D"]).transpose(0, 1) for t in (q, k, v, inp["do"]))
        drem = inp["drem"].view(inp["H"], B, L).transpose(0, 1)
        cu = None
    else:
        do, drem, cu = inp["do"], inp["drem"], inp["cu"]
    for it in range(iters + 2):
        fwd_ev, bwd_ev = timer.new_set(2), timer.new_set(3)
        native.TRACE_EVENTS = fwd_ev
        o, rem, row_stat, carry = native.forward(q, k, v, cu, lead0, maxlen, scale, False, want_carry=save_carry)
        native.TRACE_EVENTS = bwd_ev
        native.backward(do, drem, q, k, v, carry, cu, lead0, maxlen, scale, False)
        native.TRACE_EVENTS = None
        torch.cuda.synchronize()
        if it >= 2:
            sums[0] += timer.elapsed_ms(fwd_ev[0], fwd_ev[1])
            sums[1] += timer.elapsed_ms(bwd_ev[0], bwd_ev[1])
            sums[2] += timer.elapsed_ms(bwd_ev[1], bwd_ev[2])
        timer.free(fwd_ev)
        timer.free(bwd_ev)
    return [s / iters for s in sums]


def cpu_baseline(sample_len=4096, budget_s=15.0):
    """The CPU restatement (dense fp32 forward + autograd backward, the same operations as sb_ref.py including its
    L x L contraction) timed on the host: configuration C1 in full (fp32, 4 heads, head_dim 64, lengths [128, 256, 64]),
    then (head, sequence) slices of the bench workload's shape, one after another until about `budget_s` seconds of
    CPU work have been spent.  `value` is the rate on the slices."""
    sys.path.insert(0, ROOT)
    from oracle import sb_oracle as orc

    threads = torch.get_num_threads()
    c1 = make_inputs("c1", "cpu")
    orc.dense_backward_autograd(c1["q"], c1["k"], c1["v"], c1["cu"], c1["do"], c1["drem"])          # warm-up
    reps, t0 = 5, time.perf_counter()
    for _ in range(reps):
        orc.dense_backward_autograd(c1["q"], c1["k"], c1["v"], c1["cu"], c1["do"], c1["drem"])
    c1_ms = (time.perf_counter() - t0) * 1e3 / reps
    c1_tflops = 14 * c1["D"] * visible_pairs(c1["lengths"], c1["H"]) / (c1_ms * 1e-3) / 1e12

    D = 128
    g = torch.Generator().manual_seed(0)
    slices, spent = 0, 0.0
    while spent < budget_s:
        q, k, v, do = (torch.randn(1, sample_len, D, generator=g) for _ in range(4))
        drem = torch.randn(1, sample_len, generator=g)
        t0 = time.perf_counter()
        orc.dense_backward_autograd(q, k, v, [sample_len], do, drem)
        spent += time.perf_counter() - t0
        slices += 1
    flops = 14 * D * visible_pairs([sample_len], 1) * slices
    return {"value": flops / spent / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": f"fwd+bwd of {slices} (head, sequence) slices, L={sample_len}, D=128, fp32 dense restatement of "
                      f"sb_ref.py via autograd, {spent:.1f} s, os.cpu_count()={os.cpu_count()}; configuration C1 in full "
                      f"(fp32, H=4, D=64, lengths [128, 256, 64], fwd+bwd): {c1_ms:.2f} ms = {c1_tflops:.4f} TFLOP/s"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c3", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-saved-carry", action="store_true",
                    help="keep only q, k, v between the passes (save_carry=False): the backward rebuilds the forward's products")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="also launch one plain 1 GiB device copy, the known-size reference for HBM traffic counters")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU only (the operator shards by head or by sequence with no "
              "exchange, but no multi-GPU path is part of it); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    from stickbreaking_attention import _native, sb_attn, sb_attn_varlen

    dev = torch.device("cuda:0")
    inp = make_inputs(args.workload, dev)
    H, D, T, lengths = inp["H"], inp["D"], inp["T"], inp["lengths"]
    pairs = visible_pairs(lengths, H)
    q, k, v = (inp[n].requires_grad_() for n in ("q", "k", "v"))
    save_carry = not args.no_saved_carry

    def step():
        if inp["fixed"]:
            B, L = len(lengths), lengths[0]
            q4, k4, v4 = (t.view(H, B, L, D).transpose(0, 1) for t in (q, k, v))
            o, rem = sb_attn(q4, k4, v4, save_carry=save_carry)
            torch.autograd.backward([o, rem], [inp["do"].view(H, B, L, D).transpose(0, 1), inp["drem"].view(H, B, L).transpose(0, 1)])
        else:
            o, rem = sb_attn_varlen(q, k, v, inp["cu"], max(lengths), zero_start=inp["zero_start"], save_carry=save_carry)
            torch.autograd.backward([o, rem], [inp["do"], inp["drem"]])
        q.grad = k.grad = v.grad = None

    def fwd_only():
        with torch.no_grad():
            if inp["fixed"]:
                B, L = len(lengths), lengths[0]
                sb_attn(*(t.view(H, B, L, D).transpose(0, 1) for t in (q, k, v)))
            else:
                sb_attn_varlen(q, k, v, inp["cu"], max(lengths), zero_start=inp["zero_start"])

    if args.traffic_probe:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / args.steps

    for _ in range(3):
        fwd_only()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        fwd_only()
    torch.cuda.synchronize()
    ms_fwd = (time.perf_counter() - t0) * 1e3 / args.steps

    k_fwd, k_dq, k_dkv = time_kernels(inp, _native, max(5, min(args.steps, 20)), save_carry)
    # Algorithmic FLOPs per launch: forward QK^T + PV = 4 D pairs; backward 10 D pairs, of which the dQ kernel is
    # credited with the recompute (QK^T, dO V^T) and dQ = 6 D pairs and the dK/dV kernel with dK, dV = 4 D pairs
    # (its own recompute of QK^T and dO V^T is not algorithmic work).
    # The chained backward is ONE kernel with all 10 D pairs of the backward and no recompute of its own; what is timed
    # in front of it is then only the kernel that rebuilds the forward's products, when there is one.
    if _native.LAST_BWD_KERNELS == 1:
        kernels = {"fwd_kernel": (k_fwd, 4 * D * pairs), "bwd_chain_kernel": (k_dkv, 10 * D * pairs)}
        if not save_carry:
            kernels["fwd_kernel(products only)"] = (k_dq, 2 * D * pairs)
    else:
        kernels = {"fwd_kernel": (k_fwd, 4 * D * pairs), "bwd_dq_kernel": (k_dq, 6 * D * pairs), "bwd_dkv_kernel": (k_dkv, 4 * D * pairs)}
    dom = max(kernels, key=lambda n: kernels[n][0])
    dom_ms, dom_flops = kernels[dom]
    achieved = dom_flops / (dom_ms * 1e-3) / 1e12

    flops_step = 14 * D * pairs
    out = {
        "metric": "fwd+bwd TFLOP/s (algorithmic, 14*D*pairs), varlen stick-breaking attention",
        "value": flops_step / (ms_step * 1e-3) / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": str(inp["dtype"]).replace("torch.", "").replace("bfloat16", "bf16").replace("float32", "f32"),
        "data": "synthetic",
        "config": {"workload": f"{args.workload}: sb_attn{'_varlen' if not inp['fixed'] else ''} fwd+bwd, H={H}, D={D}, "
                               f"T={T}, {len(lengths)} sequences (max {max(lengths)}), pairs={pairs}"
                               + ("" if save_carry else ", products rebuilt in the backward")},
        "frac_bf16_mfma_peak": flops_step / (ms_step * 1e-3) / MFMA_BF16_PEAK,
        "tokens_per_s": T / (ms_step * 1e-3),
        "fwd": {"ms": ms_fwd, "tflops": 4 * D * pairs / (ms_fwd * 1e-3) / 1e12, "tokens_per_s": T / (ms_fwd * 1e-3),
                "frac_bf16_mfma_peak": 4 * D * pairs / (ms_fwd * 1e-3) / MFMA_BF16_PEAK},
        "kernels_ms": {n: round(kernels[n][0], 4) for n in kernels},
        "roofline": {"bound": "mfma", "kernel": dom, "achieved": achieved, "peak": MFMA_BF16_PEAK / 1e12, "unit": "TFLOP/s",
                     "frac": achieved * 1e12 / MFMA_BF16_PEAK,
                     "traffic": measured_traffic(args.workload, dom)},
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
