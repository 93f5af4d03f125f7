#!/usr/bin/env python3
"""Milliseconds against sequence length for the fixed-length operator, the sweep of the reference's
benchmarks/attn.py:52-64: batch 4, 12 heads, head_dim 128, bf16, lengths 4096 .. 16384, (B, L, H, D)-major inputs
viewed as (B, H, L, D), forward + backward of ``sb_attn`` with the gradient arriving through ``o`` only
(benchmarks/attn.py:13-20, 88-93), and the forward alone.  Only the stick-breaking provider exists here; times are
medians of HIP-event timings on the current stream.

    python stickbreaking-attention_amd/benchmarks/attn.py [--lengths 4096 8192 ...] [--num-heads 12] [--rep 50]
"""
import argparse
import math
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from stickbreaking_attention.sb_attn import sb_attn  # noqa: E402


def median_ms(fn, warmup, rep):
    for _ in range(warmup):
        fn()
    times = []
    for _ in range(rep):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        b.synchronize()
        times.append(a.elapsed_time(b))
    return sorted(times)[len(times) // 2]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--lengths", type=int, nargs="+", default=[4096, 2 * 4096, 3 * 4096, 4 * 4096])
    ap.add_argument("--batch-size", type=int, default=4)
    ap.add_argument("--num-heads", type=int, default=12)
    ap.add_argument("--head-dim", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--rep", type=int, default=50)
    args = ap.parse_args()
    device = torch.device("cuda:0")
    torch.manual_seed(1337)
    print(f"{'length':>8} {'fwd ms':>10} {'fwd+bwd ms':>12} {'fwd TFLOP/s':>12} {'fwd+bwd TFLOP/s':>16}")
    for length in args.lengths:
        B, H, D = args.batch_size, args.num_heads, args.head_dim
        q, k, v = (torch.randn(B, length, H, D, device=device, dtype=torch.bfloat16).requires_grad_() for _ in range(3))
        do = torch.randn(B, length, H, D, device=device, dtype=torch.bfloat16)

        def fwd():
            o, rem = sb_attn(q.permute(0, 2, 1, 3), k.permute(0, 2, 1, 3), v.permute(0, 2, 1, 3), inv_temp=1 / math.sqrt(D))
            return o.permute(0, 2, 1, 3)

        def fwd_bwd():
            torch.autograd.grad(fwd(), inputs=(q, k, v), grad_outputs=do)

        def fwd_only():
            with torch.no_grad():
                fwd()

        ms_f = median_ms(fwd_only, args.warmup, args.rep)
        ms_fb = median_ms(fwd_bwd, args.warmup, args.rep)
        pairs = H * B * length * (length - 1) // 2
        print(f"{length:>8} {ms_f:>10.3f} {ms_fb:>12.3f} {4 * D * pairs / ms_f / 1e9:>12.1f} {14 * D * pairs / ms_fb / 1e9:>16.1f}",
              flush=True)


if __name__ == "__main__":
    main()
