"""Length sweep of the two operators on the shapes upstream's own benchmarks use
(benchmarks/varlen.py:84-96 and benchmarks/attn.py:49-60: 4 sequences of 4096 ... 16384 tokens,
12 heads, head_dim 128, bf16, forward + backward, inputs stored token-major and viewed
head-major), without upstream's flash-attn / transformers / triton dependencies.

    python stickbreaking-attention_amd/benchmarks/sweep.py [--op varlen|attn] [--fwd-only] [--fused]

Prints one line per length: milliseconds per call (median of --reps timed with HIP events after
--warmup calls) and TFLOP/s on the causal FLOP count (4*d per causal pair forward, 14*d forward +
backward).
"""
import argparse
import os
import statistics
import sys

import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))

from stickbreaking_attention import sb_attn, sb_attn_fused, sb_attn_varlen, sb_attn_varlen_fused  # noqa: E402


def timed(fn, warmup, reps):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    times = []
    for _ in range(reps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        e1.synchronize()
        times.append(e0.elapsed_time(e1))
    return statistics.median(times)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--op", default="varlen", choices=["varlen", "attn"])
    ap.add_argument("--lengths", default="4096,8192,12288,16384")
    ap.add_argument("--batch", type=int, default=4)
    ap.add_argument("--heads", type=int, default=12)
    ap.add_argument("--head-dim", type=int, default=128)
    ap.add_argument("--fwd-only", action="store_true")
    ap.add_argument("--fused", action="store_true", help="time the fused o + rem * v operators")
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--reps", type=int, default=20)
    args = ap.parse_args()
    if not torch.cuda.is_available():
        sys.exit("needs an MI355X GPU")
    dev = torch.device("cuda:0")
    B, H, d = args.batch, args.heads, args.head_dim
    gen = torch.Generator(device="cpu").manual_seed(1337)
    print(f"# {args.op} {'fwd' if args.fwd_only else 'fwd+bwd'}{' fused' if args.fused else ''} "
          f"batch={B} heads={H} head_dim={d} bf16")
    print(f"{'length':>8} {'ms':>9} {'TFLOP/s':>9}")
    for L in (int(x) for x in args.lengths.split(",")):
        rand = lambda *shape: torch.randn(shape, generator=gen).to(torch.bfloat16).to(dev)
        if args.op == "varlen":
            # stored [tokens, heads, d], handed over as [heads, tokens, d] views (benchmarks/varlen.py:43-45)
            q, k, v = (rand(B * L, H, d).permute(1, 0, 2).requires_grad_(not args.fwd_only) for _ in range(3))
            do = rand(H, B * L, d)
            cu = torch.arange(1, B + 1, dtype=torch.int32, device=dev) * L
            if args.fused:
                call = lambda: sb_attn_varlen_fused(q, k, v, cu, L, zero_start=False)
            else:
                call = lambda: sb_attn_varlen(q, k, v, cu, L, zero_start=False)[0]
        else:
            q, k, v = (rand(B, L, H, d).permute(0, 2, 1, 3).requires_grad_(not args.fwd_only) for _ in range(3))
            do = rand(B, L, H, d).permute(0, 2, 1, 3)
            call = (lambda: sb_attn_fused(q, k, v)) if args.fused else (lambda: sb_attn(q, k, v)[0])
        if args.fwd_only:
            def fn():
                with torch.no_grad():
                    call()
        else:
            def fn():
                torch.autograd.grad(call(), (q, k, v), do)
        ms = timed(fn, args.warmup, args.reps)
        pairs = B * H * L * L / 2
        flops = (4.0 if args.fwd_only else 14.0) * d * pairs
        print(f"{L:>8} {ms:>9.3f} {flops / ms / 1e9:>9.1f}", flush=True)


if __name__ == "__main__":
    main()
