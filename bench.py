"""Benchmark of the stick-breaking attention hot path on one MI355X.

A "step" is one forward + backward of sb_attn_varlen over the headline workload (config c3:
32 heads, head_dim 128, 16384 packed tokens in 8 documents, bf16, inputs resident in HBM).
Prints ONE JSON line: whole-job fwd+bwd TFLOP/s on the causal FLOP count, the roofline of the
dominant kernel (duration measured with HIP events on the launch stream, inside libsba.so)
and the CPU oracle timed on a bounded sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "stickbreaking-attention_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

PEAK_BF16_TFLOPS = 2500.0   # MI355X published dense bf16 MFMA peak

# HBM bytes per launch on workload c3, from two `rocprofv3 --pmc` runs of this script
# (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch, summed over XCDs), each scaled by what the
# same counter reads for the 256 MiB device copy of --calibrate-copy (FETCH_SIZE x2.0,
# WRITE_SIZE x1.0).  Counters cannot be read from inside the process, so these are recorded
# constants; other workloads report null.
MEASURED_TRAFFIC_BYTES = {"c3": {"fwd_kernel": 1.164e9, "bwd_dq_kernel": 1.111e9, "bwd_dkdv_kernel": 1.202e9}}


def workload(name):
    if name == "c2":   # fixed-length sb_attn: batch 4 x 16 heads x 2048 tokens x d=64, every (batch, head) one document
        return [2048] * 4, dict(H=16, d=64, scale=1.0, zero_start=False, backward=True, fixed=True)
    with open(os.path.join(ROOT, "tests", "golden", "doc_lengths.json")) as f:
        lengths = json.load(f)[name]
    cfg = {"c3": dict(H=32, d=128, scale=1.0, zero_start=False, backward=True),
           "c4": dict(H=32, d=64, scale=1.0, zero_start=True, backward=True),
           "c5": dict(H=32, d=128, scale=0.5, zero_start=False, backward=False)}[name]
    return lengths, cfg


def causal_pairs(lengths):
    return sum(l * l for l in lengths) / 2.0


def cpu_baseline(lengths, d):
    """The fp32 CPU oracle (running-sum form) on ONE of the 32 heads of the same documents,
    forward + autograd backward, on this host's cores."""
    import torch
    from oracle import sb_oracle as orc
    T = sum(lengths)
    q, k, v, do = (t.float() for t in orc.make_inputs((1, T, d), 1))
    t0 = time.perf_counter()
    reps = 0
    while True:
        orc.sb_varlen_grads(q, k, v, lengths, do, row_chunk=1024)
        reps += 1
        if time.perf_counter() - t0 > 10.0 or reps >= 3:
            break
    dt = (time.perf_counter() - t0) / reps
    flops = 14.0 * d * causal_pairs(lengths)
    return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"oracle/sb_oracle.sb_varlen_grads fp32, 1 of 32 heads x all documents, fwd+bwd, "
                      f"{reps} reps, {dt * 1e3:.0f} ms each"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c3", choices=["c2", "c3", "c4", "c5"])
    ap.add_argument("--lengths", default=None,
                    help="comma-separated document lengths replacing the workload's own (shape sweeps; "
                         "heads, head_dim and scaling stay those of --workload)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--log-space", action="store_true", help="log2-sum carry instead of product carry")
    ap.add_argument("--epilogue", default="none", choices=["none", "torch", "fused"],
                    help="also form o + rem[..., None] * v, what callers do next (and differentiate through it): "
                         "with PyTorch elementwise ops, or inside the kernels (sb_attn_varlen_fused). "
                         "The headline metric is measured with 'none'.")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 256 MiB device copy (reference dispatch for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; --gpus must be 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from oracle import sb_oracle as orc
    from stickbreaking_attention import _native, _ops, sb_attn, sb_attn_fused, sb_attn_varlen, sb_attn_varlen_fused
    if args.log_space:
        _ops.PRODUCT_SPACE = False
    lib = _native.load()
    dev = torch.device("cuda:0")
    props = torch.cuda.get_device_properties(dev)
    lengths, cfg = workload(args.workload)
    if args.lengths:
        lengths = [int(x) for x in args.lengths.split(",")]
        args.workload = f"{args.workload}/custom"
    H, d, T = cfg["H"], cfg["d"], sum(lengths)
    fixed = cfg.get("fixed", False)
    if fixed:
        B, T = len(lengths), lengths[0]
        q, k, v, do = (t.to(dev) for t in orc.make_inputs((B, H, T, d), 1337, scale=cfg["scale"]))
    else:
        q, k, v, do = (t.to(dev) for t in orc.make_inputs((H, T, d), 1337, scale=cfg["scale"]))
    cu = torch.tensor(lengths, dtype=torch.int64).cumsum(0)
    if cfg["zero_start"]:
        cu = torch.cat([torch.zeros(1, dtype=torch.int64), cu])
    cu = cu.to(torch.int32).to(dev)
    max_len = max(lengths)
    backward = cfg["backward"]
    if backward:
        q.requires_grad_(); k.requires_grad_(); v.requires_grad_()

    def attention():
        if args.epilogue == "fused":
            if fixed:
                return sb_attn_fused(q, k, v), None
            return sb_attn_varlen_fused(q, k, v, cu, max_len, zero_start=cfg["zero_start"]), None
        if fixed:
            o, rem = sb_attn(q, k, v)
        else:
            o, rem = sb_attn_varlen(q, k, v, cu, max_len, zero_start=cfg["zero_start"])
        if args.epilogue == "torch":
            o = o + rem[..., None] * v
        return o, rem

    def step():
        if backward:
            o, rem = attention()
            return torch.autograd.grad(o, (q, k, v), do)
        with torch.no_grad():
            return attention()

    def fwd_only():
        with torch.no_grad():
            return attention()

    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
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

    # forward alone (reported beside the headline)
    for _ in range(3):
        fwd_only()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        fwd_only()
    torch.cuda.synchronize()
    ms_fwd = (time.perf_counter() - t0) * 1e3 / args.steps

    # per-kernel durations: HIP events recorded by the library on the stream it launches on
    lib.sba_set_timing(1)
    names = ["fwd_kernel", "bwd_dq_kernel", "bwd_dkdv_kernel"]
    acc = [0.0, 0.0, 0.0]
    reps = 5
    for _ in range(reps):
        step()
        for i in range(3):
            acc[i] += lib.sba_last_kernel_ms(i)
    lib.sba_set_timing(0)
    kern_ms = [a / reps for a in acc]
    if not backward:
        kern_ms[1] = kern_ms[2] = 0.0

    pairs = H * causal_pairs(lengths)
    # Algorithmic FLOPs: forward 4*d per causal pair (QK^T, AV); backward 10*d (recompute QK^T,
    # dO V^T, dQ, dK, dV).  The backward is split in two kernels: the dq pass carries the two
    # recomputed products and dQ (6*d), the dk/dv pass carries dK and dV (4*d); its own
    # recomputation of QK^T and dO V^T is executed work, not algorithmic work.
    alg = [4.0 * d * pairs, 6.0 * d * pairs, 4.0 * d * pairs]
    executed = [4.0 * d * pairs, 6.0 * d * pairs, 8.0 * d * pairs]
    total_flops = (14.0 if backward else 4.0) * d * pairs
    dom = max(range(3), key=lambda i: kern_ms[i])
    achieved = alg[dom] / (kern_ms[dom] * 1e-3) / 1e12
    out = {
        "metric": "fwd+bwd TFLOP/s (causal FLOP count), sb_attn_varlen bf16 H=32 d=128 16K tokens"
                  if args.workload == "c3" else f"TFLOP/s (causal FLOP count), workload {args.workload}",
        "value": total_flops / (ms_step * 1e-3) / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": (f"{args.workload}: sb_attn fwd+bwd B={len(lengths)} H={H} T={T} d={d}, N(0,1)" if fixed else
                               f"{args.workload}: sb_attn_varlen {'fwd+bwd' if backward else 'fwd'} H={H} d={d} "
                               f"T={T} in {len(lengths)} documents (tests/golden/doc_lengths.json), N(0,1)*{cfg['scale']}"),
                   "carry": "product" if _ops.PRODUCT_SPACE else "log2-sum", "epilogue": args.epilogue, "sum_L2": sum(l * l for l in lengths)},
        "fwd_ms": ms_fwd, "fwd_tflops": 4.0 * d * pairs / (ms_fwd * 1e-3) / 1e12,
        "frac_of_bf16_peak": total_flops / (ms_step * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
        "kernel_ms": dict(zip(names, kern_ms)),
        "kernel_executed_tflops": {n: (executed[i] / (kern_ms[i] * 1e-3) / 1e12 if kern_ms[i] > 0 else 0.0)
                                   for i, n in enumerate(names)},
        "roofline": {"bound": "mfma", "kernel": names[dom], "achieved": achieved, "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": achieved / PEAK_BF16_TFLOPS,
                     "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload, {}).get(names[dom])
                     if _ops.PRODUCT_SPACE else None},
        "device": {"name": props.name, "cus": props.multi_processor_count,
                   "clock_mhz": getattr(props, "clock_rate", 0) / 1e3},
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(lengths, d)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
