"""Benchmark of the stick-breaking attention hot path on one MI355X.

A "step" is one forward + backward of sb_attn_varlen over the headline workload (config c3:
32 heads, head_dim 128, 16384 packed tokens in 8 documents, bf16, inputs resident in HBM).
Prints ONE JSON line: whole-job fwd+bwd TFLOP/s on the causal FLOP count, the roofline of the
dominant kernel (duration measured with HIP events on the launch stream, inside libsba.so),
the other BASELINE workloads (c2, c4, c5) and a head_dim 256 run (d256) measured the same way in the same run, and the CPU
oracle timed on this host: the dense sb_ref restatement on config c1 and the running-sum
form on a bounded sample of the headline workload.
"""
import argparse
import ctypes
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "stickbreaking-attention_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

PEAK_BF16_TFLOPS = 2500.0   # MI355X published dense bf16 MFMA peak
PEAK_HBM_GBS = 8000.0       # MI355X published HBM3E bandwidth

# Figures that only rocprofv3 can see, on workload c3, recorded from the runs whose summaries are under profiles/
# and valid for the library version they were measured with (any other version of libsba.so reports null).
#   traffic: HBM bytes per launch from two `--pmc` runs of this script (FETCH_SIZE, then WRITE_SIZE, KiB per
#     dispatch, summed over XCDs), each scaled by what the same counter reads for the 256 MiB device copy of
#     --calibrate-copy (FETCH_SIZE x2.0, WRITE_SIZE x1.0): profiles/c3_hbm_traffic_pmc.txt
#   mfma_busy, valu_busy, coexec: fractions of the launch's SIMD-cycles in which the matrix pipe is busy
#     (SQ_VALU_MFMA_BUSY_CYCLES), a vector instruction is active (4 x SQ_ACTIVE_INST_VALU) and both at once
#     (SQ_VALU_MFMA_COEXEC_CYCLES), over 1024 SIMDs x GRBM_GUI_ACTIVE / 8: profiles/c3_sq_counters_pmc.txt
MEASURED = {"sba_version": 213,
            "c3": {"fwd_kernel": {"traffic": 1.097e9, "mfma_busy": 0.462, "valu_busy": 0.554, "coexec": 0.193},
                   "bwd_dq_kernel": {"traffic": 1.108e9, "mfma_busy": 0.428, "valu_busy": 0.578, "coexec": 0.166},
                   "bwd_dkdv_kernel": {"traffic": 1.228e9, "mfma_busy": 0.421, "valu_busy": 0.503, "coexec": 0.181}}}

KERNELS = ["fwd_kernel", "bwd_dq_kernel", "bwd_dkdv_kernel"]


def workload(name):
    if name == "c2":   # fixed-length sb_attn: batch 4 x 16 heads x 2048 tokens x d=64, every (batch, head) one document
        return [2048] * 4, dict(H=16, d=64, scale=1.0, zero_start=False, backward=True, fixed=True, bound="mfma")
    with open(os.path.join(ROOT, "tests", "golden", "doc_lengths.json")) as f:
        lengths = json.load(f)["c3" if name == "d256" else name]
    cfg = {"c3": dict(H=32, d=128, scale=1.0, zero_start=False, backward=True, bound="mfma"),
           # many short documents: ~9 GFLOP of forward work against 256 MiB of mandatory traffic -> HBM bound
           "c4": dict(H=32, d=64, scale=1.0, zero_start=True, backward=True, bound="hbm"),
           "c5": dict(H=32, d=128, scale=0.5, zero_start=False, backward=False, bound="mfma"),
           # not a BASELINE workload: c3's documents with half the heads at twice the head_dim (the same FLOP count)
           "d256": dict(H=16, d=256, scale=1.0, zero_start=False, backward=True, bound="mfma")}[name]
    return lengths, cfg


def causal_pairs(lengths):
    return sum(l * l for l in lengths) / 2.0


def device_clock_mhz(torch):
    """Peak engine clock from hipDeviceAttributeClockRate (kHz); 0.0 if the runtime cannot be asked."""
    try:
        hip = ctypes.CDLL("libamdhip64.so")
        val = ctypes.c_int(0)
        if hip.hipDeviceGetAttribute(ctypes.byref(val), 5, torch.cuda.current_device()) == 0:   # 5 = hipDeviceAttributeClockRate
            return val.value / 1e3
    except OSError:
        pass
    return 0.0


def cpu_baseline(lengths, d):
    """Two CPU figures from the oracle on this host's cores.
    (1) BASELINE config c1 exactly: the dense sb_ref-shaped ``stickbreaking`` (fp32, 1 x 4 heads x
        512 tokens x 64, N(0,1)), forward and forward + autograd backward, median of 10 runs each.
    (2) The running-sum form on ONE of the 32 heads of the headline documents, forward + backward:
        the same work per head as the GPU step, bounded to about ten seconds."""
    import torch
    from oracle import sb_oracle as orc
    # (1)
    q, k, v, do = (t.float() for t in orc.make_inputs((1, 4, 512, 64), 1337 + 1))
    mask, cw = orc.causal_mask_and_weights(512, False, torch.float32)
    fwd, both = [], []
    for _ in range(11):
        t0 = time.perf_counter()
        with torch.no_grad():
            orc.stickbreaking(q, k, v, mask, cw)
        fwd.append(time.perf_counter() - t0)
        qq, kk, vv = (t.clone().requires_grad_() for t in (q, k, v))
        t0 = time.perf_counter()
        o, _ = orc.stickbreaking(qq, kk, vv, mask, cw)
        torch.autograd.grad(o, (qq, kk, vv), do)
        both.append(time.perf_counter() - t0)
    fwd, both = statistics.median(fwd[1:]), statistics.median(both[1:])
    pairs1 = 4 * 512 * 512 / 2.0
    c1 = {"workload": "c1: oracle.stickbreaking (dense sb_ref form) fp32, 1 x 4 heads x 512 tokens x d=64, N(0,1)",
          "fwd_ms": fwd * 1e3, "fwd_bwd_ms": both * 1e3, "reps": 10,
          "fwd_gflops": 4.0 * 64 * pairs1 / fwd / 1e9, "fwd_bwd_gflops": 14.0 * 64 * pairs1 / both / 1e9}
    # (2)
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
                      f"{reps} reps, {dt * 1e3:.0f} ms each",
            "c1_dense": c1}


def measure(name, steps, warmup, args, torch, lib, lengths_override=None):
    """Times one workload; returns a dict of raw figures."""
    from oracle import sb_oracle as orc
    from stickbreaking_attention import sb_attn, sb_attn_fused, sb_attn_varlen, sb_attn_varlen_fused
    dev = torch.device("cuda:0")
    lengths, cfg = workload(name)
    if lengths_override:
        lengths = lengths_override
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

    # An idle MI355X sits at a few hundred MHz and takes some tenths of a second of load to reach
    # its working clock; a handful of warm-up steps (10 ms) ends long before that.  The same step is
    # therefore repeated, untimed, for `ramp_ms` before the W warm-up steps and the K timed steps.
    t0 = time.perf_counter()
    ramp_steps = 0
    while (time.perf_counter() - t0) * 1e3 < args.ramp_ms:
        for _ in range(10):
            step()
        torch.cuda.synchronize()
        ramp_steps += 10
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / steps

    for _ in range(3):
        fwd_only()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fwd_only()
    torch.cuda.synchronize()
    ms_fwd = (time.perf_counter() - t0) * 1e3 / steps

    # per-kernel durations: HIP events recorded by the library on the stream it launches on.  The
    # library keeps the events of the most recent launch of each kernel, and reading them waits for
    # that launch, so each sample is the LAST of three steps queued back to back: the kernels that are
    # measured run behind a busy queue exactly as the steps of the timed loop above do, not behind a
    # host wait.
    lib.sba_set_timing(1)
    acc = [0.0, 0.0, 0.0]
    reps = 10
    for _ in range(reps):
        for _ in range(3):
            step()
        for i in range(3):
            acc[i] += lib.sba_last_kernel_ms(i)   # waits for that kernel of the step just queued
    lib.sba_set_timing(0)
    kern_ms = [a / reps for a in acc]
    if not backward:
        kern_ms[1] = kern_ms[2] = 0.0

    pairs = H * causal_pairs(lengths)        # (fixed-length: `lengths` lists the batch entries)
    tensor_bytes = (len(lengths) if fixed else 1) * H * T * d * 2.0
    del q, k, v, do
    torch.cuda.empty_cache()
    return dict(name=name, lengths=lengths, cfg=cfg, H=H, d=d, T=T, fixed=fixed, backward=backward, pairs=pairs,
                tensor_bytes=tensor_bytes, ms_step=ms_step, ms_fwd=ms_fwd, kern_ms=kern_ms, ramp_steps=ramp_steps)


def roofline(m, lib):
    """Roofline object of the dominant kernel of a measured workload.
    MFMA bound: algorithmic FLOPs per launch -- forward 4*d per causal pair (QK^T, AV); the
    backward's 10*d (recompute QK^T, dO V^T, dQ, dK, dV) split as 6*d for the dq pass and 4*d for
    the dk/dv pass, whose own recomputation of QK^T and dO V^T is executed, not algorithmic, work.
    HBM bound: the tensors a kernel must read and write once -- forward q,k,v in and o out (4 N,
    N = heads*tokens*head_dim*2 bytes), dq pass q,k,v,dO in and dq out (5 N), dk/dv pass
    q,k,v,dO in and dk,dv out (6 N)."""
    d, pairs, kern_ms = m["d"], m["pairs"], m["kern_ms"]
    dom = max(range(3), key=lambda i: kern_ms[i])
    seen = {"traffic": None, "mfma_busy": None, "valu_busy": None, "coexec": None}
    if lib.sba_version() == MEASURED["sba_version"]:
        seen.update(MEASURED.get(m["name"], {}).get(KERNELS[dom], {}))
    traffic = seen["traffic"]
    counters = {k: seen[k] for k in ("mfma_busy", "valu_busy", "coexec")}
    if m["cfg"]["bound"] == "hbm":
        alg = [4.0, 5.0, 6.0][dom] * m["tensor_bytes"]
        achieved = alg / (kern_ms[dom] * 1e-3) / 1e9
        return {"bound": "hbm", "kernel": KERNELS[dom], "achieved": achieved, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                "frac": achieved / PEAK_HBM_GBS, "traffic": traffic, **counters}
    alg = [4.0, 6.0, 4.0][dom] * d * pairs
    achieved = alg / (kern_ms[dom] * 1e-3) / 1e12
    return {"bound": "mfma", "kernel": KERNELS[dom], "achieved": achieved, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
            "frac": achieved / PEAK_BF16_TFLOPS, "traffic": traffic, **counters}


def describe(m):
    if m["fixed"]:
        return f"{m['name']}: sb_attn fwd+bwd B={len(m['lengths'])} H={m['H']} T={m['T']} d={m['d']}, N(0,1)"
    return (f"{m['name']}: sb_attn_varlen {'fwd+bwd' if m['backward'] else 'fwd'} H={m['H']} d={m['d']} T={m['T']} in "
            f"{len(m['lengths'])} documents (tests/golden/doc_lengths.json), N(0,1)*{m['cfg']['scale']}")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--ramp-ms", type=float, default=400.0,
                    help="untimed repetitions of the step before the warm-up, until the device clock has settled")
    ap.add_argument("--workload", default="c3", choices=["c2", "c3", "c4", "c5", "d256"])
    ap.add_argument("--lengths", default=None,
                    help="comma-separated document lengths replacing the workload's own (shape sweeps; "
                         "heads, head_dim and scaling stay those of --workload)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-secondary", action="store_true",
                    help="skip the other workloads (c2, c4, c5, d256) that a default run measures beside c3")
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
    from stickbreaking_attention import _native, _ops
    if args.log_space:
        _ops.PRODUCT_SPACE = False
    lib = _native.load()
    dev = torch.device("cuda:0")
    props = torch.cuda.get_device_properties(dev)
    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    override = [int(x) for x in args.lengths.split(",")] if args.lengths else None
    m = measure(args.workload, args.steps, args.warmup, args, torch, lib, override)
    label = args.workload + ("/custom" if override else "")
    d, pairs, backward = m["d"], m["pairs"], m["backward"]
    executed = [4.0 * d * pairs, 6.0 * d * pairs, 8.0 * d * pairs]
    total_flops = (14.0 if backward else 4.0) * d * pairs
    step_bytes = (11.0 if backward else 4.0) * m["tensor_bytes"]
    out = {
        "metric": "fwd+bwd TFLOP/s (causal FLOP count), sb_attn_varlen bf16 H=32 d=128 16K tokens"
                  if label == "c3" else f"TFLOP/s (causal FLOP count), workload {label}",
        "value": total_flops / (m["ms_step"] * 1e-3) / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": m["ms_step"],
        "clock_ramp": {"ms": args.ramp_ms, "untimed_steps_before_warmup": m["ramp_steps"]},
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": describe(m).replace(m["name"] + ":", label + ":", 1),
                   "carry": "product" if _ops.PRODUCT_SPACE else "log2-sum", "epilogue": args.epilogue,
                   "sum_L2": sum(l * l for l in m["lengths"])},
        "fwd_ms": m["ms_fwd"], "fwd_tflops": 4.0 * d * pairs / (m["ms_fwd"] * 1e-3) / 1e12,
        "frac_of_bf16_peak": total_flops / (m["ms_step"] * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
        "step_gbs_mandatory": step_bytes / (m["ms_step"] * 1e-3) / 1e9,
        "kernel_ms": dict(zip(KERNELS, m["kern_ms"])),
        "kernel_executed_tflops": {n: (executed[i] / (m["kern_ms"][i] * 1e-3) / 1e12 if m["kern_ms"][i] > 0 else 0.0)
                                   for i, n in enumerate(KERNELS)},
        "roofline": roofline(m, lib) if _ops.PRODUCT_SPACE else dict(roofline(m, lib), traffic=None, mfma_busy=None, valu_busy=None, coexec=None),
        "device": {"name": props.name, "cus": props.multi_processor_count, "clock_mhz": device_clock_mhz(torch),
                   "sba_version": lib.sba_version()},
    }
    if label == "c3" and not args.no_secondary and args.epilogue == "none":
        # the other BASELINE workloads, same method, fewer steps: measured in the same run so that
        # whoever runs this script sees them (they are not the headline metric)
        sec = {}
        for w in ("c2", "c4", "c5", "d256"):
            s = measure(w, max(5, args.steps // 2), 3, args, torch, lib)
            fl = (14.0 if s["backward"] else 4.0) * s["d"] * s["pairs"]
            by = (11.0 if s["backward"] else 4.0) * s["tensor_bytes"]
            sec[w] = {"workload": describe(s), "ms_per_step": s["ms_step"], "fwd_ms": s["ms_fwd"],
                      "tflops": fl / (s["ms_step"] * 1e-3) / 1e12,
                      "frac_of_bf16_peak": fl / (s["ms_step"] * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
                      "step_gbs_mandatory": by / (s["ms_step"] * 1e-3) / 1e9,
                      "frac_of_hbm_peak": by / (s["ms_step"] * 1e-3) / 1e9 / PEAK_HBM_GBS,
                      "kernel_ms": dict(zip(KERNELS, s["kern_ms"])), "roofline": roofline(s, lib)}
        out["secondary"] = sec
    if not args.no_cpu_baseline:
        lengths3, cfg3 = workload("c3")
        out["cpu_baseline"] = cpu_baseline(m["lengths"] if not m["fixed"] else lengths3, d if not m["fixed"] else cfg3["d"])
    print(json.dumps(out))


if __name__ == "__main__":
    main()
