"""Shared helpers for the parity tests: seeded workloads, error metrics, oracle drivers."""
import json
import math
import os

import torch

from oracle import sb_oracle as orc

GOLDEN_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
TOL = 2e-2   # max-abs tolerance of bf16 kernels against the fp32 oracle on the same bf16 inputs


def doc_lengths(name):
    with open(os.path.join(GOLDEN_DIR, "doc_lengths.json")) as f:
        return json.load(f)[name]


def cu_from_lengths(lengths, leading_zero=False, dtype=torch.int32, device="cpu"):
    cu = torch.tensor(lengths, dtype=torch.int64).cumsum(0)
    if leading_zero:
        cu = torch.cat([torch.zeros(1, dtype=torch.int64), cu])
    return cu.to(dtype).to(device)


def err_stats(name, got, ref):
    got, ref = got.detach().float().cpu(), ref.detach().float().cpu()
    diff = (got - ref).abs()
    big = ref.abs() > 1e-3
    rel = (diff[big] / ref.abs()[big]).median().item() if big.any() else 0.0
    return {"name": name, "max_abs": diff.max().item() if diff.numel() else 0.0, "median_rel": rel}


def assert_close(name, got, ref, tol=TOL):
    """max-abs gate.  The kernels return bf16, whose own rounding is up to |x| * 2^-8 (0.031
    for |x| in [8, 16)), so on top of the absolute tolerance an element may differ by half a
    bf16 ulp of the reference value; for |ref| < 2.5 the bound is the plain 2e-2 to within 1e-2."""
    assert torch.isfinite(got.float()).all(), f"{name}: non-finite values"
    s = err_stats(name, got, ref)
    g, r = got.detach().float().cpu(), ref.detach().float().cpu()
    excess = ((g - r).abs() - (tol + r.abs() * 2.0 ** -8)).max().item() if g.numel() else -1.0
    print(f"  {name}: max_abs={s['max_abs']:.3e} median_rel={s['median_rel']:.3e} max|ref|={r.abs().max().item() if r.numel() else 0:.2f}")
    assert excess <= 0, f"{name}: error exceeds {tol} + bf16 half-ulp by {excess:.4e} (max_abs {s['max_abs']:.4e})"
    return s


def oracle_varlen(q, k, v, do, lengths, attend_current=False, inv_temp=None, drem=None, row_chunk=0):
    """fp32 oracle on the bf16-rounded inputs (upcast), returns o, rem, dq, dk, dv (fp32, cpu)."""
    qf, kf, vf, dof = (t.detach().float().cpu() for t in (q, k, v, do))
    dr = None if drem is None else drem.detach().float().cpu()
    return orc.sb_varlen_grads(qf, kf, vf, lengths, dof, dr, attend_current, inv_temp, row_chunk)


def oracle_fixed(q, k, v, do, attend_current=False, inv_temp=None, drem=None, row_chunk=0):
    qf, kf, vf, dof = (t.detach().float().cpu() for t in (q, k, v, do))
    dr = None if drem is None else drem.detach().float().cpu()
    return orc.sb_fixed_grads(qf, kf, vf, dof, dr, attend_current, inv_temp, row_chunk)
