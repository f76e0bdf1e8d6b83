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


def assert_close(name, got, ref, tol=TOL, scale=1.0):
    """The parity gate.  Flat part: max-abs error <= 2e-2 -- asserted as is for ``rem`` and for every
    tensor whose reference values stay below 2.5 in magnitude.  Larger values cannot meet a flat
    bound in bf16 at all (the rounding of the OUTPUT alone is up to |x| * 2^-8: 1.6e-2 at |x| = 4,
    3.1e-2 at 8), so there an element may additionally differ by half a bf16 ulp of the
    reference value.  ``scale`` > 1 widens the flat part for inputs hotter than N(0,1): the error
    of rounding the bf16 MFMA operands P and dZ grows with the cube of the input scale (dz ~
    scale^2, k ~ scale; oracle/rounding_model.py reproduces it on the CPU).  Prints, per tensor,
    the max-abs error, the median relative error, and how many elements exceed the flat 2e-2."""
    assert torch.isfinite(got.float()).all(), f"{name}: non-finite values"
    s = err_stats(name, got, ref)
    g, r = got.detach().float().cpu(), ref.detach().float().cpu()
    flat = tol * max(1.0, float(scale)) ** 3
    diff = (g - r).abs()
    max_ref = r.abs().max().item() if r.numel() else 0.0
    over_flat = int((diff > TOL).sum()) if g.numel() else 0
    excess_flat = (diff - flat).max().item() if g.numel() else -1.0
    excess = (diff - (flat + r.abs() * 2.0 ** -8)).max().item() if g.numel() else -1.0
    s.update(max_ref=max_ref, over_flat=over_flat, numel=g.numel())
    print(f"  {name}: max_abs={s['max_abs']:.3e} median_rel={s['median_rel']:.3e} max|ref|={max_ref:.2f} "
          f"over_flat_2e-2={over_flat}/{g.numel()}")
    if name == "rem" or max_ref < 2.5:
        assert excess_flat <= 0, f"{name}: error exceeds the flat {flat:g} by {excess_flat:.4e} (max_abs {s['max_abs']:.4e})"
    assert excess <= 0, f"{name}: error exceeds {flat:g} + bf16 half-ulp by {excess:.4e} (max_abs {s['max_abs']:.4e})"
    return s


def assert_matches_rounding_model(names, got, q, k, v, do, lengths, drem=None, attend_current=False, inv_temp=None):
    """Compare with oracle/rounding_model.py (float64 arithmetic with the kernels' bf16 rounding
    points).  What may still differ: fp32 against float64 accumulation, which now and then moves an
    operand or an output across a bf16 rounding boundary -- one bf16 ulp of the value (2^-7 relative)
    plus a small absolute term."""
    from oracle import rounding_model as rm
    model = dict(zip(("o", "rem", "dq", "dk", "dv"),
                     rm.varlen(q.cpu(), k.cpu(), v.cpu(), do.cpu(), lengths, None if drem is None else drem.cpu(),
                               attend_current, inv_temp)))
    worst = {}
    for name, g in zip(names, got):
        m = model[name]
        diff = (g.detach().double().cpu() - m).abs()
        bound = 6e-3 + m.abs() * 2.0 ** -7
        worst[name] = diff.max().item()
        print(f"  {name} vs rounding model: max_abs={worst[name]:.3e}")
        assert (diff <= bound).all(), f"{name}: differs from the rounding model by {(diff - bound).max().item():.3e} beyond one bf16 ulp"
    return worst


def oracle_varlen(q, k, v, do, lengths, attend_current=False, inv_temp=None, drem=None, row_chunk=0):
    """fp32 oracle on the bf16-rounded inputs (upcast), returns o, rem, dq, dk, dv (fp32, cpu)."""
    qf, kf, vf, dof = (t.detach().float().cpu() for t in (q, k, v, do))
    dr = None if drem is None else drem.detach().float().cpu()
    return orc.sb_varlen_grads(qf, kf, vf, lengths, dof, dr, attend_current, inv_temp, row_chunk)


def oracle_fixed(q, k, v, do, attend_current=False, inv_temp=None, drem=None, row_chunk=0):
    qf, kf, vf, dof = (t.detach().float().cpu() for t in (q, k, v, do))
    dr = None if drem is None else drem.detach().float().cpu()
    return orc.sb_fixed_grads(qf, kf, vf, dof, dr, attend_current, inv_temp, row_chunk)
