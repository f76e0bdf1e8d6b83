"""The edges of the supported input envelope: logits far outside N(0,1) in both carry spaces,
genuinely fp32 inputs, float16 inputs on the float16 kernels, and upstream's own long single-document case (tests/test_varlen.py:68-93:
one 16384-token document, head_dim 128, shifted q/k that keep weight alive hundreds of keys
from the diagonal)."""
import os
import warnings

import pytest
import torch

from oracle import sb_oracle as orc
from tests.helpers import assert_close, assert_matches_rounding_model, cu_from_lengths, oracle_varlen

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module", autouse=True)
def _need_gpu():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from stickbreaking_attention import _native as nat
    assert os.path.exists(nat.LIB_PATH), "libsba.so must be built before the GPU tests run"
    nat.load()


def _run(q, k, v, do, lengths, ac=False):
    from stickbreaking_attention import sb_attn_varlen
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    cu = cu_from_lengths(lengths, device=DEV)
    o, rem = sb_attn_varlen(qg, kg, vg, cu, max(lengths), zero_start=False, attend_current=ac)
    dq, dk, dv = torch.autograd.grad(o, (qg, kg, vg), do.to(DEV))
    torch.cuda.synchronize()
    return o.detach(), rem.detach(), dq, dk, dv


@pytest.mark.parametrize("product_space", [False, True])
@pytest.mark.parametrize("qk_scale", [3.0, 8.0])
@pytest.mark.parametrize("d", [64, 128, 256])
def test_large_logits(product_space, qk_scale, d, monkeypatch):
    """q and k scaled so that the logits reach +-35 (x3) or +-250 (x8): sigmoid saturates, 2^z
    overflows fp32 (product space: r = 0; log2 space: logit clamped at 126), the forward's clamp
    of the odds at 2^30 and the backward's unclamped 1 - sigmoid differ by at most 2^-30.
    Everything must stay finite and agree with the oracle; the gate is widened as for any
    hot input (dq and dk carry the factor of k resp. q)."""
    from stickbreaking_attention import _ops
    monkeypatch.setattr(_ops, "PRODUCT_SPACE", product_space)
    lengths = [300, 129, 64]
    q, k, v, do = orc.make_inputs((2, sum(lengths), d), 500 + d)
    q, k = (q.float() * qk_scale).to(torch.bfloat16), (k.float() * qk_scale).to(torch.bfloat16)
    for ac in (False, True):
        got = _run(q, k, v, do, lengths, ac)
        ref = oracle_varlen(q, k, v, do, lengths, ac)
        for name, g, r in zip(("o", "rem", "dq", "dk", "dv"), got, ref):
            assert_close(name, g, r, scale=qk_scale ** (1.0 / 3.0) if name in ("dq", "dk") else 1.0)
        assert_matches_rounding_model(("o", "rem", "dq", "dk", "dv"), got, q, k, v, do, lengths, None, ac)


def test_fp32_inputs_are_rounded_to_bf16_and_say_so():
    """fp32 N(0,1) inputs that are NOT bf16-representable, against the oracle on those fp32
    values: the library rounds q, k, v, grad_o to bf16 (and warns once per dtype).  Rounding the
    inputs moves every logit by about 2^-9 sqrt(2) |z|, which stays inside the usual gate."""
    from stickbreaking_attention import _ops, sb_attn_varlen
    _ops._warned_dtypes.discard(torch.float32)
    lengths = [257, 640, 95]
    T = sum(lengths)
    g = torch.Generator().manual_seed(4321)
    q, k, v, do = (torch.randn((3, T, 64), generator=g) for _ in range(4))
    assert not torch.equal(q, q.to(torch.bfloat16).float())
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    cu = cu_from_lengths(lengths, device=DEV)
    with pytest.warns(UserWarning, match="rounded to bfloat16"):
        o, rem = sb_attn_varlen(qg, kg, vg, cu, max(lengths), zero_start=False)
    assert o.dtype == torch.float32 and rem.dtype == torch.float32
    with warnings.catch_warnings():
        warnings.simplefilter("error")          # said once, not on every call
        dq, dk, dv = torch.autograd.grad(o, (qg, kg, vg), do.to(DEV))
    torch.cuda.synchronize()
    ref = orc.sb_varlen_grads(q, k, v, lengths, do)
    for name, gt, r in zip(("o", "rem", "dq", "dk", "dv"), (o.detach(), rem.detach(), dq, dk, dv), ref):
        assert_close(name + " (fp32 inputs)", gt, r)


@pytest.mark.parametrize("gscale", [1.0, 1e-6, 3e4])
def test_float32_inputs_on_the_float16_kernels(gscale, monkeypatch):
    """SBA_F32_AS_F16: float32 callers get operands of 11 significant bits (what TF32 gives upstream's float32
    dots, utils.py:8) instead of bfloat16's 8.  The incoming gradient may have any scale -- 1e-6 would be a
    float16 subnormal, 3e4 * sqrt(d) would overflow dz -- so it is normalised by a power of two and the gradients
    scaled back: the error relative to the gradient's scale must not depend on it, and must be several times
    below what the bfloat16 route gives on the same values.  No precision warning; float32 outputs."""
    from stickbreaking_attention import _ops, sb_attn_varlen
    lengths = [257, 640, 95]
    T = sum(lengths)
    g = torch.Generator().manual_seed(4321)
    q, k, v, do = (torch.randn((3, T, 64), generator=g) for _ in range(4))
    do = do * gscale
    drem = torch.randn((3, T), generator=g) * gscale
    ref = orc.sb_varlen_grads(q, k, v, lengths, do, drem)
    cu = cu_from_lengths(lengths, device=DEV)

    def run():
        qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
        o, rem = sb_attn_varlen(qg, kg, vg, cu, max(lengths), zero_start=False)
        grads = torch.autograd.grad((o, rem), (qg, kg, vg), (do.to(DEV), drem.to(DEV)))
        torch.cuda.synchronize()
        return (o.detach(), rem.detach()) + grads

    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        coarse = run()                                  # the default: rounded to bfloat16
    monkeypatch.setattr(_ops, "F32_AS_F16", True)
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        fine = run()
    for name, gt, gc, r in zip(("o", "rem", "dq", "dk", "dv"), fine, coarse, ref):
        assert gt.dtype == torch.float32
        unit = 1.0 if name in ("o", "rem") else gscale
        diff = (gt.cpu() - r).abs()
        worse = (gc.cpu() - r).abs().max().item()
        print(f"  {name} (float32 on float16 kernels, gradient scale {gscale:g}): max_abs={diff.max().item():.3e}, "
              f"rounded to bfloat16: {worse:.3e}")
        assert (diff <= 4e-3 * unit + r.abs() * 2.0 ** -11).all(), f"{name}: {diff.max().item():.3e}"
        assert diff.max().item() * 3 < worse, f"{name}: not clearly finer than the bfloat16 route"


@pytest.mark.parametrize("d", [32, 64, 128, 256])
def test_float16_runs_on_the_float16_kernels(d):
    """float16 q, k, v, grad_o are multiplied as float16 (11 significant bits instead of bfloat16's 8;
    upstream's tl.dot does the same, sb_varlen_fwd.py:42): the operands P and dZ and the outputs are
    rounded eight times finer, so the error against the fp32 oracle on the same float16 values must
    be several times below the bfloat16 gate.  No precision warning; float16 outputs; a refused
    launch fills float16 NaNs."""
    from stickbreaking_attention import _ops, sb_attn_varlen, sb_attn_varlen_fused
    lengths = [300, 129, 64, 519]
    T = sum(lengths)
    g = torch.Generator().manual_seed(99 + d)
    q, k, v, do = (torch.randn((3, T, d), generator=g).to(torch.float16) for _ in range(4))
    assert not torch.equal(q, q.to(torch.bfloat16).to(torch.float16))      # not bf16-representable
    ref = orc.sb_varlen_grads(q.float(), k.float(), v.float(), lengths, do.float())
    for ac in (False, True):
        with warnings.catch_warnings():
            warnings.simplefilter("error")
            got = _run(q, k, v, do, lengths, ac)
        if ac:
            ref = orc.sb_varlen_grads(q.float(), k.float(), v.float(), lengths, do.float(), None, True)
        for name, gt, r in zip(("o", "rem", "dq", "dk", "dv"), got, ref):
            assert gt.dtype == torch.float16
            diff = (gt.float().cpu() - r).abs()
            bound = 4e-3 + r.abs() * 2.0 ** -11
            print(f"  {name} (float16, attend_current={ac}): max_abs={diff.max().item():.3e}")
            assert (diff <= bound).all(), f"{name}: {diff.max().item():.3e}"
    # fused output and its gradient
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    cu = cu_from_lengths(lengths, device=DEV)
    out = sb_attn_varlen_fused(qg, kg, vg, cu, max(lengths), zero_start=False)
    o_ref, rem_ref = orc.sb_varlen(q.float(), k.float(), v.float(), lengths)[:2]
    fused_ref = o_ref + rem_ref[..., None] * v.float()
    assert out.dtype == torch.float16
    assert ((out.float().cpu() - fused_ref).abs() <= 4e-3 + fused_ref.abs() * 2.0 ** -11).all()


def test_float16_refused_launch_gives_nan(monkeypatch):
    from stickbreaking_attention import _ops
    monkeypatch.setattr(_ops, "SYNC_FREE", True)
    _ops.release_workspaces()
    lengths = [700, 300]
    g = torch.Generator().manual_seed(5)
    q, k, v, do = (torch.randn((2, 1000, 64), generator=g).to(torch.float16) for _ in range(4))
    from stickbreaking_attention import sb_attn_varlen
    qg = q.to(DEV).requires_grad_()
    o, rem = sb_attn_varlen(qg, k.to(DEV), v.to(DEV), cu_from_lengths(lengths, device=DEV), 64, zero_start=False)
    torch.cuda.synchronize()
    assert o.dtype == torch.float16 and torch.isnan(o).all() and torch.isnan(rem).all()


def test_upstream_single_16k_document():
    """One 16384-token document, head_dim 128, upstream's shifted distribution, forward and
    backward; the oracle checks both heads, 1024 query rows at a time."""
    L = 16384
    q, k, v, do = orc.make_inputs((2, L, 128), 1337, dist="upstream")
    got = _run(q, k, v, do, [L])
    ref = oracle_varlen(q, k, v, do, [L], row_chunk=1024)
    for name, g, r in zip(("o", "rem", "dq", "dk", "dv"), got, ref):
        assert_close(name, g, r)
