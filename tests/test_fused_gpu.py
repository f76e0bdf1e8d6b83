"""GPU parity tests of the fused output ``o + rem[..., None] * v`` (what every upstream caller
forms from the two outputs: tests/test_varlen.py:101, tests/test_attn.py:64) and of its gradient,
against the fp32 CPU oracle composed the same way.  Tolerance as for the plain operators:
max-abs 2e-2 (plus the bf16 half-ulp of large values, see helpers.assert_close)."""
import os

import pytest
import torch

from oracle import sb_oracle as orc
from tests.helpers import assert_close, cu_from_lengths, oracle_fixed, oracle_varlen

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module", autouse=True)
def _need_gpu():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from stickbreaking_attention import _native as nat
    assert os.path.exists(nat.LIB_PATH), "libsba.so must be built before the GPU tests run"
    nat.load()


def fused_reference(q, k, v, dout, lengths=None, ac=False):
    """out and its gradients from the oracle: the gradient of the sum reaches rem through v
    (d rem = dout . v per row) and v directly (rem * dout)."""
    vf, df = v.float().cpu(), dout.float().cpu()
    drem = (df * vf).sum(-1)
    if lengths is None:
        o, rem, dq, dk, dv = oracle_fixed(q, k, v, dout, ac, drem=drem)
    else:
        o, rem, dq, dk, dv = oracle_varlen(q, k, v, dout, lengths, ac, drem=drem)
    return o + rem[..., None] * vf, dq, dk, dv + rem[..., None] * df


def check(got, ref):
    for name, g, r in zip(("out", "dq", "dk", "dv"), got, ref):
        assert_close(name, g, r)


def run_fused_varlen(q, k, v, dout, lengths, ac=False, prepare=lambda t: t.to(DEV)):
    from stickbreaking_attention import sb_attn_varlen_fused
    qg, kg, vg = (prepare(t).requires_grad_() for t in (q, k, v))
    out = sb_attn_varlen_fused(qg, kg, vg, cu_from_lengths(lengths, device=DEV), max(lengths), zero_start=False,
                               attend_current=ac)
    grads = torch.autograd.grad(out, (qg, kg, vg), prepare(dout))
    torch.cuda.synchronize()
    return (out.detach(),) + grads


@pytest.mark.parametrize("lengths", [[1], [3, 1, 1, 2], [63, 64, 65, 127, 128, 129, 1, 31, 33], [257, 640]])
@pytest.mark.parametrize("ac", [False, True])
@pytest.mark.parametrize("d", [32, 64, 128, 256])
def test_fused_varlen_ragged_documents(lengths, ac, d):
    T = sum(lengths)
    q, k, v, dout = orc.make_inputs((3, T, d), 11 + T + d, dist="upstream")
    check(run_fused_varlen(q, k, v, dout, lengths, ac), fused_reference(q, k, v, dout, lengths, ac))


@pytest.mark.parametrize("product_space", [False, True])
def test_fused_varlen_long_documents_normal_inputs(product_space, monkeypatch):
    from stickbreaking_attention import _ops
    monkeypatch.setattr(_ops, "PRODUCT_SPACE", product_space)
    lengths = [1100, 437]
    q, k, v, dout = orc.make_inputs((2, sum(lengths), 128), 78)
    check(run_fused_varlen(q, k, v, dout, lengths), fused_reference(q, k, v, dout, lengths))


@pytest.mark.parametrize("B,H,T,d,ac", [(2, 3, 200, 64, False), (1, 2, 384, 128, True), (2, 2, 300, 32, True), (1, 2, 450, 256, False)])
def test_fused_fixed_length(B, H, T, d, ac):
    from stickbreaking_attention import sb_attn_fused
    q, k, v, dout = orc.make_inputs((B, H, T, d), 3 + T, dist="upstream")
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    out = sb_attn_fused(qg, kg, vg, attend_current=ac)
    grads = torch.autograd.grad(out, (qg, kg, vg), dout.to(DEV))
    torch.cuda.synchronize()
    check((out.detach(),) + grads, fused_reference(q, k, v, dout, None, ac))


def test_fused_agrees_with_the_two_output_operator():
    """Same kernels, same inputs: the fused result differs from composing the two bf16 outputs
    afterwards only by output rounding, and tokens outside every document stay zero."""
    from stickbreaking_attention import sb_attn_varlen, sb_attn_varlen_fused
    lengths, T = [300, 150], 500
    q, k, v, dout = orc.make_inputs((4, T, 128), 31)
    cu = cu_from_lengths(lengths, device=DEV)
    res = []
    for fused in (False, True):
        qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
        if fused:
            out = sb_attn_varlen_fused(qg, kg, vg, cu, max(lengths), zero_start=False)
        else:
            o, rem = sb_attn_varlen(qg, kg, vg, cu, max(lengths), zero_start=False)
            out = o.float() + rem.float()[..., None] * vg.float()
        res.append((out.detach().float(),) + tuple(g.float() for g in torch.autograd.grad(out, (qg, kg, vg), dout.to(DEV).to(out.dtype))))
    torch.cuda.synchronize()
    for name, a, b in zip(("out", "dq", "dk", "dv"), *res):
        assert (a - b).abs().max().item() <= 2e-2 + a.abs().max().item() * 2.0 ** -7, name
    out, dq, dk, dv = res[1]
    for t in (out, dq, dk, dv):
        assert torch.count_nonzero(t[:, sum(lengths):]).item() == 0


def test_fused_token_major_and_padded_head_dim():
    """v, the incoming gradient and the output all with token-major strides; head_dim 50 runs
    zero-padded to 64."""
    lengths, H, d = [212, 90], 4, 50
    q, k, v, dout = orc.make_inputs((H, sum(lengths), d), 6, dist="upstream")
    tm = lambda t: t.to(DEV).permute(1, 0, 2).contiguous().permute(1, 0, 2)
    check(run_fused_varlen(q, k, v, dout, lengths, prepare=tm), fused_reference(q, k, v, dout, lengths))


def test_fused_forward_only_needs_no_table():
    from stickbreaking_attention import sb_attn_varlen_fused
    q, k, v, _ = orc.make_inputs((2, 300, 64), 2)
    with torch.no_grad():
        out = sb_attn_varlen_fused(q.to(DEV), k.to(DEV), v.to(DEV), cu_from_lengths([300], device=DEV), 300,
                                   zero_start=False)
    o, rem = orc.sb_varlen(q.float(), k.float(), v.float(), [300])
    assert_close("out", out, o + rem[..., None] * v.float())
