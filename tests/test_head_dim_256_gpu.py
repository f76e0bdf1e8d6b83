"""head_dim 256 (upstream takes any head_dim through BLOCK_D = next_power_of_2(d), sb_varlen_fwd.py:479).
The forward and the dq pass are the kernels of the smaller head dims instantiated with one wave per
SIMD; the dk/dv pass is a kernel of its own kind (four independent waves per key tile, the queries
streamed through LDS, two passes: dv, then dk).  Everything here goes against the fp32 CPU oracle
with the gate of the other head dims: max-abs 2e-2 before the output's own bf16 rounding."""
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


def _run(q, k, v, do, lengths, ac=False, drem=None, fused=False):
    from stickbreaking_attention import sb_attn_varlen, sb_attn_varlen_fused
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    cu = cu_from_lengths(lengths, device=DEV)
    if fused:
        out = sb_attn_varlen_fused(qg, kg, vg, cu, max(lengths), zero_start=False, attend_current=ac)
        grads = torch.autograd.grad(out, (qg, kg, vg), do.to(DEV))
        torch.cuda.synchronize()
        return (out.detach(),) + grads
    o, rem = sb_attn_varlen(qg, kg, vg, cu, max(lengths), zero_start=False, attend_current=ac)
    outs, gs = ((o,), (do.to(DEV),)) if drem is None else ((o, rem), (do.to(DEV), drem.to(DEV)))
    grads = torch.autograd.grad(outs, (qg, kg, vg), gs)
    torch.cuda.synchronize()
    return (o.detach(), rem.detach()) + grads


@pytest.mark.parametrize("product_space", [False, True])
@pytest.mark.parametrize("ac", [False, True])
def test_long_documents(ac, product_space, monkeypatch):
    """Documents of 23 and 5 key tiles and a short one: the streamed query blocks wrap the two LDS buffers many
    times in both passes of the dk/dv kernel; a gradient for rem as well."""
    from stickbreaking_attention import _ops
    monkeypatch.setattr(_ops, "PRODUCT_SPACE", product_space)
    lengths = [2900, 611, 77]
    T = sum(lengths)
    q, k, v, do = orc.make_inputs((2, T, 256), 256 + int(ac))
    drem = torch.randn((2, T), generator=torch.Generator().manual_seed(3)).to(torch.bfloat16)
    ref = oracle_varlen(q, k, v, do, lengths, ac, drem=drem, row_chunk=1024)
    for name, g, r in zip(("o", "rem", "dq", "dk", "dv"), _run(q, k, v, do, lengths, ac, drem=drem), ref):
        assert_close(name, g, r)


@pytest.mark.parametrize("seed", range(6))
def test_random_documents(seed):
    import random
    rng = random.Random(2560 + seed)
    H = rng.choice((1, 2, 3))
    lengths = [rng.choice((1, 2, 31, 32, 33, 64, 97, 127, 128, 129, 160, 255, 256, 257, 300, 385, 511, 640, 900)) for _ in range(rng.randint(1, 8))]
    ac = bool(seed & 1)
    q, k, v, do = orc.make_inputs((H, sum(lengths), 256), 900 + seed, dist="upstream" if seed % 3 == 0 else "normal")
    ref = oracle_varlen(q, k, v, do, lengths, ac)
    for name, g, r in zip(("o", "rem", "dq", "dk", "dv"), _run(q, k, v, do, lengths, ac), ref):
        assert_close(f"seed {seed} {name}", g, r)


def test_fused_output_on_long_documents():
    lengths = [1100, 437]
    q, k, v, dout = orc.make_inputs((2, sum(lengths), 256), 78)
    qf, kf, vf = (t.float().requires_grad_() for t in (q, k, v))
    ro, rrem = orc.sb_varlen(qf, kf, vf, lengths, False)
    rout = ro + rrem[..., None] * vf
    rg = torch.autograd.grad(rout, (qf, kf, vf), dout.float())
    got = _run(q, k, v, dout, lengths, fused=True)
    for name, g, r in zip(("o+rem*v", "dq", "dk", "dv"), got, (rout.detach(),) + rg):
        assert_close(name, g, r)


def test_fixed_length_batch():
    from stickbreaking_attention import sb_attn
    q, k, v, do = orc.make_inputs((2, 3, 1024, 256), 31)
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    o, rem = sb_attn(qg, kg, vg, attend_current=True)
    dq, dk, dv = torch.autograd.grad(o, (qg, kg, vg), do.to(DEV))
    torch.cuda.synchronize()
    for name, g, r in zip(("o", "rem", "dq", "dk", "dv"), (o.detach(), rem.detach(), dq, dk, dv), oracle_fixed(q, k, v, do, True)):
        assert_close(name, g, r)


def test_rebuilt_table_and_repeat_are_bit_identical(monkeypatch):
    """The table-only forward at head_dim 256 rebuilds exactly the table the forward wrote, and the backward is
    deterministic (no atomics in any of its kernels)."""
    from stickbreaking_attention import _ops
    lengths = [700, 130, 41]
    q, k, v, do = orc.make_inputs((3, sum(lengths), 256), 55)
    first = _run(q, k, v, do, lengths)
    again = _run(q, k, v, do, lengths)
    monkeypatch.setattr(_ops, "RECOMPUTE_TABLE", True)
    rebuilt = _run(q, k, v, do, lengths)
    for name, a, b, c in zip(("o", "rem", "dq", "dk", "dv"), first, again, rebuilt):
        assert torch.equal(a, b), f"{name}: two runs differ"
        assert torch.equal(a, c), f"{name}: differs with the table rebuilt"


def test_token_major_strides_and_padding_from_200():
    """[tokens, heads, 200] storage viewed as [heads, tokens, 200]: zero-padded to 256 on the way in, sliced on the
    way out."""
    from stickbreaking_attention import sb_attn_varlen
    lengths, H, d = [300, 200], 2, 200
    T = sum(lengths)
    q, k, v, do = orc.make_inputs((H, T, d), 12)
    tm = lambda t: t.to(DEV).transpose(0, 1).contiguous().transpose(0, 1)
    qg, kg, vg = (tm(t).requires_grad_() for t in (q, k, v))
    o, rem = sb_attn_varlen(qg, kg, vg, cu_from_lengths(lengths, device=DEV), max(lengths), zero_start=False)
    assert o.shape == (H, T, d)
    dq, dk, dv = torch.autograd.grad(o, (qg, kg, vg), tm(do))
    torch.cuda.synchronize()
    for name, g, r in zip(("o", "rem", "dq", "dk", "dv"), (o.detach(), rem.detach(), dq, dk, dv), oracle_varlen(q, k, v, do, lengths)):
        assert_close(name, g, r)


def test_head_dims_beyond_256_are_refused():
    from stickbreaking_attention import sb_attn
    q = torch.zeros((1, 1, 64, 257), dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ValueError, match="head_dim 257 is not supported"):
        sb_attn(q, q, q)
