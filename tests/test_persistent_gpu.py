"""The main kernel of the dk/dv pass has two launch forms: one workgroup per (key tile, head), or a
persistent launch of a fixed number of workgroups that draw their tiles from counters at the end of
the gradient table (own XCD's class first, then the classes of the other XCDs).  Every tile is
computed by the same instructions in the same order whichever workgroup takes it, so the two forms
must agree BIT FOR BIT; `sba_set_dkdv_workgroups` forces the persistent form with few workgroups so
that small problems walk many tiles per workgroup and exhaust and cross the classes."""
import os

import pytest
import torch

from tests import helpers as hp
from oracle import sb_oracle as orc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _lib():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from stickbreaking_attention import _native as nat
    assert os.path.exists(nat.LIB_PATH), "libsba.so must be built before the GPU tests run"
    lib = nat.load()
    yield lib
    lib.sba_set_dkdv_workgroups(0)


def _grads_varlen(lib, workgroups, q, k, v, do, cu, max_len, **kw):
    from stickbreaking_attention import sb_attn_varlen
    lib.sba_set_dkdv_workgroups(workgroups)
    qq, kk, vv = (t.detach().clone().requires_grad_() for t in (q, k, v))
    o, rem = sb_attn_varlen(qq, kk, vv, cu, max_len, zero_start=False, **kw)
    g = torch.autograd.grad(o, (qq, kk, vv), do)
    torch.cuda.synchronize()
    return [t.detach().clone() for t in g]


# (head_dim, heads, document lengths): d = 128 has no tail kernel (every key tile is an item of the main kernel),
# d <= 64 gives the main kernel all but the last tile of documents longer than 256 tokens
CASES = [
    (128, 4, [700, 130, 1, 515, 256, 33]),
    (128, 3, [1300, 129]),
    (64, 5, [900, 300, 257, 40, 1024]),
    (32, 2, [1500, 384]),
]


@pytest.mark.parametrize("d,H,lengths", CASES)
@pytest.mark.parametrize("attend_current", [False, True])
def test_persistent_launch_matches_one_workgroup_per_tile_bit_for_bit(_lib, d, H, lengths, attend_current):
    dev = torch.device("cuda:0")
    T = sum(lengths)
    q, k, v, do = (t.to(dev) for t in orc.make_inputs((H, T, d), 4242 + d + H))
    cu = hp.cu_from_lengths(lengths, device=dev)
    kw = dict(attend_current=attend_current)
    base = _grads_varlen(_lib, -1, q, k, v, do, cu, max(lengths), **kw)
    for wg in (8, 16, 40):       # 40 -> 40 workgroups, five per class
        got = _grads_varlen(_lib, wg, q, k, v, do, cu, max(lengths), **kw)
        for name, a, b in zip(("dq", "dk", "dv"), got, base):
            assert torch.equal(a, b), f"{name} differs between {wg} persistent workgroups and one workgroup per tile"
    # and the same call twice in a row (the dq pass has to clear the counters every time)
    again = _grads_varlen(_lib, 8, q, k, v, do, cu, max(lengths), **kw)
    for a, b in zip(again, base):
        assert torch.equal(a, b)


@pytest.mark.parametrize("seed", range(8))
def test_random_documents_walked_by_few_workgroups(_lib, seed):
    """Random splits with many short key tiles (items of one to five steps take every branch of the queue's
    counted waits and of the late-tile guards), 8 or 24 workgroups for a few hundred items."""
    import random
    rng = random.Random(1000 + seed)
    d = (128, 64, 128, 32)[seed % 4]
    H = rng.choice((1, 2, 3, 5))
    lengths = [rng.choice((1, 31, 32, 33, 64, 97, 128, 129, 160, 200, 255, 256, 257, 300, 511, 640, 900)) for _ in range(rng.randint(3, 9))]
    dev = torch.device("cuda:0")
    q, k, v, do = (t.to(dev) for t in orc.make_inputs((H, sum(lengths), d), 500 + seed))
    cu = hp.cu_from_lengths(lengths, device=dev)
    kw = dict(attend_current=bool(seed & 1))
    base = _grads_varlen(_lib, -1, q, k, v, do, cu, max(lengths), **kw)
    for wg in (8, 24):
        got = _grads_varlen(_lib, wg, q, k, v, do, cu, max(lengths), **kw)
        for name, a, b in zip(("dq", "dk", "dv"), got, base):
            assert torch.equal(a, b), f"seed {seed}, lengths {lengths}: {name} differs with {wg} persistent workgroups"


@pytest.mark.parametrize("d", [128, 64])
def test_log_space_carry_and_fused_output_with_persistent_workgroups(_lib, monkeypatch, d):
    """The two other instantiations of the kernel's step: the log2-space carry (no hand-pipelined block at all) and
    the fused output o + rem * v (rem joins the diagonal of P in the dk/dv pass)."""
    from stickbreaking_attention import _ops, sb_attn_varlen_fused
    dev = torch.device("cuda:0")
    H, lengths = 3, [650, 129, 300, 64]
    q, k, v, do = (t.to(dev) for t in orc.make_inputs((H, sum(lengths), d), 77 + d))
    cu = hp.cu_from_lengths(lengths, device=dev)
    monkeypatch.setattr(_ops, "PRODUCT_SPACE", False)
    base = _grads_varlen(_lib, -1, q, k, v, do, cu, max(lengths))
    got = _grads_varlen(_lib, 16, q, k, v, do, cu, max(lengths))
    for name, a, b in zip(("dq", "dk", "dv"), got, base):
        assert torch.equal(a, b), f"log space: {name} differs"
    monkeypatch.setattr(_ops, "PRODUCT_SPACE", True)
    outs = []
    for wg in (-1, 16):
        _lib.sba_set_dkdv_workgroups(wg)
        qq, kk, vv = (t.detach().clone().requires_grad_() for t in (q, k, v))
        out = sb_attn_varlen_fused(qq, kk, vv, cu, max(lengths), zero_start=False)
        outs.append(torch.autograd.grad(out, (qq, kk, vv), do))
        torch.cuda.synchronize()
    for name, a, b in zip(("dq", "dk", "dv"), outs[1], outs[0]):
        assert torch.equal(a, b), f"fused output: {name} differs"


def test_persistent_launch_against_the_oracle(_lib):
    dev = torch.device("cuda:0")
    d, H, lengths = 128, 2, [777, 128, 390]
    T = sum(lengths)
    q, k, v, do = (t.to(dev) for t in orc.make_inputs((H, T, d), 99))
    cu = hp.cu_from_lengths(lengths, device=dev)
    got = _grads_varlen(_lib, 8, q, k, v, do, cu, max(lengths))
    ref = orc.sb_varlen_grads(q.float().cpu(), k.float().cpu(), v.float().cpu(), lengths, do.float().cpu())
    for name, g, r in zip(("dq", "dk", "dv"), got, ref[2:5]):
        hp.assert_close(name, g, r)


def test_fixed_length_persistent_launch(_lib):
    from stickbreaking_attention import sb_attn
    dev = torch.device("cuda:0")
    q, k, v, do = (t.to(dev) for t in orc.make_inputs((2, 3, 1024, 64), 7))
    outs = []
    for wg in (-1, 8, 24):
        _lib.sba_set_dkdv_workgroups(wg)
        qq, kk, vv = (t.detach().clone().requires_grad_() for t in (q, k, v))
        o, rem = sb_attn(qq, kk, vv)
        outs.append(torch.autograd.grad(o, (qq, kk, vv), do))
        torch.cuda.synchronize()
    for other in outs[1:]:
        for a, b in zip(other, outs[0]):
            assert torch.equal(a, b)
