"""GPU parity tests: the HIP path (through the Python operators, which call libsba.so through
its C ABI) against the fp32 CPU oracle on identical bf16-rounded inputs, against the
committed float64 fixtures, and -- at the benchmark's full sizes -- through properties that
need no oracle.  Tolerance: max-abs 2e-2 on o, rem, dq, dk, dv (see helpers.assert_close for
how bf16 output rounding of large values enters)."""
import math
import os

import numpy as np
import pytest
import torch

from oracle import sb_oracle as orc
from tests.helpers import (GOLDEN_DIR, assert_close, cu_from_lengths, doc_lengths, oracle_fixed,
                           oracle_varlen)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module", autouse=True)
def _need_gpu():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import ctypes
    from stickbreaking_attention import _native as nat
    assert os.path.exists(nat.LIB_PATH), "libsba.so must be built before the GPU tests run"
    nat.load()


def run_varlen(q, k, v, do, lengths, ac=False, drem=None, zero_start=False, cu_dtype=torch.int32,
               inv_temp=None, max_seqlens="auto"):
    from stickbreaking_attention import sb_attn_varlen
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    cu = cu_from_lengths(lengths, leading_zero=zero_start, dtype=cu_dtype, device=DEV)
    ms = max(lengths) if max_seqlens == "auto" else max_seqlens
    o, rem = sb_attn_varlen(qg, kg, vg, cu, ms, inv_temp=inv_temp, zero_start=zero_start, attend_current=ac)
    outs, grads = (o,), (do.to(DEV),)
    if drem is not None:
        outs, grads = (o, rem), (do.to(DEV), drem.to(DEV))
    dq, dk, dv = torch.autograd.grad(outs, (qg, kg, vg), grads)
    torch.cuda.synchronize()
    return o.detach(), rem.detach(), dq, dk, dv


def check_all(got, ref, heads=None):
    for name, g, r in zip(("o", "rem", "dq", "dk", "dv"), got, ref):
        if heads is not None:
            g = g[heads]
        assert_close(name, g, r)


# ---------------------------------------------------------------------------------------------
# committed fixtures (float64 expectations)
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name", ["a", "b", "c", "d"])
@pytest.mark.parametrize("product_space", [False, True])
def test_golden_fixture(name, product_space, monkeypatch):
    from stickbreaking_attention import _ops
    monkeypatch.setattr(_ops, "PRODUCT_SPACE", product_space)
    z = np.load(os.path.join(GOLDEN_DIR, "small_cases.npz"))
    t = {k: torch.from_numpy(z[f"{name}_{k}"]) for k in ("q", "k", "v", "do", "dr", "o", "rem", "dq", "dk", "dv")}
    lengths = [int(x) for x in z[f"{name}_lengths"]]
    ac = bool(z[f"{name}_ac"][0])
    bf = lambda x: x.to(torch.bfloat16)
    got = run_varlen(bf(t["q"]), bf(t["k"]), bf(t["v"]), bf(t["do"]), lengths, ac, drem=bf(t["dr"]))
    check_all(got, (t["o"], t["rem"], t["dq"], t["dk"], t["dv"]))


# ---------------------------------------------------------------------------------------------
# oracle comparisons on seeded inputs
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("product_space", [False, True])
def test_config1_shape(product_space, monkeypatch):
    """1 document x 512 tokens, 4 heads, d=64, N(0,1), strict causal."""
    from stickbreaking_attention import _ops
    monkeypatch.setattr(_ops, "PRODUCT_SPACE", product_space)
    q, k, v, do = orc.make_inputs((4, 512, 64), 1337 + 1)
    check_all(run_varlen(q, k, v, do, [512]), oracle_varlen(q, k, v, do, [512]))


@pytest.mark.parametrize("ac", [False, True])
def test_log_space_carry_on_long_documents(ac, monkeypatch):
    """The log2-sum variant of the kernels (the reference's formulation) over documents long enough
    to wrap the dk/dv pass's tile ring several times, head_dim 128."""
    from stickbreaking_attention import _ops
    monkeypatch.setattr(_ops, "PRODUCT_SPACE", False)
    lengths = [1100, 437]
    q, k, v, do = orc.make_inputs((2, sum(lengths), 128), 77)
    check_all(run_varlen(q, k, v, do, lengths, ac), oracle_varlen(q, k, v, do, lengths, ac))


@pytest.mark.parametrize("lengths", [[1], [2], [3, 1, 1, 2], [63, 64, 65, 127, 128, 129, 1, 31, 33], [257, 640]])
@pytest.mark.parametrize("ac", [False, True])
@pytest.mark.parametrize("d", [32, 64, 128, 256])
def test_ragged_documents(lengths, ac, d):
    T = sum(lengths)
    q, k, v, do = orc.make_inputs((3, T, d), 7 + T + d, dist="upstream")
    g = torch.Generator().manual_seed(T)
    drem = torch.randn((3, T), generator=g).to(torch.bfloat16)
    check_all(run_varlen(q, k, v, do, lengths, ac, drem=drem), oracle_varlen(q, k, v, do, lengths, ac, drem=drem))


def _poison_free_blocks(shape, n=6):
    # The operators allocate their outputs uninitialised; leave NaN patterns in the allocator's
    # free blocks of that size so that a row nobody writes cannot pass for a zero.
    blocks = [torch.full(shape, float("nan"), dtype=torch.bfloat16, device=DEV) for _ in range(n)]
    blocks += [torch.full(shape[:-1], float("nan"), dtype=torch.bfloat16, device=DEV) for _ in range(n)]
    torch.cuda.synchronize()
    del blocks


def test_rejected_cu_seqlens_raise_or_poison_the_outputs(monkeypatch):
    """Malformed cu_seqlens: with the host copy of cu_seqlens (the default) the call raises before
    anything is launched; without it (SBA_SYNC_FREE, torch.compile) the device scheduler refuses
    the input, no attention is computed and every output element is NaN -- never a plausible value."""
    from stickbreaking_attention import _ops, sb_attn_varlen
    q = torch.randn(2, 256, 64, device=DEV).to(torch.bfloat16)
    bad = torch.tensor([100, 50, 256], dtype=torch.int32, device=DEV)
    with pytest.raises(ValueError, match="non-decreasing"):
        sb_attn_varlen(q, q, q, bad, 256, zero_start=False)
    monkeypatch.setattr(_ops, "SYNC_FREE", True)
    _ops.release_workspaces()
    _poison_free_blocks((2, 256, 64))
    qg = q.clone().requires_grad_()
    o, rem = sb_attn_varlen(qg, qg, qg, bad, 256, zero_start=False)
    (dq,) = torch.autograd.grad(o, (qg,), torch.ones_like(o))
    torch.cuda.synchronize()
    assert torch.isnan(o).all() and torch.isnan(rem).all() and torch.isnan(dq).all()


def test_understated_max_seqlens(monkeypatch):
    """Upstream silently drops rows when max_seqlens under-states a document (sb_varlen_fwd.py:478).
    Here results do not depend on max_seqlens when the lengths are known on the host; without them
    the tables sized from the understated bound are too small, which the device detects: NaN
    outputs, and a ValueError when validation is switched on."""
    from stickbreaking_attention import _ops, sb_attn_varlen
    lengths = [700, 300]
    q, k, v, do = orc.make_inputs((2, 1000, 64), 77)
    ref = oracle_varlen(q, k, v, do, lengths)
    got = run_varlen(q, k, v, do, lengths, max_seqlens=64)          # default: lengths read back once, exact tables
    check_all(got, ref)
    monkeypatch.setattr(_ops, "SYNC_FREE", True)
    _ops.release_workspaces()
    got = run_varlen(q, k, v, do, lengths, max_seqlens=64)
    for t in got:
        assert torch.isnan(t).all()
    got = run_varlen(q, k, v, do, lengths, max_seqlens=700)         # a correct bound: same results as above
    check_all(got, ref)
    monkeypatch.setattr(_ops, "VALIDATE", True)
    with pytest.raises(ValueError, match="too small"):
        run_varlen(q, k, v, do, lengths, max_seqlens=64)


def test_understated_max_seqlens_with_roomy_tables(monkeypatch):
    """Without the lengths on the host the backward's launches are sized with max_seqlens.  A
    document longer than declared whose tables still fit (many short documents leave room) is seen
    by the device: the forward, which does not depend on the bound, is right; the backward
    returns NaN, and validation names the reason."""
    from stickbreaking_attention import _ops, sb_attn_varlen
    monkeypatch.setattr(_ops, "SYNC_FREE", True)
    _ops.release_workspaces()
    lengths = [300] + [20] * 60
    T = sum(lengths)
    q, k, v, do = orc.make_inputs((2, T, 64), 78)
    ref = oracle_varlen(q, k, v, do, lengths)
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    cu = cu_from_lengths(lengths, device=DEV)
    o, rem = sb_attn_varlen(qg, kg, vg, cu, 256, zero_start=False)          # 300 > 256
    dq, dk, dv = torch.autograd.grad(o, (qg, kg, vg), do.to(DEV))
    torch.cuda.synchronize()
    check_all((o.detach(), rem.detach()), ref[:2])
    for t in (dq, dk, dv):
        assert torch.isnan(t).all()
    monkeypatch.setattr(_ops, "VALIDATE", True)
    with pytest.raises(ValueError, match="longer than max_seqlens"):
        sb_attn_varlen(qg, kg, vg, cu, 256, zero_start=False)


def test_no_documents_give_zero_outputs():
    from stickbreaking_attention import sb_attn_varlen
    q = torch.randn(2, 128, 64, device=DEV).to(torch.bfloat16).requires_grad_()
    _poison_free_blocks((2, 128, 64))
    o, rem = sb_attn_varlen(q, q, q, torch.zeros(0, dtype=torch.int32, device=DEV), 128, zero_start=False)
    (dq,) = torch.autograd.grad(o, (q,), torch.ones_like(o))
    torch.cuda.synchronize()
    assert (o == 0).all() and (rem == 0).all() and (dq == 0).all()


def test_empty_documents_and_tail_tokens():
    # zero-length documents in the middle, and 40 tokens after the last document
    lengths = [50, 0, 0, 130, 0, 20]
    T = sum(lengths) + 40
    q, k, v, do = orc.make_inputs((2, T, 64), 11)
    _poison_free_blocks((2, T, 64))
    got = run_varlen(q, k, v, do, lengths)
    ref = oracle_varlen(q, k, v, do, lengths)
    check_all(got, ref)
    for t in got:
        assert (t[:, sum(lengths):] == 0).all(), "tokens outside every document must come back as zeros"


@pytest.mark.parametrize("ac", [False, True])
@pytest.mark.parametrize("d", [32, 64, 128, 256])
def test_key_tile_group_boundaries(d, ac, monkeypatch):
    """Document lengths on both sides of every boundary of the dk/dv pass's tile grouping (all key
    tiles of a document of up to 256 tokens and the last tile of a longer one go to the four-wave
    kernel at head_dim 64): 1, 32, 33, 128, 129, 255, 256, 257, 384, 385 tokens, with a gradient
    for rem as well, once with the lengths on the host and once with launches sized from the bound."""
    from stickbreaking_attention import _ops
    lengths = [257, 1, 128, 385, 33, 256, 129, 32, 384, 255]
    T = sum(lengths)
    q, k, v, do = orc.make_inputs((2, T, d), 4242 + d)
    drem = torch.randn((2, T), generator=torch.Generator().manual_seed(7)).to(torch.bfloat16)
    ref = oracle_varlen(q, k, v, do, lengths, ac, drem=drem)
    check_all(run_varlen(q, k, v, do, lengths, ac, drem=drem), ref)
    monkeypatch.setattr(_ops, "SYNC_FREE", True)
    _ops.release_workspaces()
    check_all(run_varlen(q, k, v, do, lengths, ac, drem=drem, max_seqlens=400), ref)


@pytest.mark.parametrize("ac", [False, True])
@pytest.mark.parametrize("H,L", [(3, 4096), (12, 4096), (3, 8192)])
def test_upstream_varlen_grid(H, L, ac):
    """The upstream test's own shapes and input distribution (single long document, d=128,
    q shifted +1, k shifted -1, int64 cu_seqlens, o + rem*v epilogue in the caller)."""
    from stickbreaking_attention import sb_attn_varlen
    q, k, v, do = orc.make_inputs((H, L, 128), 1337, dist="upstream")
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    cu = cu_from_lengths([L], dtype=torch.int64, device=DEV)
    o, rem = sb_attn_varlen(qg, kg, vg, cu_seqlens=cu, max_seqlens=L, inv_temp=1 / math.sqrt(128),
                            zero_start=False, attend_current=ac)
    out = o + rem[..., None] * vg
    dq, dk, dv = torch.autograd.grad(out, (qg, kg, vg), do.to(DEV))
    torch.cuda.synchronize()
    qf, kf, vf = (t.float().requires_grad_() for t in (q, k, v))
    ro, rrem = orc.sb_varlen(qf, kf, vf, [L], ac, row_chunk=1024)
    rout = ro + rrem[..., None] * vf
    rdq, rdk, rdv = torch.autograd.grad(rout, (qf, kf, vf), do.float())
    assert_close("o+rem*v", out.detach(), rout.detach())
    assert_close("dq", dq, rdq)
    assert_close("dk", dk, rdk)
    assert_close("dv", dv, rdv)


@pytest.mark.parametrize("ac", [False, True])
@pytest.mark.parametrize("B,H,T,d", [(2, 3, 500, 64), (1, 7, 256, 64), (2, 2, 1024, 128), (2, 3, 700, 32), (1, 2, 2048, 32),
                                     (2, 2, 700, 256)])
def test_fixed_length(B, H, T, d, ac):
    from stickbreaking_attention import sb_attn
    q, k, v, do = orc.make_inputs((B, H, T, d), 5 + T, dist="upstream")
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    o, rem = sb_attn(qg, kg, vg, attend_current=ac)
    dq, dk, dv = torch.autograd.grad(o, (qg, kg, vg), do.to(DEV))
    torch.cuda.synchronize()
    check_all((o.detach(), rem.detach(), dq, dk, dv), oracle_fixed(q, k, v, do, ac))


def test_config2_fixed_length_full():
    """B=4, H=16, T=2048, d=64, N(0,1): kernel on the full problem, oracle per batch entry."""
    from stickbreaking_attention import sb_attn
    q, k, v, do = orc.make_inputs((4, 16, 2048, 64), 1337 + 2)
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    o, rem = sb_attn(qg, kg, vg)
    dq, dk, dv = torch.autograd.grad(o, (qg, kg, vg), do.to(DEV))
    torch.cuda.synchronize()
    for b in range(4):
        print(f" batch {b}")
        ref = oracle_fixed(q[b:b + 1], k[b:b + 1], v[b:b + 1], do[b:b + 1])
        check_all(tuple(t[b:b + 1] for t in (o.detach(), rem.detach(), dq, dk, dv)), ref)


def test_config3_headline_varlen():
    """32 heads, d=128, 16384 tokens in 8 documents: kernel on the full problem; the oracle
    checks 4 of the 32 heads (all tokens) to stay within seconds."""
    lengths = doc_lengths("c3")
    q, k, v, do = orc.make_inputs((32, 16384, 128), 1337 + 3)
    got = run_varlen(q, k, v, do, lengths)
    heads = [0, 9, 22, 31]
    ref = oracle_varlen(q[heads], k[heads], v[heads], do[heads], lengths, row_chunk=1024)
    check_all(got, ref, heads=heads)


def test_config4_many_short_documents():
    """32 heads, d=64, 16384 tokens in ~200 documents of 16..256 tokens, zero_start=True."""
    lengths = doc_lengths("c4")
    q, k, v, do = orc.make_inputs((32, 16384, 64), 1337 + 4)
    got = run_varlen(q, k, v, do, lengths, zero_start=True)
    heads = list(range(0, 32, 4))
    ref = oracle_varlen(q[heads], k[heads], v[heads], do[heads], lengths)
    check_all(got, ref, heads=heads)


def test_config5_long_context_forward():
    """32 heads, d=128, 65536 tokens (one 32768-token document + 6 more), inputs x0.5, forward
    only.  Oracle: heads 0 and 17, all rows, evaluated 1024 query rows at a time."""
    from stickbreaking_attention import sb_attn_varlen
    lengths = doc_lengths("c5")
    q, k, v, _ = orc.make_inputs((32, 65536, 128), 1337 + 5, scale=0.5)
    cu = cu_from_lengths(lengths, device=DEV)
    with torch.no_grad():
        o, rem = sb_attn_varlen(q.to(DEV), k.to(DEV), v.to(DEV), cu, max(lengths), zero_start=False)
    torch.cuda.synchronize()
    assert torch.isfinite(o.float()).all() and torch.isfinite(rem.float()).all()
    heads = [0, 17]
    with torch.no_grad():
        ro, rrem = orc.sb_varlen(q[heads].float(), k[heads].float(), v[heads].float(), lengths, row_chunk=1024)
    assert_close("o", o[heads], ro)
    assert_close("rem", rem[heads], rrem)


# ---------------------------------------------------------------------------------------------
# properties at full size (no oracle)
# ---------------------------------------------------------------------------------------------
def test_full_size_properties_config3():
    from stickbreaking_attention import sb_attn, sb_attn_varlen
    lengths = doc_lengths("c3")
    q, k, v, _ = orc.make_inputs((32, 16384, 128), 1337 + 3)
    q, k, v = q.to(DEV), k.to(DEV), v.to(DEV)
    cu = cu_from_lengths(lengths, device=DEV)
    with torch.no_grad():
        o, rem = sb_attn_varlen(q, k, v, cu, max(lengths), zero_start=False)
        # (1) with v == 1 every output column is the stick that was used: o = 1 - rem
        ones = torch.ones_like(v)
        o1, rem1 = sb_attn_varlen(q, k, ones, cu, max(lengths), zero_start=False)
        assert torch.equal(rem1, rem)
        assert ((o1.float() - (1 - rem1.float())[..., None]).abs().max().item()) < 1e-2
        assert (rem.float() >= 0).all() and (rem.float() <= 1).all()
        # (2) first token of every document: o = 0, rem = 1
        starts = [0] + list(np.cumsum(lengths)[:-1])
        assert (o[:, starts] == 0).all() and (rem[:, starts] == 1).all()
        # (3) document independence: the packed result equals each document run on its own
        s = 0
        for n in lengths[:3]:
            od, remd = sb_attn(q[None, :, s:s + n], k[None, :, s:s + n], v[None, :, s:s + n])
            assert torch.equal(od[0], o[:, s:s + n]) and torch.equal(remd[0], rem[:, s:s + n])
            s += n
        # (4) the op is linear in v
        o2, _ = sb_attn_varlen(q, k, (2 * v), cu, max(lengths), zero_start=False)
        assert ((o2.float() - 2 * o.float()).abs().max().item()) < 3e-2
    torch.cuda.synchronize()


def test_backward_is_deterministic():
    lengths = [700, 300, 1100]
    q, k, v, do = orc.make_inputs((4, sum(lengths), 128), 3)
    a = run_varlen(q, k, v, do, lengths)
    b = run_varlen(q, k, v, do, lengths)
    for x, y in zip(a, b):
        assert torch.equal(x, y)


# ---------------------------------------------------------------------------------------------
# API behaviour
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("ac", [False, True])
def test_later_tokens_cannot_reach_earlier_rows(ac):
    """Exact causality: replacing the keys and values of every token after position c leaves the
    rows up to c bit-identical (a masked weight must be exactly zero, not zero to rounding)."""
    from stickbreaking_attention import sb_attn_varlen
    lengths, c = [333, 180], 201
    q, k, v, _ = orc.make_inputs((2, sum(lengths), 128), 15)
    cu = cu_from_lengths(lengths, device=DEV)
    k2, v2 = k.clone(), v.clone()
    k2[:, c + 1:lengths[0]] = 3.0
    v2[:, c + 1:lengths[0]] = -50.0
    with torch.no_grad():
        o1, r1 = sb_attn_varlen(q.to(DEV), k.to(DEV), v.to(DEV), cu, max(lengths), zero_start=False, attend_current=ac)
        o2, r2 = sb_attn_varlen(q.to(DEV), k2.to(DEV), v2.to(DEV), cu, max(lengths), zero_start=False, attend_current=ac)
    torch.cuda.synchronize()
    assert torch.equal(o1[:, :c + 1], o2[:, :c + 1]) and torch.equal(r1[:, :c + 1], r2[:, :c + 1])
    assert torch.equal(o1[:, lengths[0]:], o2[:, lengths[0]:])
    assert not torch.equal(o1[:, c + 2:lengths[0]], o2[:, c + 2:lengths[0]])


@pytest.mark.parametrize("lengths", [[4] * 4096, [3] * 5000 + [700], [1] * 2000 + [129] * 20],
                         ids=["4096x4", "5000x3+700", "2000x1+20x129"])
def test_thousands_of_tiny_documents(lengths):
    """The device scheduler with thousands of documents, below and above the number it still
    ranks by length."""
    q, k, v, do = orc.make_inputs((2, sum(lengths), 64), 3)
    check_all(run_varlen(q, k, v, do, lengths), oracle_varlen(q, k, v, do, lengths))


def test_zero_start_int64_and_inv_temp():
    lengths = [100, 260, 77]
    q, k, v, do = orc.make_inputs((2, sum(lengths), 64), 21)
    got = run_varlen(q, k, v, do, lengths, zero_start=True, cu_dtype=torch.int64, inv_temp=0.2)
    check_all(got, oracle_varlen(q, k, v, do, lengths, inv_temp=0.2))


def test_token_major_layout_keeps_strides():
    """Inputs stored [tokens, heads, d] and viewed as [heads, tokens, d] (how the upstream
    benchmark feeds the op): o keeps q's strides, results unchanged."""
    from stickbreaking_attention import sb_attn_varlen
    lengths = [300, 212]
    T, H, d = sum(lengths), 4, 128
    q, k, v, do = orc.make_inputs((H, T, d), 5)
    tm = lambda t: t.to(DEV).permute(1, 0, 2).contiguous().permute(1, 0, 2)
    qg, kg, vg = (tm(t).requires_grad_() for t in (q, k, v))
    assert qg.stride() == (d, H * d, 1)
    o, rem = sb_attn_varlen(qg, kg, vg, cu_from_lengths(lengths, device=DEV), max(lengths), zero_start=False)
    assert o.stride() == qg.stride() and o.dtype == torch.bfloat16 and rem.shape == (H, T)
    dq, dk, dv = torch.autograd.grad(o, (qg, kg, vg), tm(do))
    torch.cuda.synchronize()
    check_all((o.detach(), rem.detach(), dq, dk, dv), oracle_varlen(q, k, v, do, lengths))


@pytest.mark.parametrize("d", [16, 32, 50, 96, 160, 200])
def test_other_head_dims_run_zero_padded(d):
    """Upstream's fixed-length test grid (tests/test_attn.py:39: 64, 32, 16, 50).  32 has kernels of its
    own; 16 is padded to 32, 50 to 64, 96 to 128, 160 and 200 to 256."""
    from stickbreaking_attention import sb_attn
    q, k, v, do = orc.make_inputs((1, 2, 200, d), d, dist="upstream")
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    o, rem = sb_attn(qg, kg, vg)
    assert o.shape == q.shape
    dq, dk, dv = torch.autograd.grad(o, (qg, kg, vg), do.to(DEV))
    torch.cuda.synchronize()
    check_all((o.detach(), rem.detach(), dq, dk, dv), oracle_fixed(q, k, v, do))


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_other_dtypes_keep_their_dtype(dtype):
    from stickbreaking_attention import sb_attn
    q, k, v, do = orc.make_inputs((1, 2, 160, 64), 9, dist="upstream")   # bf16-representable values
    qg, kg, vg = (t.to(DEV).to(dtype).requires_grad_() for t in (q, k, v))
    o, rem = sb_attn(qg, kg, vg)
    assert o.dtype == dtype and rem.dtype == dtype
    dq, dk, dv = torch.autograd.grad(o, (qg, kg, vg), do.to(DEV).to(dtype))
    assert dq.dtype == dtype and dk.dtype == dtype
    torch.cuda.synchronize()
    check_all((o.detach(), rem.detach(), dq, dk, dv), oracle_fixed(q, k, v, do))


def test_malformed_cu_seqlens_are_reported(monkeypatch):
    from stickbreaking_attention import _ops, sb_attn_varlen
    q = torch.zeros(2, 256, 64, dtype=torch.bfloat16, device=DEV)
    for sync_free in (False, True):          # host-side check by default, device status word otherwise
        monkeypatch.setattr(_ops, "SYNC_FREE", sync_free)
        monkeypatch.setattr(_ops, "VALIDATE", sync_free)
        _ops.release_workspaces()
        with pytest.raises(ValueError, match="non-decreasing"):
            sb_attn_varlen(q, q, q, torch.tensor([100, 50, 256], dtype=torch.int32, device=DEV), 256, zero_start=False)
        with pytest.raises(ValueError, match="non-decreasing"):
            sb_attn_varlen(q, q, q, torch.tensor([100, 300], dtype=torch.int32, device=DEV), 256, zero_start=False)
        with pytest.raises(AssertionError):
            sb_attn_varlen(q, q, q, torch.tensor([5, 256], dtype=torch.int32, device=DEV), 256, zero_start=True)
    torch.cuda.synchronize()


def test_many_documents_at_head_dim_128_stay_inside_the_key_tile_list():
    """Ten documents in 2112 tokens at head_dim 128: the launch bounds of the dk/dv pass's two tile
    groups add up to more tiles than the key-tile list has room for, and every workgroup reads its
    tile before it knows the list's true length -- the grid must stop at the room."""
    lengths = [292, 2, 403, 193, 151, 369, 257, 244, 161, 0]
    T = sum(lengths) + 40
    q, k, v, do = orc.make_inputs((1, T, 128), 1208, dist="upstream")
    check_all(run_varlen(q, k, v, do, lengths, True, max_seqlens=420), oracle_varlen(q, k, v, do, lengths, True))


def test_gradient_through_rem_alone():
    """Only ``rem`` is differentiated: the gradient of ``o`` arrives as None (the functions do not ask
    PyTorch to materialise zeros for unused outputs) and must behave as zeros."""
    from stickbreaking_attention import sb_attn, sb_attn_varlen
    lengths = [150, 90]
    q, k, v, _ = orc.make_inputs((2, sum(lengths), 64), 17)
    drem = torch.randn((2, sum(lengths)), generator=torch.Generator().manual_seed(3)).to(torch.bfloat16)
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    o, rem = sb_attn_varlen(qg, kg, vg, cu_from_lengths(lengths, device=DEV), max(lengths), zero_start=False)
    dq, dk, dv = torch.autograd.grad(rem, (qg, kg, vg), drem.to(DEV))
    torch.cuda.synchronize()
    ref = oracle_varlen(q, k, v, torch.zeros_like(q), lengths, False, drem=drem)
    check_all((o.detach(), rem.detach(), dq, dk, dv), ref)
    qf, kf, vf = (t[None].to(DEV).requires_grad_() for t in (q[:, :150], k[:, :150], v[:, :150]))
    o2, rem2 = sb_attn(qf, kf, vf)
    g2 = torch.autograd.grad(rem2, (qf, kf, vf), drem[None, :, :150].to(DEV))
    torch.cuda.synchronize()
    for a, b in zip(g2, (dq, dk, dv)):
        assert torch.equal(a[0], b[:, :150])


@pytest.mark.parametrize("fixed", [False, True])
def test_backward_can_rebuild_the_carry_table(fixed, monkeypatch):
    """SBA_RECOMPUTE_TABLE: the forward keeps no table (a layer holds q, k, v only), the backward runs
    the forward kernel again to rebuild it.  Same kernels on the same inputs: identical bits."""
    from stickbreaking_attention import _ops, sb_attn, sb_attn_varlen
    lengths = [700, 130, 41]
    shape = (2, 3, 600, 64) if fixed else (3, sum(lengths), 128)
    q, k, v, do = orc.make_inputs(shape, 55)
    drem = torch.randn(shape[:-1], generator=torch.Generator().manual_seed(9)).to(torch.bfloat16)
    cu = cu_from_lengths(lengths, device=DEV)

    def run():
        qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
        o, rem = sb_attn(qg, kg, vg) if fixed else sb_attn_varlen(qg, kg, vg, cu, max(lengths), zero_start=False)
        saved = [t for t in o.grad_fn.saved_tensors if t.dtype == torch.float32]
        grads = torch.autograd.grad((o, rem), (qg, kg, vg), (do.to(DEV), drem.to(DEV)))
        torch.cuda.synchronize()
        return (o.detach(), rem.detach()) + grads, sum(t.numel() for t in saved)

    plain, kept = run()
    monkeypatch.setattr(_ops, "RECOMPUTE_TABLE", True)
    rebuilt, kept2 = run()
    assert kept > 0 and kept2 == 0, "with the switch on no fp32 table may be saved for the backward"
    for name, a, b in zip(("o", "rem", "dq", "dk", "dv"), plain, rebuilt):
        assert torch.equal(a, b), name


def test_forward_only_needs_no_table():
    from stickbreaking_attention import sb_attn_varlen
    q, k, v, _ = orc.make_inputs((2, 300, 64), 2)
    with torch.no_grad():
        o, rem = sb_attn_varlen(q.to(DEV), k.to(DEV), v.to(DEV), cu_from_lengths([300], device=DEV), 300, zero_start=False)
    ro, rrem = orc.sb_varlen(q.float(), k.float(), v.float(), [300])
    assert_close("o", o, ro)
    assert_close("rem", rem, rrem)


# ---------------------------------------------------------------------------------------------
# torch.compile: the launchers are opaque operators under upstream's names (utils.py:20-39),
# so a model that calls the attention traces into ONE graph
# ---------------------------------------------------------------------------------------------
def test_torch_compile_traces_through_the_registered_operators():
    from stickbreaking_attention import sb_attn, sb_attn_varlen
    lengths = [200, 56]
    q, k, v, do = orc.make_inputs((2, sum(lengths), 64), 21)
    cu = cu_from_lengths(lengths, device=DEV)

    def block(q, k, v):
        o, rem = sb_attn_varlen(q, k, v, cu, max(lengths), zero_start=False)
        return o + rem[..., None] * v          # the epilogue every caller applies (tests/test_varlen.py:101)

    compiled = torch.compile(block, fullgraph=True, backend="aot_eager")
    outs = []
    for fn in (block, compiled):
        qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
        y = fn(qg, kg, vg)
        outs.append((y.detach(),) + torch.autograd.grad(y, (qg, kg, vg), do.to(DEV)))
    torch.cuda.synchronize()
    for a, b in zip(*outs):
        assert torch.equal(a, b), "the compiled graph must run the same kernels as eager mode"

    qf, kf, vf, dof = orc.make_inputs((1, 2, 160, 64), 22)

    def fixed_block(q, k, v):
        o, rem = sb_attn(q, k, v)
        return o + rem[..., None] * v

    cfix = torch.compile(fixed_block, fullgraph=True, backend="aot_eager")
    outs = []
    for fn in (fixed_block, cfix):
        qg, kg, vg = (t.to(DEV).requires_grad_() for t in (qf, kf, vf))
        y = fn(qg, kg, vg)
        outs.append((y.detach(),) + torch.autograd.grad(y, (qg, kg, vg), dof.to(DEV)))
    torch.cuda.synchronize()
    for a, b in zip(*outs):
        assert torch.equal(a, b)


def test_cu_seqlens_are_read_back_once_per_tensor():
    """The leading-zero assertion and the table sizing read the device once per cu_seqlens tensor,
    not once per call, and still see a new or modified tensor."""
    from stickbreaking_attention import _ops, sb_attn_varlen
    _ops.release_workspaces()
    q = torch.zeros(2, 256, 64, dtype=torch.bfloat16, device=DEV)
    cu = torch.tensor([0, 100, 256], dtype=torch.int32, device=DEV)
    sb_attn_varlen(q, q, q, cu, 256)
    assert any(e[0]() is cu and e[2] == (0, 100, 256) for e in _ops._host_cu_cache)
    reads = []
    orig = torch.Tensor.tolist
    try:
        torch.Tensor.tolist = lambda self: (reads.append(1), orig(self))[1]
        sb_attn_varlen(q, q, q, cu, 256)                   # same tensor: no second read
        assert not reads
    finally:
        torch.Tensor.tolist = orig
    cu[0] = 3                                              # in-place change bumps the version: read again
    with pytest.raises(AssertionError):
        sb_attn_varlen(q, q, q, cu, 256)
    with pytest.raises(AssertionError):
        sb_attn_varlen(q, q, q, torch.tensor([5, 256], dtype=torch.int32, device=DEV), 256)
    torch.cuda.synchronize()
