"""Pins the CPU oracle (oracle/sb_oracle.py) WITHOUT retyping its formulas: closed forms,
a float64 product-form double loop, invariants of the stick, finite differences and the
hand-derived backward.  A dropped term, a flipped mask, an off-by-one in the running sum or
a transposed operand fails at least one of these."""
import math

import pytest
import torch

from oracle import sb_oracle as orc


def rand(shape, seed, dtype=torch.float64, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g, dtype=torch.float64).to(dtype) * scale


# -- closed forms -----------------------------------------------------------------------------
@pytest.mark.parametrize("attend_current", [False, True])
def test_constant_logit_closed_form(attend_current):
    # q = 0 -> every logit 0 -> beta = 1/2: A[i,j] = 2^-(i-j) (strict) or 2^-(i-j+1); rem = 2^-(#visible)
    L, d = 40, 8
    q = torch.zeros(1, 1, L, d, dtype=torch.float64)
    k = rand((1, 1, L, d), 1)
    v = torch.ones(1, 1, L, d, dtype=torch.float64)
    mask, cw = orc.causal_mask_and_weights(L, attend_current, torch.float64)
    o, rem = orc.stickbreaking(q, k, v, mask, cw)
    nvis = torch.arange(L, dtype=torch.float64) + (1 if attend_current else 0)
    assert torch.allclose(rem[0, 0], 0.5 ** nvis, atol=1e-12)
    assert torch.allclose(o[0, 0, :, 0], 1 - 0.5 ** nvis, atol=1e-12)
    A = orc.attention_weights(q[0, 0], k[0, 0], attend_current)
    i, j = 17, 11
    assert abs(A[i, j].item() - 0.5 ** (i - j + (1 if attend_current else 0))) < 1e-14


def test_constant_nonzero_logit_geometric():
    # q = k = e_0 * a  ->  z = a^2/sqrt(d) = c for all pairs: A[i,j] = s (1-s)^(i-1-j), s = sigmoid(c)
    L, d, a = 30, 4, 1.3
    q = torch.zeros(L, d, dtype=torch.float64); q[:, 0] = a
    k = q.clone()
    s = 1 / (1 + math.exp(-a * a / math.sqrt(d)))
    A = orc.attention_weights(q, k)
    for (i, j) in [(1, 0), (9, 3), (29, 0), (29, 28)]:
        assert abs(A[i, j].item() - s * (1 - s) ** (i - 1 - j)) < 1e-13
    o, rem = orc.sb_document(q, k, torch.ones(L, d, dtype=torch.float64))
    assert torch.allclose(rem, (1 - s) ** torch.arange(L, dtype=torch.float64), atol=1e-13)


def test_length_two_textbook():
    q, k, v = rand((2, 8), 3), rand((2, 8), 4), rand((2, 8), 5)
    o, rem = orc.sb_document(q, k, v)
    z10 = float(q[1] @ k[0]) / math.sqrt(8)
    sig = 1 / (1 + math.exp(-z10))
    assert torch.allclose(o[0], torch.zeros(8, dtype=torch.float64))
    assert abs(rem[0].item() - 1.0) < 1e-15
    assert torch.allclose(o[1], sig * v[0], atol=1e-14)
    assert abs(rem[1].item() - (1 - sig)) < 1e-14


# -- independent product-form evaluation ------------------------------------------------------
@pytest.mark.parametrize("attend_current", [False, True])
@pytest.mark.parametrize("L,d", [(1, 4), (7, 16), (48, 8)])
def test_matches_bruteforce_product_form(L, d, attend_current):
    q, k, v = rand((L, d), 10 + L), rand((L, d), 20 + L), rand((L, d), 30 + L)
    o_bf, rem_bf, A_bf = orc.bruteforce(q, k, v, attend_current)
    mask, cw = orc.causal_mask_and_weights(L, attend_current, torch.float64)
    o1, rem1 = orc.stickbreaking(q[None, None], k[None, None], v[None, None], mask, cw)
    o2, rem2 = orc.sb_document(q, k, v, attend_current)
    o3, rem3 = orc.sb_document(q, k, v, attend_current, row_chunk=5)
    for o, rem in ((o1[0, 0], rem1[0, 0]), (o2, rem2), (o3, rem3)):
        assert torch.allclose(o, o_bf, atol=1e-12) and torch.allclose(rem, rem_bf, atol=1e-12)
    assert torch.allclose(orc.attention_weights(q, k, attend_current), A_bf, atol=1e-13)


def test_dense_and_running_sum_forms_agree_fp32():
    # the two fp32 formulations the parity tests and the CPU baseline use
    H, L, d = 3, 96, 16
    q, k, v = (rand((1, H, L, d), s, torch.float32) for s in (1, 2, 3))
    mask, cw = orc.causal_mask_and_weights(L)
    o1, r1 = orc.stickbreaking(q, k, v, mask, cw)
    o2, r2 = orc.sb_document(q, k, v)
    assert torch.allclose(o1, o2, atol=2e-5) and torch.allclose(r1, r2, atol=2e-5)


# -- invariants -------------------------------------------------------------------------------
@pytest.mark.parametrize("attend_current", [False, True])
def test_stick_invariants_and_causality(attend_current):
    L, d = 33, 8
    q, k, v = rand((L, d), 1, scale=2.0), rand((L, d), 2, scale=2.0), rand((L, d), 3)
    A = orc.attention_weights(q, k, attend_current)
    o, rem = orc.sb_document(q, k, v, attend_current)
    assert (A >= 0).all() and (rem >= -1e-15).all() and (rem <= 1 + 1e-15).all()
    assert torch.allclose(A.sum(-1) + rem, torch.ones(L, dtype=torch.float64), atol=1e-13)
    assert (A.triu(1 if attend_current else 0) == 0).all()
    # perturbing keys/values a row cannot see leaves the row unchanged
    i = 12
    k2, v2 = k.clone(), v.clone()
    first_hidden = i + 1 if attend_current else i
    k2[first_hidden:] += 5.0
    v2[first_hidden:] -= 3.0
    o2, rem2 = orc.sb_document(q, k2, v2, attend_current)
    assert torch.equal(o2[: i + 1], o[: i + 1]) and torch.equal(rem2[: i + 1], rem[: i + 1])


def test_attend_current_shifts_by_one_key():
    # strict weights of row i over keys 0..i-1 equal attend_current weights of a row that sees
    # exactly the same keys: query i placed at position i-1 of a sequence without key i.
    L, d = 20, 8
    q, k = rand((L, d), 7), rand((L, d), 8)
    A_strict = orc.attention_weights(q, k, False)
    i = 13
    qs = torch.cat([q[:i - 1], q[i:i + 1]])           # query i sits at index i-1
    A_ac = orc.attention_weights(qs, k[:i], True)
    assert torch.allclose(A_ac[i - 1, :i], A_strict[i, :i], atol=1e-14)


def test_documents_and_heads_are_independent():
    H, d = 2, 8
    lengths = [5, 1, 17, 9]
    T = sum(lengths)
    q, k, v = rand((H, T, d), 1), rand((H, T, d), 2), rand((H, T, d), 3)
    o, rem = orc.sb_varlen(q, k, v, lengths)
    o_dense, rem_dense = orc.sb_varlen(q, k, v, lengths, dense=True)
    assert torch.allclose(o, o_dense, atol=1e-12) and torch.allclose(rem, rem_dense, atol=1e-12)
    start = 0
    for n in lengths:
        for h in range(H):
            o1, r1, _ = orc.bruteforce(q[h, start:start + n], k[h, start:start + n], v[h, start:start + n])
            assert torch.allclose(o[h, start:start + n], o1, atol=1e-12)
            assert torch.allclose(rem[h, start:start + n], r1, atol=1e-12)
        start += n
    assert orc.lengths_from_cu_seqlens([0, 5, 6, 23, 32]) == lengths
    assert orc.lengths_from_cu_seqlens([5, 6, 23, 32]) == lengths


def test_tail_tokens_outside_documents_are_zero():
    q, k, v = rand((1, 10, 4), 1), rand((1, 10, 4), 2), rand((1, 10, 4), 3)
    o, rem = orc.sb_varlen(q, k, v, [4, 3])
    assert (o[:, 7:] == 0).all() and (rem[:, 7:] == 0).all()


# -- backward ---------------------------------------------------------------------------------
@pytest.mark.parametrize("attend_current", [False, True])
def test_autograd_matches_finite_differences(attend_current):
    L, d = 6, 4
    q, k, v = (rand((L, d), s).requires_grad_(True) for s in (1, 2, 3))
    fn = lambda a, b, c: orc.sb_document(a, b, c, attend_current)
    assert torch.autograd.gradcheck(fn, (q, k, v), eps=1e-6, atol=1e-6)


@pytest.mark.parametrize("attend_current", [False, True])
def test_analytic_backward_matches_autograd(attend_current):
    L, d = 37, 8
    q, k, v, do = (rand((L, d), s) for s in (1, 2, 3, 4))
    dr = rand((L,), 5)
    _, _, dq, dk, dv = orc.sb_fixed_grads(q, k, v, do, dr, attend_current)
    aq, ak, av = orc.analytic_backward(q, k, v, do, dr, attend_current)
    assert torch.allclose(dq, aq, atol=1e-11) and torch.allclose(dk, ak, atol=1e-11)
    assert torch.allclose(dv, av, atol=1e-11)


def test_row_sum_identity_of_G():
    # sum_j A[i,j] (do_i . v_j - drem_i) = do_i . o_i - drem_i (1 - rem_i)
    L, d = 25, 8
    q, k, v, do = (rand((L, d), s) for s in (1, 2, 3, 4))
    dr = rand((L,), 5)
    A = orc.attention_weights(q, k)
    o, rem = orc.sb_document(q, k, v)
    G = A * (do @ v.T - dr[:, None])
    assert torch.allclose(G.sum(-1), (do * o).sum(-1) - dr * (1 - rem), atol=1e-12)


def test_inv_temp_is_a_plain_logit_scale():
    L, d = 12, 8
    q, k, v = rand((L, d), 1), rand((L, d), 2), rand((L, d), 3)
    o1, r1 = orc.sb_document(q * 3.0, k, v, inv_temp=0.2)
    o2, r2 = orc.sb_document(q, k, v, inv_temp=0.6)
    assert torch.allclose(o1, o2, atol=1e-13) and torch.allclose(r1, r2, atol=1e-13)


def test_make_inputs_is_seeded_and_ordered():
    a = orc.make_inputs((2, 5, 4), 1337)
    b = orc.make_inputs((2, 5, 4), 1337)
    assert all(torch.equal(x, y) for x, y in zip(a, b))
    g = torch.Generator().manual_seed(1337)
    assert torch.equal(a[0], torch.randn((2, 5, 4), generator=g).to(torch.bfloat16))


def test_package_dense_definition_matches_the_oracle():
    # stickbreaking_attention.sb_ref mirrors the upstream import path (sb_ref.py:8-25); it must
    # agree with the oracle's dense form, which the closed forms and brute force above pin.
    from stickbreaking_attention.sb_ref import stickbreaking as dense
    torch.manual_seed(3)
    q, k, v = (torch.randn(2, 3, 40, 16, dtype=torch.float64) for _ in range(3))
    for ac in (False, True):
        mask, cw = orc.causal_mask_and_weights(40, ac)
        o1, r1 = dense(q, k, v, mask, cw)
        o2, r2 = orc.stickbreaking(q, k, v, mask, cw)
        assert torch.allclose(o1, o2, atol=1e-10) and torch.allclose(r1, r2, atol=1e-10)


def test_varlen_grads_match_bruteforce_and_analytic_backward_per_document():
    # the check the golden-fixture generator relies on: autograd through the packed-documents
    # driver == product-form double loop (forward) and hand-derived formulas (backward), per document
    H, lengths, d = 2, [70, 1, 150, 33], 16
    T = sum(lengths)
    for ac in (False, True):
        q, k, v, do = (t.double() for t in orc.make_inputs((H, T, d), 4242 + T, dist="upstream"))
        dr = torch.randn((H, T), generator=torch.Generator().manual_seed(99 + T)).to(torch.bfloat16).double()
        o, rem, dq, dk, dv = orc.sb_varlen_grads(q, k, v, lengths, do, dr, ac)
        start = 0
        for n in lengths:
            sl = slice(start, start + n)
            for h in range(H):
                ob, rb, _ = orc.bruteforce(q[h, sl], k[h, sl], v[h, sl], ac)
                assert torch.allclose(o[h, sl], ob, atol=1e-11) and torch.allclose(rem[h, sl], rb, atol=1e-11)
                aq, ak, av = orc.analytic_backward(q[h, sl], k[h, sl], v[h, sl], do[h, sl], dr[h, sl], ac)
                assert torch.allclose(dq[h, sl], aq, atol=1e-10) and torch.allclose(dk[h, sl], ak, atol=1e-10)
                assert torch.allclose(dv[h, sl], av, atol=1e-10)
            start += n
