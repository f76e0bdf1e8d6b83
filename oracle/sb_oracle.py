"""CPU oracle for stick-breaking attention.  TEST INFRASTRUCTURE ONLY.

This module restates, for the CPU, the mathematics of the upstream PyTorch
reference ``stickbreaking_attention/sb_ref.py:8-25`` and of the drivers the
upstream tests wrap around it (``tests/test_varlen.py:10-41``,
``tests/test_attn.py:10-32``).  Nothing in the shipped package imports it: only
the test-suite, the smoke check and the CPU-baseline leg of the benchmark do,
and only as the checker.

Every function below is pinned by tests that do not retype its formula
(``tests/test_oracle.py``): closed forms for constant logits, a float64
product-form double loop, the stick invariant ``sum(A) + rem == 1``, causality
and document independence, ``torch.autograd.gradcheck`` finite differences and
the hand-derived analytic backward.

Definitions (one head, one causal document of length L, scale s = 1/sqrt(d)):

    z[i,j]  = s * <q_i, k_j>
    beta    = sigmoid(z)
    A[i,j]  = beta[i,j] * prod_{j<k<i} (1 - beta[i,k])        j <  i  (strict)
              beta[i,j] * prod_{j<k<=i}(1 - beta[i,k])        j <= i  (attend_current)
    o_i     = sum_j A[i,j] v_j
    rem_i   = 1 - sum_j A[i,j]
"""
from __future__ import annotations

import math
from typing import Optional, Sequence, Tuple

import torch
import torch.nn.functional as F

MASK_FILL = -1e5  # the reference fills masked log-weights with -1e5, not -inf (sb_ref.py:17)


# ---------------------------------------------------------------------------------------------
# 1. Dense restatement with the reference's signature (sb_ref.py:8-25)
# ---------------------------------------------------------------------------------------------
def stickbreaking(q, k, v, mask, cum_weight):
    """Dense O(L^3) formulation, argument-for-argument the reference's oracle.

    q, k, v    : [b, h, L, d]
    mask       : [L, L] bool, True = key NOT visible (triu(0) strict, triu(1) attend_current)
    cum_weight : [L, L], ones below the diagonal (tril(-1)); contracting the key axis
                 with it yields, at key column c, the sum over keys j > c.

    Follows sb_ref.py:12 (scaled logits), :17 (log sigmoid(z), masked to -1e5),
    :19 (log(1-sigmoid(z)) = logsigmoid(-z), masked to 0), :21-22 (contraction with
    cum_weight), :23-25 (exp, weighted sum, remainder).  Intermediates are rounded back to
    the dtype of the logits like the reference does (a no-op for fp32/fp64 inputs).
    """
    d = q.shape[-1]
    z = torch.matmul(q, k.transpose(-2, -1)) * (1.0 / math.sqrt(d))
    in_dtype = z.dtype
    zf = z.float() if z.dtype in (torch.bfloat16, torch.float16) else z
    log_hit = F.logsigmoid(zf).masked_fill(mask, MASK_FILL).to(in_dtype)
    log_miss = F.logsigmoid(-zf).masked_fill(mask, 0.0).to(in_dtype)
    later_miss = torch.einsum("bhij,jc->bhic", log_miss, cum_weight.to(log_miss))
    att = torch.exp(log_hit + later_miss)
    return torch.matmul(att, v), 1.0 - att.sum(dim=-1)


def causal_mask_and_weights(length: int, attend_current: bool = False, dtype=torch.float32):
    """The (mask, cum_weight) pair the upstream tests build (tests/test_varlen.py:13-14)."""
    cum_weight = torch.ones(length, length, dtype=dtype).tril(-1)
    mask = torch.ones(length, length).triu(1 if attend_current else 0).bool()
    return mask, cum_weight


# ---------------------------------------------------------------------------------------------
# 2. O(L^2) formulation: the same log-space weights with a reversed running sum instead of
#    the dense contraction.  Used for the big configurations where L^3 is out of reach.
# ---------------------------------------------------------------------------------------------
def attention_weights(q, k, attend_current: bool = False, inv_temp: Optional[float] = None):
    """Stick-breaking weights A [..., L, L] for one causal document per leading index."""
    L, d = q.shape[-2], q.shape[-1]
    s = (1.0 / math.sqrt(d)) if inv_temp is None else inv_temp
    z = torch.matmul(q, k.transpose(-2, -1)) * s
    visible = torch.ones(L, L, dtype=torch.bool, device=q.device).tril(0 if attend_current else -1)
    log_miss = torch.where(visible, F.logsigmoid(-z), torch.zeros_like(z))
    # suffix[i, j] = sum_{c > j} log_miss[i, c]  (exclusive, reversed running sum along keys)
    incl = torch.flip(torch.cumsum(torch.flip(log_miss, dims=(-1,)), dim=-1), dims=(-1,))
    suffix = incl - log_miss
    log_a = F.logsigmoid(z) + suffix
    return torch.where(visible, torch.exp(log_a), torch.zeros_like(z))


def sb_document(q, k, v, attend_current: bool = False, inv_temp: Optional[float] = None,
                row_chunk: int = 0):
    """(o, rem) for q,k,v [..., L, d]; every leading index is an independent causal document.

    ``row_chunk`` > 0 evaluates that many query rows at a time (memory O(chunk * L)), each
    chunk only against the keys it can see; results are identical to the unchunked path up
    to fp summation order inside matmul.
    """
    L = q.shape[-2]
    if row_chunk <= 0 or row_chunk >= L:
        a = attention_weights(q, k, attend_current, inv_temp)
        return torch.matmul(a, v), 1.0 - a.sum(dim=-1)
    d = q.shape[-1]
    s = (1.0 / math.sqrt(d)) if inv_temp is None else inv_temp
    outs, rems = [], []
    for r0 in range(0, L, row_chunk):
        r1 = min(L, r0 + row_chunk)
        kk, vv = k[..., :r1, :], v[..., :r1, :]
        z = torch.matmul(q[..., r0:r1, :], kk.transpose(-2, -1)) * s
        rows = torch.arange(r0, r1, device=q.device)[:, None]
        cols = torch.arange(0, r1, device=q.device)[None, :]
        visible = (cols <= rows) if attend_current else (cols < rows)
        log_miss = torch.where(visible, F.logsigmoid(-z), torch.zeros_like(z))
        incl = torch.flip(torch.cumsum(torch.flip(log_miss, dims=(-1,)), dim=-1), dims=(-1,))
        a = torch.where(visible, torch.exp(F.logsigmoid(z) + incl - log_miss), torch.zeros_like(z))
        outs.append(torch.matmul(a, vv))
        rems.append(1.0 - a.sum(dim=-1))
    return torch.cat(outs, dim=-2), torch.cat(rems, dim=-1)


# ---------------------------------------------------------------------------------------------
# 3. Product-form double loop in float64 (independent of log space) for tiny inputs.
# ---------------------------------------------------------------------------------------------
def bruteforce(q, k, v, attend_current: bool = False, inv_temp: Optional[float] = None):
    """q,k,v [L, d] (any dtype) -> (o [L,d], rem [L], A [L,L]) in float64 by direct products."""
    q64, k64, v64 = (t.detach().double() for t in (q, k, v))
    L, d = q64.shape
    s = (1.0 / math.sqrt(d)) if inv_temp is None else inv_temp
    A = torch.zeros(L, L, dtype=torch.float64)
    rem = torch.ones(L, dtype=torch.float64)
    for i in range(L):
        stick = 1.0  # what is left of the unit stick walking from the newest visible key back
        last = i if attend_current else i - 1
        for j in range(last, -1, -1):
            beta = 1.0 / (1.0 + math.exp(-s * float(torch.dot(q64[i], k64[j]))))
            A[i, j] = beta * stick
            stick *= (1.0 - beta)
        rem[i] = stick
    return A @ v64, rem, A


# ---------------------------------------------------------------------------------------------
# 4. Packed variable-length and fixed-length drivers (tests/test_varlen.py:10-27,
#    tests/test_attn.py:10-18) -- without the caller-side "+ rem * v" epilogue.
# ---------------------------------------------------------------------------------------------
def lengths_from_cu_seqlens(cu_seqlens: Sequence[int]) -> list:
    """Inclusive-cumsum document ends (optionally with a leading 0) -> list of lengths."""
    cu = [int(c) for c in cu_seqlens]
    if len(cu) and cu[0] == 0:
        cu = cu[1:]
    out, prev = [], 0
    for c in cu:
        out.append(c - prev)
        prev = c
    return out


def sb_varlen(q, k, v, lengths: Sequence[int], attend_current: bool = False,
              inv_temp: Optional[float] = None, dense: bool = False, row_chunk: int = 0):
    """q,k,v [H, T, d] packed documents -> (o [H,T,d], rem [H,T]).

    Tokens past sum(lengths) get o = 0, rem = 0.  ``dense=True`` goes through the
    reference-shaped ``stickbreaking`` (O(L^3), small documents only, default scale only).
    """
    H, T, d = q.shape
    o = torch.zeros_like(q)
    rem = torch.zeros(H, T, dtype=q.dtype, device=q.device)
    start = 0
    outs, rems = [], []
    for n in lengths:
        n = int(n)
        if n > 0:
            sl = slice(start, start + n)
            if dense:
                assert inv_temp is None or abs(inv_temp - 1 / math.sqrt(d)) < 1e-12
                mask, cw = causal_mask_and_weights(n, attend_current, dtype=q.dtype)
                oo, rr = stickbreaking(q[None, :, sl], k[None, :, sl], v[None, :, sl], mask, cw)
                oo, rr = oo[0], rr[0]
            else:
                oo, rr = sb_document(q[:, sl], k[:, sl], v[:, sl], attend_current, inv_temp, row_chunk)
            outs.append(oo)
            rems.append(rr)
        start += n
    if start < T:
        outs.append(torch.zeros(H, T - start, d, dtype=q.dtype, device=q.device))
        rems.append(torch.zeros(H, T - start, dtype=q.dtype, device=q.device))
    return torch.cat(outs, dim=1), torch.cat(rems, dim=1)


def sb_fixed(q, k, v, attend_current: bool = False, inv_temp: Optional[float] = None,
             row_chunk: int = 0):
    """q,k,v [B, H, T, d]: every (batch, head) is one causal document of T tokens."""
    return sb_document(q, k, v, attend_current, inv_temp, row_chunk)


def sb_varlen_grads(q, k, v, lengths, grad_o, grad_rem=None, attend_current=False,
                    inv_temp=None, row_chunk: int = 0):
    """Forward + autograd backward the way tests/test_varlen.py:29-41 takes gradients.

    Returns (o, rem, dq, dk, dv).  ``grad_rem`` defaults to zeros (rem unused downstream).
    """
    qq, kk, vv = (t.detach().clone().requires_grad_(True) for t in (q, k, v))
    o, rem = sb_varlen(qq, kk, vv, lengths, attend_current, inv_temp, row_chunk=row_chunk)
    loss = (o * grad_o).sum()
    if grad_rem is not None:
        loss = loss + (rem * grad_rem).sum()
    dq, dk, dv = torch.autograd.grad(loss, (qq, kk, vv))
    return o.detach(), rem.detach(), dq, dk, dv


def sb_fixed_grads(q, k, v, grad_o, grad_rem=None, attend_current=False, inv_temp=None,
                   row_chunk: int = 0):
    qq, kk, vv = (t.detach().clone().requires_grad_(True) for t in (q, k, v))
    o, rem = sb_fixed(qq, kk, vv, attend_current, inv_temp, row_chunk)
    loss = (o * grad_o).sum()
    if grad_rem is not None:
        loss = loss + (rem * grad_rem).sum()
    dq, dk, dv = torch.autograd.grad(loss, (qq, kk, vv))
    return o.detach(), rem.detach(), dq, dk, dv


# ---------------------------------------------------------------------------------------------
# 5. Hand-derived backward (the formulas the device kernels implement), one document.
#    Mirrors the quantities of sb_varlen_bwd.py:439-453 and :476.
# ---------------------------------------------------------------------------------------------
def analytic_backward(q, k, v, grad_o, grad_rem, attend_current=False, inv_temp=None):
    """q,k,v,grad_o [L,d], grad_rem [L] -> (dq, dk, dv), float64.

        dA = do . v^T - drem                         G  = A * dA
        C[i,j] = sum_{c<=j} G[i,c]                   dz = G - beta * C
        dq = s * dz k      dk = s * dz^T q           dv = A^T do
    """
    q, k, v, grad_o, grad_rem = (t.detach().double() for t in (q, k, v, grad_o, grad_rem))
    L, d = q.shape
    s = (1.0 / math.sqrt(d)) if inv_temp is None else inv_temp
    A = attention_weights(q, k, attend_current, s)
    beta = torch.sigmoid(q @ k.T * s)
    dA = grad_o @ v.T - grad_rem[:, None]
    G = A * dA
    C = torch.cumsum(G, dim=-1)
    visible = torch.ones(L, L, dtype=torch.bool).tril(0 if attend_current else -1)
    dz = torch.where(visible, G - beta * C, torch.zeros_like(G))
    return s * dz @ k, s * dz.T @ q, A.T @ grad_o


# ---------------------------------------------------------------------------------------------
# 6. Workload generators shared by tests and the benchmark (seeded, CPU generator).
# ---------------------------------------------------------------------------------------------
def make_inputs(shape: Tuple[int, ...], seed: int, scale: float = 1.0, dist: str = "normal",
                dtype=torch.bfloat16):
    """Draw q, k, v, grad_o in that order from a CPU generator.

    dist="normal": i.i.d. N(0,1) * scale.  dist="upstream": the upstream tests' shifted draw
    (tests/test_varlen.py:83-93): v = .25 N, q = .25 (N + 1), k = .25 (N - 1), do = N, which
    keeps weight alive a few hundred keys away from the diagonal.
    """
    g = torch.Generator(device="cpu").manual_seed(seed)
    if dist == "normal":
        q, k, v, do = (torch.randn(shape, generator=g) * scale for _ in range(4))
    elif dist == "upstream":
        v = 0.25 * torch.randn(shape, generator=g)
        q = 0.25 * (torch.randn(shape, generator=g) + 1)
        k = 0.25 * (torch.randn(shape, generator=g) - 1)
        do = torch.randn(shape, generator=g)
    else:
        raise ValueError(dist)
    return tuple(t.to(dtype) for t in (q, k, v, do))
