"""Test infrastructure (never imported by the product path): a CPU model of WHERE the HIP
kernels round, used to tell rounding of the bf16 MFMA operands apart from arithmetic mistakes.

The kernels take bf16 q, k, v, grad_o, form the scores, the stick weights A and the gradient
of the logits dz in fp32, and round exactly three kinds of values to bf16:
  * A, as the operand of o = A v (forward) and dv = A^T grad_o (dk/dv pass);
  * dz, as the operand of dq = s dz k (dq pass) and dk = s dz^T q (dk/dv pass);
  * the outputs o, rem, dq, dk, dv themselves.
Everything else (scores, products of 1 - sigmoid, the running sum of G, accumulation) is fp32,
which this model replaces by float64: what is left is exactly the error the operand and output
roundings cause, for one document of one head.  Mathematics as in upstream
stickbreaking_attention/sb_ref.py:8-25 (forward) and sb_varlen/sb_varlen_bwd.py:439-453 (backward).
"""
import math

import torch


def _bf16(x: torch.Tensor) -> torch.Tensor:
    return x.to(torch.float32).to(torch.bfloat16).to(torch.float64)


def document(q, k, v, do, drem=None, attend_current=False, inv_temp=None, round_operands=True, round_outputs=True):
    """q, k, v, do: [L, d] (bf16-representable values); drem: [L] or None.
    Returns (o, rem, dq, dk, dv) in float64 with the kernels' rounding points applied (or not)."""
    q, k, v, do = (t.to(torch.float64) for t in (q, k, v, do))
    L, d = q.shape
    s = 1.0 / math.sqrt(d) if inv_temp is None else float(inv_temp)
    dr = torch.zeros(L, dtype=torch.float64) if drem is None else drem.to(torch.float64)
    z = s * (q @ k.T)
    idx = torch.arange(L)
    allowed = (idx[None, :] <= idx[:, None]) if attend_current else (idx[None, :] < idx[:, None])
    beta = torch.sigmoid(z)
    log_r = torch.where(allowed, torch.nn.functional.logsigmoid(-z), torch.zeros_like(z))
    # sum of log(1 - beta) over allowed keys newer than j: reverse exclusive cumulative sum
    suffix = torch.flip(torch.cumsum(torch.flip(log_r, [1]), 1), [1]) - log_r
    A = torch.where(allowed, beta * torch.exp(suffix), torch.zeros_like(z))
    rem = 1.0 - A.sum(1)
    A_op = _bf16(A) if round_operands else A
    o = A_op @ v
    da = do @ v.T
    G = A * (da - dr[:, None])
    C = torch.cumsum(G, 1)
    dz = torch.where(allowed, G - beta * C, torch.zeros_like(z))
    dz_op = _bf16(dz) if round_operands else dz
    dq = s * (dz_op @ k)
    dk = s * (dz_op.T @ q)
    dv = A_op.T @ do
    outs = (o, rem, dq, dk, dv)
    return tuple(_bf16(t) for t in outs) if round_outputs else outs


def varlen(q, k, v, do, lengths, drem=None, attend_current=False, inv_temp=None, **kw):
    """[H, T, d] packed documents -> five float64 tensors shaped like the operator's outputs."""
    H, T, d = q.shape
    o = torch.zeros(H, T, d, dtype=torch.float64)
    dq, dk, dv = torch.zeros_like(o), torch.zeros_like(o), torch.zeros_like(o)
    rem = torch.zeros(H, T, dtype=torch.float64)
    start = 0
    for n in lengths:
        if n > 0:
            sl = slice(start, start + n)
            for hd in range(H):
                r = document(q[hd, sl], k[hd, sl], v[hd, sl], do[hd, sl], None if drem is None else drem[hd, sl],
                             attend_current, inv_temp, **kw)
                o[hd, sl], rem[hd, sl], dq[hd, sl], dk[hd, sl], dv[hd, sl] = r
        start += n
    return o, rem, dq, dk, dv
