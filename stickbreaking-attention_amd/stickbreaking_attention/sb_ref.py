"""Dense definition of stick-breaking attention, for checking results on small inputs.

Same name, arguments and return values as upstream ``stickbreaking_attention/sb_ref.py:8-25``
so that test code written against it keeps working.  It materialises the full [L, L] weight
matrix with ordinary PyTorch operations on whatever device its inputs live on; the operators
``sb_attn`` / ``sb_attn_varlen`` never call it.
"""
import torch
from torch.nn import functional as F


def stickbreaking(q, k, v, mask, cum_weight):
    """q, k, v: [batch, heads, L, d].  ``mask`` [L, L] is True where key j is NOT visible to query
    i; ``cum_weight`` [L, L] has cum_weight[j', j] = 1 where key j' lies between key j and the
    query (strictly newer than j), so that ``log(1 - beta) @ cum_weight`` is the log of the stick
    left when key j is reached.  Returns (att @ v, 1 - att.sum(-1))."""
    z = torch.matmul(q, k.transpose(-1, -2)) * (q.shape[-1] ** -0.5)
    dtype = z.dtype
    if z.dtype in (torch.float16, torch.bfloat16):
        z = z.float()      # half-precision logits are evaluated in fp32 and rounded back
    log_take = (-F.softplus(-z)).masked_fill(mask, -1e5).to(dtype)    # log sigmoid(z): share taken by key j
    log_leave = (-F.softplus(z)).masked_fill(mask, 0).to(dtype)       # log(1 - sigmoid(z)): share passed on
    log_stick = torch.matmul(log_leave, cum_weight.to(log_leave))     # summed over the keys newer than j
    att = torch.exp(log_take + log_stick)
    return torch.matmul(att, v), 1 - att.sum(dim=-1)
