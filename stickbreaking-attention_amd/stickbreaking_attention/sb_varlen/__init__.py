"""Variable-length (packed documents) stick-breaking attention.

Drop-in for upstream ``stickbreaking_attention/sb_varlen/__init__.py``: same public names,
argument order, defaults and return values (``sb_attn_varlen`` :71-78, ``sb_attn_varlen_``
:81-82, ``StickBreakingAttention`` :24-68).  The device work is done by libsba.so.
"""
import math

import torch

from .. import _ops

FWD_BLOCK_M = 128
FWD_BLOCK_N = 64
BWD_BLOCK_M = 128
BWD_BLOCK_N = 64


def varlen_fwd(q, k, v, cu_seqlens, max_seqlens, logit_scale, attend_current=False, no_grad=False):
    """Host launcher of the forward; returns (o, rem, state) where ``state`` is what the
    backward needs (plan + carry table) -- upstream returns its fp32 ``neg_log_acc`` there."""
    plan = _ops.make_plan(q, False, cu_seqlens, max_seqlens, logit_scale, attend_current)
    o, rem, table = _ops.forward(plan, q, k, v, need_table=not no_grad)
    return o, rem, (plan, table)


def varlen_bwd(do, dr, q, k, v, state, logit_scale=None, attend_current=None):
    plan, table = state
    return _ops.backward(plan, q, k, v, do, dr, table)


class StickBreakingAttention(torch.autograd.Function):

    @staticmethod
    def forward(ctx, q, k, v, cu_seqlens, max_seqlens, inv_temp, attend_current):
        no_grad = not any(ctx.needs_input_grad[:3])
        o, rem, state = varlen_fwd(q, k, v, cu_seqlens, max_seqlens, logit_scale=inv_temp,
                                   attend_current=attend_current, no_grad=no_grad)
        plan, table = state
        if table is not None:
            ctx.save_for_backward(q, k, v, table, cu_seqlens)
        ctx.plan = plan
        ctx.logit_scale = inv_temp
        ctx.max_seqlens = max_seqlens
        ctx.attend_current = attend_current
        return o, rem

    @staticmethod
    def backward(ctx, do, drem):
        q, k, v, table, _cu = ctx.saved_tensors
        dq, dk, dv = varlen_bwd(do, drem, q, k, v, (ctx.plan, table))
        return dq, dk, dv, None, None, None, None


def sb_attn_varlen(q, k, v, cu_seqlens, max_seqlens=None, inv_temp=None, zero_start=True, attend_current=False):
    """q, k, v: [heads, total_tokens, head_dim]; cu_seqlens: cumulative document ends (with a
    leading 0 when ``zero_start``).  Returns (o [heads, total_tokens, head_dim],
    rem [heads, total_tokens])."""
    if zero_start:
        assert cu_seqlens[0] == 0
        cu_seqlens = cu_seqlens[1:]
    if inv_temp is None:
        inv_temp = 1 / math.sqrt(q.size(-1))
    return sb_attn_varlen_(q, k, v, inv_temp, cu_seqlens, max_seqlens, attend_current)


def sb_attn_varlen_(q, k, v, inv_temp, cu_seqlens, max_seqlens, attend_current):
    return StickBreakingAttention.apply(q, k, v, cu_seqlens, max_seqlens, inv_temp, attend_current)
