"""Fixed-length stick-breaking attention over [batch, heads, tokens, head_dim].

Drop-in for upstream ``stickbreaking_attention/sb_attn/__init__.py`` (``sb_attn`` :57-60,
``sb_attn_`` :63-64, ``StickBreakingAttention`` :16-54).  Every (batch, head) pair is one
causal document; the same kernels as the variable-length op run over a regular tile list.
"""
import math

import torch

from .. import _ops

FWD_BLOCK_M = 128
FWD_BLOCK_N = 64
BWD_BLOCK_M = 128
BWD_BLOCK_N = 64


def _fwd(q, k, v, logit_scale, attend_current=False, no_grad=False):
    plan = _ops.make_plan(q, True, None, None, logit_scale, attend_current)
    o, rem, table = _ops.forward(plan, q, k, v, need_table=not no_grad)
    return o, rem, (plan, table)


def _bwd(do, dr, q, k, v, state, logit_scale=None, attend_current=None):
    plan, table = state
    return _ops.backward(plan, q, k, v, do, dr, table)


class StickBreakingAttention(torch.autograd.Function):

    @staticmethod
    def forward(ctx, q, k, v, inv_temp, attend_current=False):
        no_grad = not any(ctx.needs_input_grad[:3])
        o, rem, state = _fwd(q, k, v, logit_scale=inv_temp, attend_current=attend_current, no_grad=no_grad)
        plan, table = state
        if table is not None:
            ctx.save_for_backward(q, k, v, table)
        ctx.plan = plan
        ctx.logit_scale = inv_temp
        ctx.attend_current = attend_current
        return o, rem

    @staticmethod
    def backward(ctx, do, drem):
        q, k, v, table = ctx.saved_tensors
        dq, dk, dv = _bwd(do, drem, q, k, v, (ctx.plan, table))
        return dq, dk, dv, None, None


def sb_attn(q, k, v, inv_temp=None, zero_start=True, attend_current=False):
    """``zero_start`` is accepted and ignored, as upstream does."""
    if inv_temp is None:
        inv_temp = 1 / math.sqrt(q.size(-1))
    return sb_attn_(q, k, v, inv_temp, attend_current=attend_current)


def sb_attn_(q, k, v, inv_temp, attend_current):
    return StickBreakingAttention.apply(q, k, v, inv_temp, attend_current)
