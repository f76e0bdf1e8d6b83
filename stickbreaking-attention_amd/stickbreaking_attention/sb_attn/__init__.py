"""Fixed-length stick-breaking attention over [batch, heads, tokens, head_dim].

Drop-in for upstream ``stickbreaking_attention/sb_attn/__init__.py`` (``sb_attn`` :57-60,
``sb_attn_`` :63-64, ``StickBreakingAttention`` :16-54).  Every (batch, head) pair is one
causal document; the same kernels as the variable-length op run over a regular tile list.
"""
import math

import torch

from .. import _ops

# Tile sizes of the HIP kernels (upstream exposes its Triton block sizes under these names).
FWD_BLOCK_M = 128
FWD_BLOCK_N = 32
BWD_BLOCK_M = 128
BWD_BLOCK_N = 64


def _fwd(q, k, v, logit_scale, attend_current=False, no_grad=False, return_attention=False, fused=False):
    """(o, rem, state[, W [batch, heads, tokens, tokens]]) -- upstream sb_attn/sb_fwd.py:139-174."""
    return _ops.run_forward(q, k, v, True, None, None, logit_scale, attend_current, need_table=not no_grad,
                            fused=fused, return_attention=return_attention)


def _bwd(do, dr, q, k, v, state, logit_scale, attend_current=False, fused=False):
    return _ops.run_backward(q, k, v, do, dr, True, state, logit_scale, attend_current, fused=fused)


class StickBreakingAttention(torch.autograd.Function):

    @staticmethod
    def forward(ctx, q, k, v, inv_temp, attend_current=False):
        # an output nobody differentiates through arrives as None in backward instead of as a tensor of
        # zeros that PyTorch would have to allocate and fill
        ctx.set_materialize_grads(False)
        no_grad = not any(ctx.needs_input_grad[:3])
        o, rem, state = _fwd(q, k, v, logit_scale=inv_temp, attend_current=attend_current, no_grad=no_grad)
        table, sched, _cu, max_len, product = state
        ctx.save_for_backward(q, k, v, table, sched)
        ctx.logit_scale = inv_temp
        ctx.max_seqlens = max_len
        ctx.attend_current = attend_current
        ctx.product = product
        return o, rem

    @staticmethod
    def backward(ctx, do, drem):
        q, k, v, table, sched = ctx.saved_tensors
        state = (table, sched, None, ctx.max_seqlens, ctx.product)
        if do is None:          # only rem was used
            do = torch.zeros_like(q)
        dq, dk, dv = _bwd(do, drem, q, k, v, state, ctx.logit_scale, ctx.attend_current)
        return dq, dk, dv, None, None


def sb_attn(q, k, v, inv_temp=None, zero_start=True, attend_current=False):
    """``zero_start`` is accepted and ignored, as upstream does."""
    if inv_temp is None:
        inv_temp = 1 / math.sqrt(q.size(-1))
    return sb_attn_(q, k, v, inv_temp, attend_current=attend_current)


def sb_attn_(q, k, v, inv_temp, attend_current):
    return StickBreakingAttention.apply(q, k, v, inv_temp, attend_current)


class StickBreakingAttentionFused(torch.autograd.Function):
    """``o + rem[..., None] * v`` in one piece (see ``sb_varlen.StickBreakingAttentionFused``)."""

    @staticmethod
    def forward(ctx, q, k, v, inv_temp, attend_current=False):
        no_grad = not any(ctx.needs_input_grad[:3])
        out, _rem, state = _fwd(q, k, v, logit_scale=inv_temp, attend_current=attend_current, no_grad=no_grad,
                                fused=True)
        table, sched, _cu, max_len, product = state
        ctx.save_for_backward(q, k, v, table, sched)
        ctx.logit_scale = inv_temp
        ctx.max_seqlens = max_len
        ctx.attend_current = attend_current
        ctx.product = product
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, table, sched = ctx.saved_tensors
        state = (table, sched, None, ctx.max_seqlens, ctx.product)
        dq, dk, dv = _bwd(dout, None, q, k, v, state, ctx.logit_scale, ctx.attend_current, fused=True)
        return dq, dk, dv, None, None


def sb_attn_fused(q, k, v, inv_temp=None, zero_start=True, attend_current=False):
    """Same arguments as ``sb_attn``; returns ``o + rem[..., None] * v`` (upstream
    tests/test_attn.py:64) as one tensor."""
    if inv_temp is None:
        inv_temp = 1 / math.sqrt(q.size(-1))
    return StickBreakingAttentionFused.apply(q, k, v, inv_temp, attend_current)
