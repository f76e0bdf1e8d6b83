"""Variable-length (packed documents) stick-breaking attention.

Drop-in for upstream ``stickbreaking_attention/sb_varlen/__init__.py``: same public names,
argument order, defaults and return values (``sb_attn_varlen`` :71-78, ``sb_attn_varlen_``
:81-82, ``StickBreakingAttention`` :24-68).  The device work is done by libsba.so.
"""
import math
import weakref

import torch

from .. import _ops

# Tile sizes of the HIP kernels (upstream exposes its Triton block sizes under these names).
FWD_BLOCK_M = 128
FWD_BLOCK_N = 32
BWD_BLOCK_M = 128
BWD_BLOCK_N = 64


def varlen_fwd(q, k, v, cu_seqlens, max_seqlens, logit_scale, attend_current=False, no_grad=False,
               return_attention=False, fused=False):
    """Host launcher of the forward; returns (o, rem, state) where ``state`` is what the
    backward needs (carry table, schedule, ...) -- upstream returns its fp32 ``neg_log_acc`` there --
    and, with ``return_attention``, the dense fp32 weights ``W [heads, tokens, tokens]`` as a
    fourth value (upstream sb_varlen_fwd.py:413-451)."""
    return _ops.run_forward(q, k, v, False, cu_seqlens, max_seqlens, logit_scale, attend_current,
                            need_table=not no_grad, fused=fused, return_attention=return_attention)


def varlen_bwd(do, dr, q, k, v, state, logit_scale, attend_current=False, fused=False):
    return _ops.run_backward(q, k, v, do, dr, False, state, logit_scale, attend_current, fused=fused)


# The last cu_seqlens tensor whose first entry was read back and found to be zero.
_zero_start_checked = None


def _version_of(t):
    """The in-place modification counter of a tensor, or None where PyTorch keeps none (tensors
    created under ``torch.inference_mode()`` raise on ``_version``)."""
    try:
        return t._version
    except RuntimeError:
        return None


def _starts_at_zero(cu_seqlens) -> bool:
    """``cu_seqlens[0] == 0``, upstream's check (sb_varlen/__init__.py:73).  Reading one element of a
    device tensor stalls the host until the GPU has drained, and a model passes the same
    cu_seqlens to every layer, so the answer is remembered for as long as the same tensor object
    comes back unmodified: one synchronisation per batch instead of one per call.  Tensors without
    a modification counter (inference tensors) are checked on every call.  A write through
    ``cu_seqlens.data`` does not advance the counter and is therefore not seen: do not rewrite a
    cu_seqlens tensor that way between calls."""
    global _zero_start_checked
    if torch.compiler.is_compiling():
        return bool(cu_seqlens[0] == 0)
    version = _version_of(cu_seqlens)
    if version is None:
        return bool(cu_seqlens[0] == 0)
    seen = _zero_start_checked
    if seen is not None and seen[0]() is cu_seqlens and seen[1] == version:
        return True
    ok = bool(cu_seqlens[0] == 0)
    if ok:
        _zero_start_checked = (weakref.ref(cu_seqlens), version)
    return ok


class StickBreakingAttention(torch.autograd.Function):

    @staticmethod
    def forward(ctx, q, k, v, cu_seqlens, max_seqlens, inv_temp, attend_current):
        no_grad = not any(ctx.needs_input_grad[:3])
        o, rem, state = varlen_fwd(q, k, v, cu_seqlens, max_seqlens, logit_scale=inv_temp,
                                   attend_current=attend_current, no_grad=no_grad)
        table, sched, cu, max_len, product = state
        ctx.save_for_backward(q, k, v, table, sched, cu)
        ctx.logit_scale = inv_temp
        ctx.max_seqlens = max_len
        ctx.attend_current = attend_current
        ctx.product = product
        return o, rem

    @staticmethod
    def backward(ctx, do, drem):
        q, k, v, table, sched, cu = ctx.saved_tensors
        state = (table, sched, cu, ctx.max_seqlens, ctx.product)
        dq, dk, dv = varlen_bwd(do, drem, q, k, v, state, ctx.logit_scale, ctx.attend_current)
        return dq, dk, dv, None, None, None, None


def sb_attn_varlen(q, k, v, cu_seqlens, max_seqlens=None, inv_temp=None, zero_start=True, attend_current=False):
    """q, k, v: [heads, total_tokens, head_dim]; cu_seqlens: cumulative document ends (with a
    leading 0 when ``zero_start``).  Returns (o [heads, total_tokens, head_dim],
    rem [heads, total_tokens])."""
    if zero_start:
        assert _starts_at_zero(cu_seqlens)
        cu_seqlens = cu_seqlens[1:]
    if inv_temp is None:
        inv_temp = 1 / math.sqrt(q.size(-1))
    return sb_attn_varlen_(q, k, v, inv_temp, cu_seqlens, max_seqlens, attend_current)


def sb_attn_varlen_(q, k, v, inv_temp, cu_seqlens, max_seqlens, attend_current):
    return StickBreakingAttention.apply(q, k, v, cu_seqlens, max_seqlens, inv_temp, attend_current)


class StickBreakingAttentionFused(torch.autograd.Function):
    """``o + rem[..., None] * v`` in one piece: the sum is formed where ``o`` leaves the forward
    kernel, and its gradient's two extra terms inside the backward kernels."""

    @staticmethod
    def forward(ctx, q, k, v, cu_seqlens, max_seqlens, inv_temp, attend_current):
        no_grad = not any(ctx.needs_input_grad[:3])
        out, _rem, state = varlen_fwd(q, k, v, cu_seqlens, max_seqlens, logit_scale=inv_temp,
                                      attend_current=attend_current, no_grad=no_grad, fused=True)
        table, sched, cu, max_len, product = state
        ctx.save_for_backward(q, k, v, table, sched, cu)
        ctx.logit_scale = inv_temp
        ctx.max_seqlens = max_len
        ctx.attend_current = attend_current
        ctx.product = product
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, table, sched, cu = ctx.saved_tensors
        state = (table, sched, cu, ctx.max_seqlens, ctx.product)
        dq, dk, dv = varlen_bwd(dout, None, q, k, v, state, ctx.logit_scale, ctx.attend_current, fused=True)
        return dq, dk, dv, None, None, None, None


def sb_attn_varlen_fused(q, k, v, cu_seqlens, max_seqlens=None, inv_temp=None, zero_start=True, attend_current=False):
    """Same arguments as ``sb_attn_varlen``; returns the single tensor every upstream caller forms
    from its two outputs, ``o + rem[..., None] * v`` (upstream tests/test_varlen.py:101), without
    the extra passes over ``o`` and ``v`` in forward and backward."""
    if zero_start:
        assert _starts_at_zero(cu_seqlens)
        cu_seqlens = cu_seqlens[1:]
    if inv_temp is None:
        inv_temp = 1 / math.sqrt(q.size(-1))
    return StickBreakingAttentionFused.apply(q, k, v, cu_seqlens, max_seqlens, inv_temp, attend_current)
