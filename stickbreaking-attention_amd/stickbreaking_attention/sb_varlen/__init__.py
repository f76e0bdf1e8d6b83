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


def _starts_at_zero(cu_seqlens) -> bool:
    """``cu_seqlens[0] == 0``, upstream's check (sb_varlen/__init__.py:73).  Reading one element of a
    device tensor stalls the host until the GPU has drained, and a model passes the same
    cu_seqlens to every layer, so the whole tensor is copied to the host once per tensor object and
    version (``_ops.host_cu_seqlens``, which the launcher uses as well): one synchronisation per
    batch instead of one per call.  Tensors without a modification counter (inference tensors) are
    read on every call."""
    if torch.compiler.is_compiling():
        return bool(cu_seqlens[0] == 0)
    vals = _ops.host_cu_seqlens(cu_seqlens)
    if vals is None:
        # While the stream is being captured into a graph no value can be read back (a
        # synchronisation would end the capture): the caller's zero_start=True is taken at its word.
        if cu_seqlens.is_cuda and torch.cuda.is_current_stream_capturing():
            return True
        return bool(cu_seqlens[0] == 0)   # SBA_SYNC_FREE: upstream's assertion still needs this one value
    return len(vals) > 0 and vals[0] == 0


def _strip_leading_zero(cu_seqlens):
    """``cu_seqlens[1:]`` (upstream sb_varlen/__init__.py:74).  The same view object comes back for
    as long as the same unmodified tensor is passed in (a model hands one cu_seqlens to every
    layer), carrying the host copy of the values with it: what the launcher remembers per
    cu_seqlens tensor -- host values, schedule -- is found again by identity."""
    if torch.compiler.is_compiling():
        return cu_seqlens[1:]
    version = _ops._version_of(cu_seqlens)
    with _ops._cache_lock:
        if version is not None:
            for i in range(len(_ops._stripped_views) - 1, -1, -1):
                ref, ver, view = _ops._stripped_views[i]
                if ref() is cu_seqlens:
                    if ver == version:
                        return view
                    del _ops._stripped_views[i]
                    break
        stripped = cu_seqlens[1:]
        vals = _ops.host_cu_seqlens(cu_seqlens, allow_sync=False)
        if vals is not None:
            _ops.remember_host_cu(stripped, vals[1:])
        if version is not None:
            _ops._stripped_views[:] = [e for e in _ops._stripped_views if e[0]() is not None][-3:]
            _ops._stripped_views.append((weakref.ref(cu_seqlens), version, stripped))
        return stripped


class StickBreakingAttention(torch.autograd.Function):

    @staticmethod
    def forward(ctx, q, k, v, cu_seqlens, max_seqlens, inv_temp, attend_current):
        # an output nobody differentiates through arrives as None in backward instead of as a tensor of
        # zeros that PyTorch would have to allocate and fill
        ctx.set_materialize_grads(False)
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
        if do is None:          # only rem was used
            do = torch.zeros_like(q)
        dq, dk, dv = varlen_bwd(do, drem, q, k, v, state, ctx.logit_scale, ctx.attend_current)
        return dq, dk, dv, None, None, None, None


def sb_attn_varlen(q, k, v, cu_seqlens, max_seqlens=None, inv_temp=None, zero_start=True, attend_current=False):
    """q, k, v: [heads, total_tokens, head_dim]; cu_seqlens: cumulative document ends (with a
    leading 0 when ``zero_start``).  Returns (o [heads, total_tokens, head_dim],
    rem [heads, total_tokens])."""
    if zero_start:
        assert _starts_at_zero(cu_seqlens)
        cu_seqlens = _strip_leading_zero(cu_seqlens)
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
        cu_seqlens = _strip_leading_zero(cu_seqlens)
    if inv_temp is None:
        inv_temp = 1 / math.sqrt(q.size(-1))
    return StickBreakingAttentionFused.apply(q, k, v, cu_seqlens, max_seqlens, inv_temp, attend_current)
