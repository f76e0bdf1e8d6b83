"""Host glue between the autograd functions and libsba.so.

Mirrors what the upstream host launchers do around their Triton kernels -- allocate outputs
and private state with PyTorch, pass raw pointers and strides, launch on the current stream
(upstream ``varlen_fwd`` sb_varlen/sb_varlen_fwd.py:413-451, ``varlen_bwd``
sb_varlen/sb_varlen_bwd.py:484-539, ``_fwd`` sb_attn/sb_fwd.py:139-174, ``_bwd``
sb_attn/sb_bwd.py:163-205) -- with the device code behind a C ABI instead of a JIT.

Like upstream, every launcher exists twice: as a plain Python function used in eager mode,
and registered through ``torch.library.custom_op`` under upstream's operator names
(``stickbreaking_attention::varlen_fwd``, ``::varlen_bwd``, ``::attn_fwd``, ``::attn_bwd``;
sb_varlen_fwd.py:454, sb_varlen_bwd.py:542, sb_fwd.py:177, sb_bwd.py:208), which is what runs
while ``torch.compile`` traces.  The registered operators return nothing and write into
buffers the caller allocated, so they need no shape function.
"""
import ctypes
import functools
import math
import os
import warnings
import threading
import weakref
from typing import Optional, Sequence, Tuple

import torch

from . import _native as nat
from .utils import custom_op

# Carry the stick as a running product (2 transcendentals per score) instead of a running
# log2 sum (3 per score).  Overridable for A/B measurements.
PRODUCT_SPACE = os.environ.get("SBA_LOG_SPACE", "0") != "1"

# When True every eager forward reads back the scheduler's status words (one device sync) and
# raises on malformed cu_seqlens or undersized tables instead of returning NaN outputs.
VALIDATE = os.environ.get("SBA_VALIDATE", "0") == "1"

# Eager calls copy each NEW cu_seqlens tensor to the host once (one synchronisation per tensor
# object and version; a model hands the same tensor to every layer) so that the carry tables are
# sized exactly and malformed cu_seqlens raise at once.  With SBA_SYNC_FREE=1 -- and always while
# torch.compile traces -- nothing is read back: tables get the worst-case size for
# (tokens, max_seqlens) and errors surface as NaN outputs.
SYNC_FREE = os.environ.get("SBA_SYNC_FREE", "0") == "1"

# With SBA_RECOMPUTE_TABLE=1 a forward keeps NO carry table for its backward: the backward first runs
# the table-only variant of the forward kernel (scores and stick, no P.V, no outputs) to rebuild it.
# What a layer holds between forward and backward is then q, k, v alone -- upstream's
# O(heads x tokens) footprint -- for about 60 % of a forward pass of extra time per backward; the
# rebuilt table is one scratch buffer shared by all layers.
RECOMPUTE_TABLE = os.environ.get("SBA_RECOMPUTE_TABLE", "0") == "1"

# With SBA_F32_AS_F16=1 float32 inputs run on the float16 kernels instead of being rounded to bfloat16: operands of 11
# significant bits, what upstream's tl.dot gives float32 inputs with TF32 allowed (utils.py:8, sb_varlen_fwd.py:42),
# against bfloat16's 8.  float16 has a narrow exponent: q, k, v must stay within +-65504 (beyond that the outputs are
# NaN), which is why this is a switch and not the default; the incoming gradient, whose scale is arbitrary, is brought
# to a maximum between 4 and 8 by a power of two before it is rounded and the gradients are scaled back (exact).
F32_AS_F16 = os.environ.get("SBA_F32_AS_F16", "0") == "1"

SUPPORTED_HEAD_DIMS = (32, 64, 128, 256)

# Tile sizes the library's workspace formulas are built on (query tile, dk/dv key tile, table block).
_BM, _BKV, _BT, _SCHED_HDR, _TILE_WORDS = 128, 128, 32, 16, 8
_WORK_WORDS = 64      # words at the end of every carry table: the work counters of the library's persistent launches


def _padded_dim(d: int) -> int:
    for s in SUPPORTED_HEAD_DIMS:
        if d <= s:
            return s
    raise ValueError(f"head_dim {d} is not supported (maximum {SUPPORTED_HEAD_DIMS[-1]})")


def table_entries(length: int) -> int:
    """Carry-table entries one document of `length` tokens needs per head: with the length rounded up
    to a multiple of 32, one per (32-key block, query row at or below it) pair plus one per row
    (``tab_doc_entries`` in csrc/sba_device.hpp)."""
    nb = -(-length // _BT)
    return 16 * nb * (nb + 1) + 32 * nb


def table_entries_bound(tokens: int, max_doc_len: int, n_docs: int) -> int:
    """The most any split of `tokens` tokens into `n_docs` documents of at most `max_doc_len` can need."""
    lmax = max_doc_len if 0 < max_doc_len < tokens else tokens
    lmax = (lmax + 31) & ~31
    if lmax <= 0:
        return 0
    padded = tokens + 31 * n_docs
    return (padded // lmax) * table_entries(lmax) + table_entries(padded % lmax)


def workspace_sizes(fixed: bool, batch: int, heads: int, tokens: int, n_docs: int, max_doc_len: int,
                    lengths: Optional[Sequence[int]] = None) -> Tuple[int, int]:
    """(schedule bytes, floats of one carry table): the same numbers as ``sba_schedule_bytes`` and
    ``sba_table_bytes // 4`` (``sba_table_bytes_for_lengths // 4`` when the document lengths are
    given -- or, as an int, the table entries per head they were already found to need), computed
    without touching the library so that they can be evaluated while a graph is being traced
    (checked against the library in the tests)."""
    docs = batch if fixed else n_docs
    rows = (batch if fixed else 1) * tokens
    n_q = rows // _BM + docs + 1
    n_kv = rows // _BKV + docs + 1
    words = _SCHED_HDR + _TILE_WORDS * (n_q + n_kv) + 6 * docs + 2
    if fixed:
        entries = batch * table_entries(tokens)
    elif lengths is not None:
        entries = lengths if isinstance(lengths, int) else max(32, sum(table_entries(int(n)) for n in lengths))
    else:
        entries = table_entries_bound(tokens, max_doc_len, n_docs)
    return (4 * words + 255) & ~255, heads * entries + _WORK_WORDS


# One lock for the module-level caches below (host copies of cu_seqlens, views without the leading
# zero, schedules, scratch tables): PyTorch runs the backward on its own autograd thread, so the
# forward thread and the backward thread reach them concurrently.
_cache_lock = threading.RLock()

# cu_seqlens tensors already copied to the host: (weak reference, version, tuple of values), newest last
_host_cu_cache = []
_HOST_CU_CACHE_SIZE = 8


# views without the leading zero that sb_attn_varlen already handed out:
# (weak reference to cu_seqlens, version, view), newest last
_stripped_views = []


def _version_of(t):
    """The in-place modification counter of a tensor, or None where PyTorch keeps none (tensors
    created under ``torch.inference_mode()`` raise on ``_version``)."""
    try:
        return t._version
    except RuntimeError:
        return None


def host_cu_seqlens(cu_seqlens: torch.Tensor, allow_sync: bool = True) -> Optional[Tuple[int, ...]]:
    """The values of a cu_seqlens tensor on the host, remembered per tensor object for as long as it
    comes back unmodified; None when they are not known and may not be fetched (``allow_sync``
    False, SBA_SYNC_FREE, torch.compile).  A write through ``cu_seqlens.data`` does not advance the
    tensor's version counter and is therefore not seen: do not rewrite a cu_seqlens tensor that
    way between calls."""
    if torch.compiler.is_compiling():
        return None
    version = _version_of(cu_seqlens)
    with _cache_lock:
        if version is not None:
            for i in range(len(_host_cu_cache) - 1, -1, -1):
                ref, ver, vals = _host_cu_cache[i]
                if ref() is cu_seqlens:
                    if ver == version:
                        return vals
                    del _host_cu_cache[i]
                    break
    if cu_seqlens.is_cuda and (not allow_sync or SYNC_FREE):
        return None
    # A device-to-host copy synchronises, which a stream that is being captured into a graph does
    # not survive: values not already known stay unknown there (worst-case table size, checks on
    # the device), exactly as with SBA_SYNC_FREE.
    if cu_seqlens.is_cuda and torch.cuda.is_current_stream_capturing():
        return None
    vals = tuple(int(x) for x in cu_seqlens.tolist())   # the one synchronisation per tensor
    if version is not None:
        with _cache_lock:
            _host_cu_cache[:] = [e for e in _host_cu_cache if e[0]() is not None][-(_HOST_CU_CACHE_SIZE - 1):]
            _host_cu_cache.append((weakref.ref(cu_seqlens), version, vals))
    return vals


def remember_host_cu(cu_seqlens: torch.Tensor, vals: Sequence[int]) -> None:
    """Associate host values with a tensor whose contents are already known (the view without the
    leading zero that ``sb_attn_varlen`` passes on)."""
    version = _version_of(cu_seqlens)
    if version is None or torch.compiler.is_compiling():
        return
    with _cache_lock:
        _host_cu_cache[:] = [e for e in _host_cu_cache if e[0]() is not None][-(_HOST_CU_CACHE_SIZE - 1):]
        _host_cu_cache.append((weakref.ref(cu_seqlens), version, vals if isinstance(vals, tuple) else tuple(int(x) for x in vals)))


def _doc_lengths(cu_vals: Sequence[int], tokens: int) -> Tuple[int, ...]:
    """Document lengths from inclusive cumulative ends (no leading zero); raises on what the device
    scheduler would flag as SBA_STATUS_BAD_CU."""
    prev, out = 0, []
    for end in cu_vals:
        if end < prev or end > tokens:
            raise ValueError("sb_attn_varlen: " + nat.STATUS_MESSAGES[1])
        out.append(end - prev)
        prev = end
    return tuple(out)


@functools.lru_cache(maxsize=16)
def _lengths_info(cu_vals: Tuple[int, ...], tokens: int) -> Tuple[Tuple[int, ...], int, int]:
    """(document lengths, longest document (at least 1), carry-table entries per head) of a cu_seqlens
    whose values are on the host; remembered, because a model calls every layer with the same one."""
    lengths = _doc_lengths(cu_vals, tokens)
    return lengths, max(1, max(lengths, default=1)), max(32, sum(table_entries(n) for n in lengths))


_warned_dtypes = set()


def _warn_reduced_precision(dtype) -> None:
    """Upstream runs its dots in the input dtype (tl.dot on fp16 / TF32 on fp32 inputs,
    sb_varlen_fwd.py:42, utils.py:8).  This library has kernels for bfloat16 and for float16 and
    multiplies anything else in bfloat16.  Said once per dtype instead of silently."""
    if dtype not in _warned_dtypes:
        _warned_dtypes.add(dtype)
        warnings.warn(f"stickbreaking_attention: {dtype} inputs are rounded to bfloat16 before the matrix products "
                      "(8 bits of mantissa; outputs are returned in the input dtype)", stacklevel=4)


def compute_dtype(dtype: torch.dtype) -> torch.dtype:
    """The element type the kernels run in for inputs of `dtype`: bfloat16 and float16 natively (MFMA
    of that type, fp32 accumulation), everything else in bfloat16 (float32 in float16 with F32_AS_F16)."""
    if dtype in (torch.bfloat16, torch.float16):
        return dtype
    return torch.float16 if (dtype == torch.float32 and F32_AS_F16) else torch.bfloat16


def _prep(t: torch.Tensor, dpad: int, cdt: torch.dtype, incoming_grad: bool = False) -> torch.Tensor:
    """Element type `cdt`, head_dim padded with zeros to `dpad`, row strides multiples of 8 elements
    (traceable).  The strides of an incoming gradient are not known while a backward is being
    traced, so there it is simply made contiguous."""
    if t.dtype != cdt:
        if not torch.compiler.is_compiling() and t.dtype not in (torch.bfloat16, torch.float16) and cdt == torch.bfloat16:
            _warn_reduced_precision(t.dtype)
        t = t.to(cdt)
    d = t.shape[-1]
    if d != dpad:
        t = torch.nn.functional.pad(t, (0, dpad - d))
    if incoming_grad and torch.compiler.is_compiling():
        return t.contiguous()
    ok = t.stride(-1) == 1 and all(s % 8 == 0 for s in t.stride()[:-1])
    return t if ok else t.contiguous()


def _aligned(t: torch.Tensor) -> torch.Tensor:
    """Inputs whose storage offset breaks 16-byte alignment are copied (launch time only)."""
    return t if t.data_ptr() % 16 == 0 else t.clone(memory_format=torch.contiguous_format)


def _dtype_code(t: torch.Tensor) -> int:
    return nat.SBA_F16 if t.dtype == torch.float16 else nat.SBA_BF16


def _problem(q: torch.Tensor, fixed: bool, cu_seqlens: Optional[torch.Tensor], max_doc_len: int,
             inv_temp: float, attend_current: bool, product: bool, fused: bool, extra_flags: int = 0):
    """The ``sba_problem`` of a launch plus the tensors whose pointers it holds."""
    flags = ((nat.FLAG_ATTEND_CURRENT if attend_current else 0) | (nat.FLAG_PRODUCT_SPACE if product else 0) |
             (nat.FLAG_FUSE_REMAINDER if fused else 0) | extra_flags)
    if fixed:
        B, H, T, d = q.shape
        return nat.SbaProblem(_dtype_code(q), d, H, B, T, 0, T, flags | nat.FLAG_FIXED_LENGTH,
                              float(inv_temp), None), ()
    H, T, d = q.shape
    if cu_seqlens.dtype == torch.int64:
        flags |= nat.FLAG_CU_INT64
    cu = cu_seqlens.contiguous()
    return nat.SbaProblem(_dtype_code(q), d, H, 1, T, cu.numel(), max_doc_len, flags, float(inv_temp),
                          cu.data_ptr() if cu.numel() else None), (cu,)


def _ptr(t: Optional[torch.Tensor]):
    return t.data_ptr() if t is not None and t.numel() else None


# ---------------------------------------------------------------------------------------------
# launchers: everything is allocated by the caller
# ---------------------------------------------------------------------------------------------
def _nbytes(t: Optional[torch.Tensor]) -> int:
    return 0 if t is None else t.numel() * t.element_size()


def _launch_fwd(fixed: bool, q, k, v, cu_seqlens, max_doc_len: int, logit_scale: float, attend_current: bool,
                product: bool, fused: bool, o, rem, table, sched, weights=None, build_schedule: bool = True) -> None:
    """(`o` and `rem` without elements: only the carry table is wanted, SBA_TABLE_ONLY.)"""
    nat.require_gpu(q)
    lib = nat.load()
    q, k, v = _aligned(q), _aligned(k), _aligned(v)
    table_only = o.numel() == 0 and q.numel() != 0
    if table_only:
        o = rem = None
    prob, _keep = _problem(q, fixed, cu_seqlens, max_doc_len, logit_scale, attend_current, product, fused,
                           nat.FLAG_TABLE_ONLY if table_only else 0)
    name = ("sba_attn_fwd" if fixed else "sba_varlen_fwd") + ("_weights" if weights is not None else "")
    fn = getattr(lib, name)
    extra = () if weights is None else (weights.data_ptr(), _nbytes(weights))
    with torch.cuda.device(q.device):
        stream = nat.stream_ptr(q.device)
        # every workspace goes in with its size: the library answers SBA_E_WORKSPACE instead of overrunning one
        if build_schedule:
            nat.check(lib.sba_build_schedule(ctypes.byref(prob), sched.data_ptr(), _nbytes(sched), stream), "sba_build_schedule")
        code = fn(ctypes.byref(prob), sched.data_ptr(), _nbytes(sched),
                  ctypes.byref(nat.view4(q, fixed)), ctypes.byref(nat.view4(k, fixed)),
                  ctypes.byref(nat.view4(v, fixed)), ctypes.byref(nat.view4(o, fixed)),
                  ctypes.byref(nat.view4(rem, fixed, per_row=True)), _ptr(table), _nbytes(table), *extra, stream)
    nat.check(code, name)


def _launch_bwd(fixed: bool, do, dr, q, k, v, cu_seqlens, max_doc_len: int, logit_scale: float,
                attend_current: bool, product: bool, fused: bool, table, sched, gtab, dq, dk, dv) -> None:
    nat.require_gpu(q)
    lib = nat.load()
    q, k, v, do = _aligned(q), _aligned(k), _aligned(v), _aligned(do)
    prob, _keep = _problem(q, fixed, cu_seqlens, max_doc_len, logit_scale, attend_current, product, fused)
    fn = lib.sba_attn_bwd if fixed else lib.sba_varlen_bwd
    drv = dr if dr is not None and dr.numel() else None
    if table.numel() == 0:
        raise ValueError("the backward needs the carry table of a forward that ran with gradients enabled")
    with torch.cuda.device(q.device):
        code = fn(ctypes.byref(prob), sched.data_ptr(), _nbytes(sched),
                  ctypes.byref(nat.view4(q, fixed)), ctypes.byref(nat.view4(k, fixed)),
                  ctypes.byref(nat.view4(v, fixed)), ctypes.byref(nat.view4(do, fixed)),
                  ctypes.byref(nat.view4(drv, fixed, per_row=True)),
                  table.data_ptr(), gtab.data_ptr(), min(_nbytes(table), _nbytes(gtab)),
                  ctypes.byref(nat.view4(dq, fixed)), ctypes.byref(nat.view4(dk, fixed)),
                  ctypes.byref(nat.view4(dv, fixed)), nat.stream_ptr(q.device))
    nat.check(code, "sba_attn_bwd" if fixed else "sba_varlen_bwd")


# The four operators under upstream's names.  Outputs and workspaces are arguments that are
# written in place; `table` may be empty when no backward will follow.
@custom_op("varlen_fwd", mutates_args={"o", "rem", "table", "sched"})
def _compileable_forward(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cu_seqlens: torch.Tensor,
                         max_seqlens: int, logit_scale: float, attend_current: bool, product: bool, fused: bool,
                         o: torch.Tensor, rem: torch.Tensor, table: torch.Tensor, sched: torch.Tensor,
                         build_schedule: bool = True) -> None:
    _launch_fwd(False, q, k, v, cu_seqlens, max_seqlens, logit_scale, attend_current, product, fused,
                o, rem, table, sched, build_schedule=build_schedule)


@custom_op("varlen_bwd", mutates_args={"gtab", "dq", "dk", "dv"})
def _compileable_backward(do: torch.Tensor, dr: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                          cu_seqlens: torch.Tensor, max_seqlens: int, logit_scale: float, attend_current: bool,
                          product: bool, fused: bool, table: torch.Tensor, sched: torch.Tensor, gtab: torch.Tensor,
                          dq: torch.Tensor, dk: torch.Tensor, dv: torch.Tensor) -> None:
    _launch_bwd(False, do, dr, q, k, v, cu_seqlens, max_seqlens, logit_scale, attend_current, product, fused,
                table, sched, gtab, dq, dk, dv)


@custom_op("attn_fwd", mutates_args={"o", "rem", "table", "sched"})
def _compileable_fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, logit_scale: float, attend_current: bool,
                     product: bool, fused: bool, o: torch.Tensor, rem: torch.Tensor, table: torch.Tensor,
                     sched: torch.Tensor, build_schedule: bool = True) -> None:
    _launch_fwd(True, q, k, v, None, q.shape[2], logit_scale, attend_current, product, fused, o, rem, table, sched,
                build_schedule=build_schedule)


@custom_op("attn_bwd", mutates_args={"gtab", "dq", "dk", "dv"})
def _compileable_bwd(do: torch.Tensor, dr: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                     logit_scale: float, attend_current: bool, product: bool, fused: bool, table: torch.Tensor,
                     sched: torch.Tensor, gtab: torch.Tensor, dq: torch.Tensor, dk: torch.Tensor,
                     dv: torch.Tensor) -> None:
    _launch_bwd(True, do, dr, q, k, v, None, q.shape[2], logit_scale, attend_current, product, fused,
                table, sched, gtab, dq, dk, dv)


# ---------------------------------------------------------------------------------------------
# what the autograd functions call
# ---------------------------------------------------------------------------------------------
def _check_cu(cu_seqlens: torch.Tensor, like: torch.Tensor) -> torch.Tensor:
    if cu_seqlens.dim() != 1:
        raise ValueError("cu_seqlens must be 1-d")
    if cu_seqlens.dtype not in (torch.int32, torch.int64):
        raise ValueError("cu_seqlens must be int32 or int64")
    if cu_seqlens.device != like.device:
        cu_seqlens = cu_seqlens.to(like.device)
    return cu_seqlens


# Schedules already built on a device: the tile lists depend only on the documents (cu_seqlens, or
# batch and length of a fixed-length call) and on the token count, and a model hands the same
# cu_seqlens tensor to every layer, so the scheduler kernel runs once per tensor instead of once per
# layer.  Entries: (weak reference to cu_seqlens or None, its version, key, schedule tensor), newest
# last; the key holds the stream, so a schedule is only ever reused behind the launch that wrote it.
_sched_cache = []
_SCHED_CACHE_SIZE = 8


def _schedule_workspace(cu: Optional[torch.Tensor], sched_bytes: int, batch: int, tokens: int, device):
    """(schedule tensor, whether its contents still have to be built).  Eager mode only remembers;
    while torch.compile traces, and while the stream is being captured into a graph (whose replays
    must not depend on a tensor this cache may drop), every call gets a workspace of its own."""
    if torch.compiler.is_compiling() or torch.cuda.is_current_stream_capturing():
        return torch.empty(sched_bytes, dtype=torch.uint8, device=device), True
    version = None if cu is None else _version_of(cu)
    key = (device, torch.cuda.current_stream(device).cuda_stream, batch, tokens, sched_bytes)
    with _cache_lock:
        if cu is None or version is not None:
            for i in range(len(_sched_cache) - 1, -1, -1):
                ref, ver, k, sched = _sched_cache[i]
                if k == key and (ref is None if cu is None else (ref is not None and ref() is cu)):
                    if ver == version:
                        return sched, False
                    del _sched_cache[i]
                    break
        sched = torch.empty(sched_bytes, dtype=torch.uint8, device=device)
        if cu is None or version is not None:
            _sched_cache[:] = [e for e in _sched_cache if e[0] is None or e[0]() is not None][-(_SCHED_CACHE_SIZE - 1):]
            _sched_cache.append((None if cu is None else weakref.ref(cu), version, key, sched))
        return sched, True


def run_forward(q, k, v, fixed: bool, cu_seqlens, max_seqlens, inv_temp: float, attend_current: bool,
                need_table: bool, fused: bool = False, return_attention: bool = False):
    """Returns (o, rem, state); ``state`` = (table, sched, cu_seqlens, max_doc_len, product) is what
    the backward needs (upstream keeps its fp32 ``neg_log_acc`` there).  With ``fused`` the first
    output is ``o + rem[..., None] * v``.  With ``return_attention`` a fourth value follows: the
    dense fp32 attention weights ``[(B,) H, T, T]`` (upstream sb_varlen_fwd.py:421-425,
    sb_fwd.py:147-151; eager mode only, quadratic memory)."""
    nat.require_gpu(q)
    d = q.shape[-1]
    dpad = _padded_dim(d)
    product = PRODUCT_SPACE
    cdt = compute_dtype(q.dtype)
    qp, kp, vp = (_prep(t, dpad, cdt) for t in (q, k, v))
    lengths = None
    if fixed:
        B, H, T, _ = qp.shape
        n_docs, max_len, cu = 0, T, None
    else:
        H, T, _ = qp.shape
        B = 1
        cu = _check_cu(cu_seqlens, q)
        n_docs = cu.numel()
        max_len = T if max_seqlens is None else max(1, min(int(max_seqlens), T))
        cu_vals = host_cu_seqlens(cu)
        if cu_vals is not None:
            # lengths known on the host: malformed input raises here, the tables get their exact
            # size, and results do not depend on max_seqlens at all
            _, max_len, lengths = _lengths_info(cu_vals, T)     # (`lengths`: the table entries they need)
    sched_bytes, table_floats = workspace_sizes(fixed, B, H, T, n_docs, max_len, lengths)
    # Every row is written by the library: rows of documents by the forward kernel, rows that
    # belong to no document are cleared (upstream leaves those uninitialised).
    o = torch.empty_like(qp)
    rem = torch.empty_like(qp[..., 0])
    keep_table = need_table and not RECOMPUTE_TABLE
    table = torch.empty(table_floats if keep_table else 0, dtype=torch.float32, device=q.device)
    sched, build = _schedule_workspace(cu, sched_bytes, B, T, q.device)
    if return_attention:
        weights = torch.zeros(qp.shape[:-1] + (T,), dtype=torch.float32, device=q.device)
        _launch_fwd(fixed, qp, kp, vp, cu, max_len, float(inv_temp), bool(attend_current), product, bool(fused),
                    o, rem, table, sched, weights=weights, build_schedule=build)
    elif fixed:
        _compileable_fwd(qp, kp, vp, float(inv_temp), bool(attend_current), product, bool(fused),
                         o, rem, table, sched, build)
    else:
        _compileable_forward(qp, kp, vp, cu, max_len, float(inv_temp), bool(attend_current), product,
                             bool(fused), o, rem, table, sched, build)
        if VALIDATE and not torch.compiler.is_compiling():
            check_status(sched, table, H, max_len)
    if dpad != d or q.dtype != cdt:
        o = o[..., :d].to(q.dtype)
        rem = rem.to(q.dtype)
    state = (table, sched, cu, max_len, product)
    return (o, rem, state, weights) if return_attention else (o, rem, state)


def check_status(sched: torch.Tensor, table: Optional[torch.Tensor] = None, heads: int = 1,
                 max_doc_len: Optional[int] = None) -> None:
    """Read the scheduler's status words back (synchronises) and raise on malformed cu_seqlens, on
    carry tables smaller than the documents need, or on a document longer than the declared
    ``max_doc_len`` (which the backward's launch is sized with)."""
    hdr = sched[:32].view(torch.int32).tolist()
    status, need, longest = hdr[0], hdr[3], hdr[6]
    if status == 0 and table is not None and table.numel() and need > (((table.numel() - _WORK_WORDS) // heads) & ~31):
        status = 4
    if status == 0 and max_doc_len is not None and longest > max_doc_len:
        status = 5
    if status != 0:
        raise ValueError("sb_attn_varlen: " + nat.STATUS_MESSAGES.get(status, f"scheduler status {status}"))


# One gradient table (and, with RECOMPUTE_TABLE, one rebuilt stick table) per (device, stream), shared by
# every backward on that stream: the dk/dv pass of one backward has read them before the next backward
# on the same stream writes them.  The buffer only ever grows: packed-document training changes
# cu_seqlens, and with it the exact table size, with every batch, and a buffer per size would
# allocate on every step and pin what it allocated before.  A request gets the first `numel` floats
# of the buffer; growth goes to the next eighth of a power of two, and by at least a quarter, so that a
# sequence of slowly growing sizes does not reallocate every time.
_gtab_cache = {}


def _size_class(numel: int) -> int:
    if numel <= 1 << 16:
        return 1 << 16
    step = 1 << max(0, numel.bit_length() - 4)     # an eighth of the power of two below numel
    return (numel + step - 1) // step * step


def _scratch_table(numel: int, device, role: str) -> torch.Tensor:
    # (a captured graph gets a table of its own, from the graph's memory pool: its replays must not
    # write into a tensor this cache may have dropped since)
    if torch.compiler.is_compiling() or torch.cuda.is_current_stream_capturing():
        return torch.empty(numel, dtype=torch.float32, device=device)
    key = (device, torch.cuda.current_stream(device).cuda_stream, role)
    with _cache_lock:
        buf = _gtab_cache.get(key)
        if buf is None or buf.numel() < numel:
            grown = 0 if buf is None else buf.numel() * 5 // 4     # outgrown once: leave room for the next batch too
            _gtab_cache.pop(key, None)      # (the old buffer goes back to the allocator before the new one is asked for)
            buf = None
            buf = _gtab_cache[key] = torch.empty(_size_class(max(numel, grown)), dtype=torch.float32, device=device)
        return buf[:numel]


def _grad_table(like: torch.Tensor) -> torch.Tensor:
    return _scratch_table(like.numel(), like.device, "grad")


def _rebuild_table(qp, kp, vp, fixed: bool, sched, cu, max_len: int, inv_temp: float, attend_current: bool,
                   product: bool, fused: bool) -> torch.Tensor:
    """The carry table of a forward that kept none (RECOMPUTE_TABLE): the forward kernel once more, in
    the variant that forms the weights' running stick but neither multiplies them with V nor writes
    o and rem.  Same arithmetic on the same inputs with the same schedule: the same table, bit for bit."""
    if fixed:
        B, H, T, _ = qp.shape
        n_docs, lengths = 0, None
    else:
        (H, T, _), B = qp.shape, 1
        n_docs = cu.numel()
        cu_vals = host_cu_seqlens(cu)
        lengths = None if cu_vals is None else _lengths_info(cu_vals, T)[2]
    _, table_floats = workspace_sizes(fixed, B, H, T, n_docs, max_len, lengths)
    table = _scratch_table(table_floats, qp.device, "stick")
    o = torch.empty(0, dtype=qp.dtype, device=qp.device)     # (no elements: only the table is written)
    rem = torch.empty(0, dtype=qp.dtype, device=qp.device)
    if fixed:
        _compileable_fwd(qp, kp, vp, inv_temp, attend_current, product, fused, o, rem, table, sched, False)
    else:
        _compileable_forward(qp, kp, vp, cu, max_len, inv_temp, attend_current, product, fused, o, rem, table, sched, False)
    return table


def release_workspaces() -> None:
    """Drop the cached gradient tables, schedules and host copies of cu_seqlens."""
    with _cache_lock:
        _gtab_cache.clear()
        del _host_cu_cache[:]
        del _sched_cache[:]
        del _stripped_views[:]


def run_backward(q, k, v, do, drem, fixed: bool, state, inv_temp: float, attend_current: bool, dkdv_dtype=None,
                 fused: bool = False):
    """dq, dk, dv.  With ``fused``, ``do`` is the gradient of ``o + rem[..., None] * v``."""
    table, sched, cu, max_len, product = state
    d = q.shape[-1]
    dpad = _padded_dim(d)
    cdt = compute_dtype(q.dtype)
    qp, kp, vp = (_prep(t, dpad, cdt) for t in (q, k, v))
    unscale = None
    if cdt == torch.float16 and q.dtype == torch.float32:
        # float32 caller on the float16 kernels: a power of two brings the largest incoming gradient into [4, 8)
        # (the backward is linear in (do, drem); no value is read back to the host)
        amax = do.detach().abs().amax().float()
        if drem is not None:
            amax = torch.maximum(amax, drem.detach().abs().amax().float())
        expo = torch.floor(torch.log2(amax.clamp(min=2.0 ** -100, max=2.0 ** 100)))
        scale = torch.exp2(2.0 - expo)
        unscale = torch.exp2(expo - 2.0)
        do = do.float() * scale
        if drem is not None:
            drem = drem.float() * scale
    dop = _prep(do, dpad, cdt, incoming_grad=True)
    if drem is None:
        dremp = torch.empty(0, dtype=cdt, device=q.device)
    else:
        dremp = drem if drem.dtype == cdt else drem.to(cdt)
        if torch.compiler.is_compiling():
            dremp = dremp.contiguous()
    dq, dk, dv = torch.empty_like(qp), torch.empty_like(kp), torch.empty_like(vp)
    if table.numel() == 0 and RECOMPUTE_TABLE:
        table = _rebuild_table(qp, kp, vp, fixed, sched, cu, max_len, float(inv_temp), bool(attend_current), product,
                               bool(fused))
    gtab = _grad_table(table)
    if fixed:
        _compileable_bwd(dop, dremp, qp, kp, vp, float(inv_temp), bool(attend_current), product, bool(fused),
                         table, sched, gtab, dq, dk, dv)
    else:
        _compileable_backward(dop, dremp, qp, kp, vp, cu, max_len, float(inv_temp), bool(attend_current),
                              product, bool(fused), table, sched, gtab, dq, dk, dv)
    if unscale is not None:
        dq, dk, dv = (t[..., :d].float() * unscale for t in (dq, dk, dv))
    if dpad != d or q.dtype != cdt or k.dtype != cdt or v.dtype != cdt or dkdv_dtype not in (None, cdt):
        dq = dq[..., :d].to(q.dtype)
        dk = dk[..., :d].to(k.dtype if dkdv_dtype is None else dkdv_dtype)
        dv = dv[..., :d].to(v.dtype if dkdv_dtype is None else dkdv_dtype)
    return dq, dk, dv


def default_inv_temp(head_dim: int) -> float:
    return 1.0 / math.sqrt(head_dim)
