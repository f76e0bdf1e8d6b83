"""Host glue between the autograd functions and libsba.so.

Mirrors what the upstream host launchers do around their Triton kernels -- allocate outputs
and private state with PyTorch, pass raw pointers and strides, launch on the current stream
(upstream ``varlen_fwd`` sb_varlen/sb_varlen_fwd.py:413-451, ``varlen_bwd``
sb_varlen/sb_varlen_bwd.py:484-539, ``_fwd`` sb_attn/sb_fwd.py:139-174, ``_bwd``
sb_attn/sb_bwd.py:163-205) -- with the device code behind a C ABI instead of a JIT.
"""
from __future__ import annotations

import ctypes
import math
import os
from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from . import _native as nat

# Carry the stick as a running product (2 transcendentals per score) instead of a running
# log2 sum (3 per score).  Overridable for A/B measurements.
PRODUCT_SPACE = os.environ.get("SBA_LOG_SPACE", "0") != "1"

# When True every forward reads back the scheduler's status word (one device sync) and raises
# on malformed cu_seqlens instead of returning untouched outputs.
VALIDATE = os.environ.get("SBA_VALIDATE", "0") == "1"

SUPPORTED_HEAD_DIMS = (64, 128)


@dataclass
class Plan:
    """Everything the kernels need besides the tensors; built once per forward."""
    problem: nat.SbaProblem
    schedule: torch.Tensor       # uint8 workspace holding the tile lists
    fixed: bool
    table_bytes: int
    head_dim: int                # padded head_dim the kernels run at
    orig_head_dim: int
    keepalive: tuple             # tensors whose pointers live inside `problem`


def _padded_dim(d: int) -> int:
    for s in SUPPORTED_HEAD_DIMS:
        if d <= s:
            return s
    raise ValueError(f"head_dim {d} is not supported (maximum {SUPPORTED_HEAD_DIMS[-1]})")


def _prep(t: torch.Tensor, dpad: int) -> torch.Tensor:
    """bf16, head_dim padded with zeros to `dpad`, rows 16-byte aligned."""
    if t.dtype != torch.bfloat16:
        t = t.to(torch.bfloat16)
    d = t.shape[-1]
    if d != dpad:
        t = torch.nn.functional.pad(t, (0, dpad - d))
    ok = t.stride(-1) == 1 and t.data_ptr() % 16 == 0 and all(s % 8 == 0 for s in t.stride()[:-1])
    return t if ok else t.contiguous()


def make_plan(q: torch.Tensor, fixed: bool, cu_seqlens: Optional[torch.Tensor], max_seqlens: Optional[int],
              inv_temp: float, attend_current: bool) -> Plan:
    nat.require_gpu(q)
    lib = nat.load()
    d = q.shape[-1]
    dpad = _padded_dim(d)
    flags = 0
    if attend_current:
        flags |= nat.FLAG_ATTEND_CURRENT
    if PRODUCT_SPACE:
        flags |= nat.FLAG_PRODUCT_SPACE
    keep = ()
    if fixed:
        B, H, T, _ = q.shape
        flags |= nat.FLAG_FIXED_LENGTH
        prob = nat.SbaProblem(nat.SBA_BF16, dpad, H, B, T, 0, T, flags, float(inv_temp), None)
    else:
        H, T, _ = q.shape
        if cu_seqlens.dim() != 1:
            raise ValueError("cu_seqlens must be 1-d")
        if cu_seqlens.dtype == torch.int64:
            flags |= nat.FLAG_CU_INT64
        elif cu_seqlens.dtype != torch.int32:
            raise ValueError("cu_seqlens must be int32 or int64")
        if cu_seqlens.device != q.device:
            cu_seqlens = cu_seqlens.to(q.device)
        cu_seqlens = cu_seqlens.contiguous()
        keep = (cu_seqlens,)
        bound = T if max_seqlens is None else max(1, min(int(max_seqlens), T))
        prob = nat.SbaProblem(nat.SBA_BF16, dpad, H, 1, T, cu_seqlens.numel(), bound, flags,
                              float(inv_temp), cu_seqlens.data_ptr() if cu_seqlens.numel() else None)
    nbytes = lib.sba_schedule_bytes(ctypes.byref(prob))
    if nbytes == 0:
        raise ValueError("invalid problem description for stick-breaking attention")
    sched = torch.empty(nbytes, dtype=torch.uint8, device=q.device)
    with torch.cuda.device(q.device):
        nat.check(lib.sba_build_schedule(ctypes.byref(prob), sched.data_ptr(), nat.stream_ptr(q.device)),
                  "sba_build_schedule")
    return Plan(prob, sched, fixed, lib.sba_table_bytes(ctypes.byref(prob)), dpad, d, keep)


def check_status(plan: Plan) -> None:
    """Read the scheduler's status word back (synchronises) and raise on malformed input."""
    status = int(plan.schedule[:4].view(torch.int32).item())
    if status != 0:
        raise ValueError("sb_attn_varlen: " + nat.STATUS_MESSAGES.get(status, f"scheduler status {status}"))


def forward(plan: Plan, q, k, v, need_table: bool) -> Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    lib = nat.load()
    fixed = plan.fixed
    qp, kp, vp = (_prep(t, plan.head_dim) for t in (q, k, v))
    padded = plan.head_dim != plan.orig_head_dim or q.dtype != torch.bfloat16
    # Every row is written by the library: rows of documents by the forward kernel, rows that
    # belong to no document are cleared (upstream leaves those uninitialised).
    o = torch.empty_like(qp)
    rem = torch.empty_like(qp[..., 0])
    table = None
    if need_table:
        table = torch.empty(plan.table_bytes // 4, dtype=torch.float32, device=q.device)
    fn = lib.sba_attn_fwd if fixed else lib.sba_varlen_fwd
    with torch.cuda.device(q.device):
        code = fn(ctypes.byref(plan.problem), plan.schedule.data_ptr(),
                  ctypes.byref(nat.view4(qp, fixed)), ctypes.byref(nat.view4(kp, fixed)),
                  ctypes.byref(nat.view4(vp, fixed)), ctypes.byref(nat.view4(o, fixed)),
                  ctypes.byref(nat.view4(rem, fixed, per_row=True)),
                  table.data_ptr() if table is not None else None, nat.stream_ptr(q.device))
    nat.check(code, "sba_attn_fwd" if fixed else "sba_varlen_fwd")
    if VALIDATE and not fixed:
        check_status(plan)
    if padded:
        o = o[..., :plan.orig_head_dim].to(q.dtype)
        rem = rem.to(q.dtype)
    return o, rem, table


def backward(plan: Plan, q, k, v, do, drem, table, dkdv_dtype=None):
    lib = nat.load()
    fixed = plan.fixed
    qp, kp, vp, dop = (_prep(t, plan.head_dim) for t in (q, k, v, do))
    dremp = None
    if drem is not None:
        dremp = drem if drem.dtype == torch.bfloat16 else drem.to(torch.bfloat16)
    padded = plan.head_dim != plan.orig_head_dim or q.dtype != torch.bfloat16
    dq, dk, dv = torch.empty_like(qp), torch.empty_like(kp), torch.empty_like(vp)
    gtab = torch.empty(plan.table_bytes // 4, dtype=torch.float32, device=q.device)
    fn = lib.sba_attn_bwd if fixed else lib.sba_varlen_bwd
    with torch.cuda.device(q.device):
        code = fn(ctypes.byref(plan.problem), plan.schedule.data_ptr(),
                  ctypes.byref(nat.view4(qp, fixed)), ctypes.byref(nat.view4(kp, fixed)),
                  ctypes.byref(nat.view4(vp, fixed)), ctypes.byref(nat.view4(dop, fixed)),
                  ctypes.byref(nat.view4(dremp, fixed, per_row=True)),
                  table.data_ptr(), gtab.data_ptr(),
                  ctypes.byref(nat.view4(dq, fixed)), ctypes.byref(nat.view4(dk, fixed)),
                  ctypes.byref(nat.view4(dv, fixed)), nat.stream_ptr(q.device))
    nat.check(code, "sba_attn_bwd" if fixed else "sba_varlen_bwd")
    if padded:
        dq = dq[..., :plan.orig_head_dim].to(q.dtype)
        dk = dk[..., :plan.orig_head_dim].to(k.dtype if dkdv_dtype is None else dkdv_dtype)
        dv = dv[..., :plan.orig_head_dim].to(v.dtype if dkdv_dtype is None else dkdv_dtype)
    return dq, dk, dv


def default_inv_temp(head_dim: int) -> float:
    return 1.0 / math.sqrt(head_dim)
