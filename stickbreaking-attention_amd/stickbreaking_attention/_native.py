"""ctypes binding of libsba.so (the C ABI declared in include/sba.h).

The shared library is built in-tree by ``stickbreaking-attention_amd/csrc/Makefile`` into
``stickbreaking-attention_amd/lib/libsba.so``.  There is no fallback: if the library is missing
or the device is not an MI355X the operators raise.
"""
from __future__ import annotations

import ctypes
import os
import threading
from typing import Optional

import torch

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_PKG_DIR), "lib", "libsba.so")

SBA_BF16 = 1
SBA_F16 = 2
FLAG_ATTEND_CURRENT = 1
FLAG_CU_INT64 = 2
FLAG_PRODUCT_SPACE = 4
FLAG_FIXED_LENGTH = 8
FLAG_FUSE_REMAINDER = 16
FLAG_TABLE_ONLY = 32

STATUS_MESSAGES = {
    1: "cu_seqlens is not a non-decreasing sequence within [0, total_tokens]",
    4: "the carry tables are too small for the documents in cu_seqlens (max_seqlens under-states a document)",
    5: "a document in cu_seqlens is longer than max_seqlens (the backward refuses to run: its outputs are NaN)",
}


class SbaView(ctypes.Structure):
    _fields_ = [("ptr", ctypes.c_void_p), ("stride_b", ctypes.c_int64),
                ("stride_h", ctypes.c_int64), ("stride_t", ctypes.c_int64)]


class SbaProblem(ctypes.Structure):
    _fields_ = [("dtype", ctypes.c_int32), ("head_dim", ctypes.c_int32), ("heads", ctypes.c_int32),
                ("batch", ctypes.c_int32), ("tokens", ctypes.c_int32), ("n_docs", ctypes.c_int32),
                ("max_doc_len", ctypes.c_int32), ("flags", ctypes.c_uint32),
                ("inv_temp", ctypes.c_float), ("cu_seqlens", ctypes.c_void_p)]


class SbaGeometry(ctypes.Structure):
    _fields_ = [("query_list_tiles", ctypes.c_int), ("key_list_tiles", ctypes.c_int),
                ("query_list_word", ctypes.c_int), ("key_list_word", ctypes.c_int), ("tile_words", ctypes.c_int),
                ("schedule_words", ctypes.c_longlong),
                ("fwd_tiles", ctypes.c_int), ("dq_tiles", ctypes.c_int),
                ("long_tiles_bound", ctypes.c_int), ("tail_tiles_bound", ctypes.c_int),
                ("dkdv_main_tiles", ctypes.c_int), ("dkdv_tail_tiles", ctypes.c_int)]


EXPORTS = (
    "sba_version", "sba_error_string", "sba_schedule_bytes", "sba_table_bytes", "sba_table_bytes_for_lengths",
    "sba_build_schedule",
    "sba_varlen_fwd", "sba_varlen_bwd", "sba_attn_fwd", "sba_attn_bwd", "sba_set_timing", "sba_set_dkdv_workgroups",
    "sba_last_kernel_ms", "sba_varlen_fwd_weights", "sba_attn_fwd_weights", "sba_varlen_fwd_static",
    "sba_launch_geometry",
)

_lib = None
_lock = threading.Lock()


def load():
    """Load libsba.so once and declare the prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"libsba.so not found at {LIB_PATH}: build it with "
                "`make -C stickbreaking-attention_amd/csrc` (hipcc, gfx950)")
        lib = ctypes.CDLL(LIB_PATH)
        P, V, vp = ctypes.POINTER(SbaProblem), ctypes.POINTER(SbaView), ctypes.c_void_p
        lib.sba_version.restype = ctypes.c_int
        lib.sba_error_string.restype = ctypes.c_char_p
        lib.sba_error_string.argtypes = [ctypes.c_int]
        lib.sba_launch_geometry.restype = ctypes.c_int
        lib.sba_launch_geometry.argtypes = [ctypes.POINTER(SbaProblem), ctypes.POINTER(SbaGeometry)]
        lib.sba_schedule_bytes.restype = ctypes.c_size_t
        lib.sba_schedule_bytes.argtypes = [P]
        lib.sba_table_bytes.restype = ctypes.c_size_t
        lib.sba_table_bytes.argtypes = [P]
        sz = ctypes.c_size_t
        lib.sba_table_bytes_for_lengths.restype = ctypes.c_size_t
        lib.sba_table_bytes_for_lengths.argtypes = [P, ctypes.POINTER(ctypes.c_int64), ctypes.c_int]
        lib.sba_build_schedule.restype = ctypes.c_int
        lib.sba_build_schedule.argtypes = [P, vp, sz, vp]
        for name in ("sba_varlen_fwd", "sba_attn_fwd"):
            f = getattr(lib, name)
            f.restype = ctypes.c_int
            f.argtypes = [P, vp, sz, V, V, V, V, V, vp, sz, vp]
        for name in ("sba_varlen_fwd_weights", "sba_attn_fwd_weights"):
            f = getattr(lib, name)
            f.restype = ctypes.c_int
            f.argtypes = [P, vp, sz, V, V, V, V, V, vp, sz, vp, sz, vp]
        for name in ("sba_varlen_bwd", "sba_attn_bwd"):
            f = getattr(lib, name)
            f.restype = ctypes.c_int
            f.argtypes = [P, vp, sz, V, V, V, V, V, vp, vp, sz, V, V, V, vp]
        lib.sba_varlen_fwd_static.restype = ctypes.c_int
        lib.sba_varlen_fwd_static.argtypes = [P, V, V, V, V, V, vp]
        lib.sba_set_timing.restype = None
        lib.sba_set_timing.argtypes = [ctypes.c_int]
        lib.sba_set_dkdv_workgroups.restype = None
        lib.sba_set_dkdv_workgroups.argtypes = [ctypes.c_int]
        lib.sba_last_kernel_ms.restype = ctypes.c_float
        lib.sba_last_kernel_ms.argtypes = [ctypes.c_int]
        _lib = lib
    return _lib


def check(code: int, what: str) -> None:
    if code == 0:
        return
    msg = load().sba_error_string(code).decode()
    if code < 0:
        raise ValueError(f"{what}: {msg} (SBA error {code})")
    raise RuntimeError(f"{what}: HIP error {code}: {msg}")


def view4(t: Optional[torch.Tensor], fixed: bool, per_row: bool = False) -> SbaView:
    """Describe a [B,H,T,(d)] (fixed) or [H,T,(d)] (varlen) tensor; None -> null view."""
    if t is None:
        return SbaView(None, 0, 0, 0)
    nd = t.dim()
    want = (3 if fixed else 2) + (0 if per_row else 1)
    if nd != want:
        raise ValueError(f"expected a {want}-d tensor, got shape {tuple(t.shape)}")
    if not per_row and t.stride(-1) != 1:
        raise ValueError("the head_dim axis must be contiguous (stride 1)")
    s = t.stride()
    if fixed:
        return SbaView(t.data_ptr(), s[0], s[1], s[2])
    return SbaView(t.data_ptr(), 0, s[0], s[1])


def stream_ptr(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def require_gpu(t: torch.Tensor) -> None:
    if not t.is_cuda:
        raise RuntimeError(
            "stick-breaking attention runs on MI355X (gfx950) only; got a tensor on "
            f"{t.device}. There is no CPU implementation in this package.")
