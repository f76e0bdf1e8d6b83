"""Stick-breaking attention for AMD Instinct MI355X (gfx950).

The two public operators have the names and signatures of upstream
``stickbreaking_attention/__init__.py:1-2``; the device code lives in ``libsba.so`` (hand-written
HIP behind the C ABI of ``include/sba.h``) and is loaded on first use.
"""
from ._native import LIB_PATH as _LIB_PATH
from .sb_attn import sb_attn, sb_attn_fused
from .sb_varlen import sb_attn_varlen, sb_attn_varlen_fused

__all__ = ["sb_attn", "sb_attn_varlen", "sb_attn_fused", "sb_attn_varlen_fused", "library_path"]
__version__ = "1.0.0"


def library_path() -> str:
    """Where the shared library is expected (built by ``make -C stickbreaking-attention_amd/csrc``)."""
    return _LIB_PATH
