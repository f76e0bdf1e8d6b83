"""Stick-breaking attention for AMD Instinct MI355X -- same import surface as upstream
``stickbreaking_attention/__init__.py:1-2``."""
from .sb_attn import sb_attn
from .sb_varlen import sb_attn_varlen

__all__ = ["sb_attn", "sb_attn_varlen"]
