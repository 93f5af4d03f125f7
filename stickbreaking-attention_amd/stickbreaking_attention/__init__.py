"""Stick-breaking attention for AMD MI355X: the operator API of speedcell4/stickbreaking-attention
(stickbreaking_attention/__init__.py:1-2) on hand-written gfx950 kernels."""
from ._native import set_backward_workspace_limit
from .sb_attn import sb_attn
from .sb_varlen import sb_attn_varlen

__all__ = ["sb_attn", "sb_attn_varlen", "set_backward_workspace_limit"]
