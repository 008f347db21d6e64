"""Fused LayerNorm + modulate (mirror of ``adaln_modulate_triton``, utils/adaln_triton.py:89-126)."""
from __future__ import annotations

import torch

from .. import _native


def adaln_modulate(x: torch.Tensor, e_scale: torch.Tensor, e_shift: torch.Tensor, frame_seqlen: int,
                   eps: float = 1e-6, add_one_to_scale: bool = True,
                   amax_out=None) -> torch.Tensor:
    """``LayerNorm(x) * (1 + e_scale) + e_shift`` over x [B, F*frame_seqlen, C] with per-frame
    e_scale / e_shift [B, F, 1, C]; bf16 roundings placed as in the eager graph.  ``amax_out``
    (an amax ticket, ``_native.amax_ticket``; an extension) receives the absolute maximum of the result."""
    return _native.adaln_modulate(x, e_scale, e_shift, frame_seqlen, eps, add_one_to_scale, amax_out=amax_out)


adaln_modulate_triton = adaln_modulate


def gate_residual(x: torch.Tensor, y: torch.Tensor, gate: torch.Tensor, frame_seqlen: int) -> torch.Tensor:
    """``x + (y.unflatten(1, (F, frame_seqlen)) * gate).flatten(1, 2)`` of the DiT block
    (wan_5b/modules/causal_model.py:889, 919-920) in one pass; product and sum are each rounded to bf16
    like the two eager operations."""
    return _native.gate_residual(x, y, gate, frame_seqlen)
