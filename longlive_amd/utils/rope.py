"""3-D RoPE: frequency table, per-chunk cos/sin and the fused apply kernel.

Mirrors ``rope_params`` (wan_5b/modules/model.py:29-36), the table layout of
``CausalWanModel`` (wan_5b/modules/causal_model.py:1075-1081), the per-chunk frequency gather of
``causal_rope_apply`` (causal_model.py:138-178) and ``rope_apply_triton`` (utils/rope_triton.py:94-135).
"""
from __future__ import annotations

import torch

from .. import _native


def rope_params(max_seq_len: int, dim: int, theta: float = 10000.0) -> torch.Tensor:
    """Angles pos * theta^(-2j/dim), float64 [max_seq_len, dim/2] (the reference stores exp(i*angle))."""
    assert dim % 2 == 0
    inv = 1.0 / torch.pow(theta, torch.arange(0, dim, 2, dtype=torch.float64).div(dim))
    return torch.outer(torch.arange(max_seq_len, dtype=torch.float64), inv)


def build_rope_angles(head_dim: int = 128, max_pos: int = 1024) -> torch.Tensor:
    """[max_pos, head_dim/2] float64 angles; columns = [frame | height | width] parts of sizes
    c - 2*(c//3), c//3, c//3 with c = head_dim/2, each built with its own ``dim``."""
    d = head_dim
    return torch.cat([rope_params(max_pos, d - 4 * (d // 6)), rope_params(max_pos, 2 * (d // 6)),
                      rope_params(max_pos, 2 * (d // 6))], dim=1)


def temporal_angles(frame_angles: torch.Tensor, f: int, start_frame: int, t_scale: float = 1.0,
                    temporal_offset=0.0) -> torch.Tensor:
    """Angles of the temporal part for frames start_frame .. start_frame + f - 1 (mirror of
    ``compute_temporal_freqs``, utils/position_embedding_utils.py:55-107).  Without scale and offset it is a slice
    of the table; otherwise the positions ``(frame + temporal_offset) * t_scale`` (float64) multiply the table's
    angle per position.  ``temporal_offset``: a number (the multi-shot phase offset, shot index times phi,
    pipeline/causal_diffusion_inference.py:545-549) or a 1-D tensor with one entry per frame (of the chunk, or of
    the whole stream, then frames start_frame .. are taken)."""
    is_tensor = torch.is_tensor(temporal_offset)
    if temporal_offset is None:
        temporal_offset = 0.0
    if t_scale == 1.0 and not is_tensor and float(temporal_offset) == 0.0:
        return frame_angles[start_frame:start_frame + f]
    a1 = frame_angles[1]
    base = torch.angle(torch.polar(torch.ones_like(a1), a1))   # the reference recovers it from exp(i * angle)
    positions = torch.arange(f, dtype=torch.float64) + start_frame
    if is_tensor:
        off = temporal_offset.detach().to(device="cpu", dtype=torch.float64)
        if off.ndim == 0:
            positions = positions + off
        elif off.ndim == 1 and off.numel() == f:
            positions = positions + off
        elif off.ndim == 1 and off.numel() >= start_frame + f:
            positions = positions + off[start_frame:start_frame + f]
        else:
            raise ValueError(f"temporal_offset of shape {tuple(off.shape)} does not cover frames "
                             f"{start_frame}..{start_frame + f - 1}")
    else:
        positions = positions + float(temporal_offset)
    return (positions * t_scale).unsqueeze(-1) * base.unsqueeze(0)


def rope_cos_sin(angles: torch.Tensor, f: int, h: int, w: int, start_frame: int = 0,
                 device: torch.device | str | None = None, t_scale: float = 1.0,
                 temporal_offset=0.0) -> tuple[torch.Tensor, torch.Tensor]:
    """float32 cos/sin [f*h*w, head_dim/2] for a (f, h, w) grid whose first frame sits at absolute
    frame ``start_frame``; token order (f, h, w) row-major.  ``t_scale`` / ``temporal_offset``: see
    ``temporal_angles``."""
    c = angles.shape[1]
    parts = angles.split([c - 2 * (c // 3), c // 3, c // 3], dim=1)
    ang = torch.cat([
        temporal_angles(parts[0], f, start_frame, t_scale, temporal_offset).view(f, 1, 1, -1).expand(f, h, w, -1),
        parts[1][:h].view(1, h, 1, -1).expand(f, h, w, -1),
        parts[2][:w].view(1, 1, w, -1).expand(f, h, w, -1),
    ], dim=-1).reshape(f * h * w, c)
    cos, sin = torch.cos(ang).float(), torch.sin(ang).float()
    if device is not None:
        cos, sin = cos.to(device), sin.to(device)
    return cos.contiguous(), sin.contiguous()


def rope_apply(x: torch.Tensor, cos_f32: torch.Tensor, sin_f32: torch.Tensor, seq_len: int | None = None) -> torch.Tensor:
    """x bf16 [S, N, D]: rows < seq_len get pairs (2j, 2j+1) rotated by (cos, sin)[s, j] in fp32,
    the rest are copied through; returns a new tensor of the same shape and dtype."""
    return _native.rope_apply(x, cos_f32, sin_f32, seq_len)


# the reference's name for the same entry point
rope_apply_triton = rope_apply
