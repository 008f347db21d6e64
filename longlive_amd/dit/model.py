"""Causal DiT block and model (inference with an NVFP4 KV cache).

Module and parameter names follow the reference model so that its checkpoints, its module filter
(utils/quant.py:44-58) and its NVFP4 state dicts apply unchanged:
``CausalWanAttentionBlock`` (wan_5b/modules/causal_model.py:794-930), ``CausalWanSelfAttention``
(:298-791), ``MultiShotT2VCrossAttention`` (:197-262), ``CausalHead`` (:933-959), ``CausalWanModel``
(:1040-1110, forward :1485-1654).  The ten Linear layers of every block become ``FourOverSixLinear``
through ``quantize_model_with_filter``; norms, RoPE, adaLN and attention call the gfx950 kernels;
the bf16 ends of the model (patch / time / text embeddings, head) are plain torch modules.
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import torch
import torch.nn as nn

from .. import _native
from ..fouroversix.model.modules.linear import FourOverSixLinear
from ..utils import kv_cache as kvc
from ..utils.adaln import adaln_modulate, gate_residual
from ..utils.rope import build_rope_angles, rope_apply, rope_cos_sin


@dataclass
class DiTConfig:
    """Wan2.2-TI2V-5B shape by default (wan_5b/configs/wan_ti2v_5B.py:20-29)."""

    dim: int = 3072
    ffn_dim: int = 14336
    num_heads: int = 24
    num_layers: int = 30
    in_dim: int = 48
    out_dim: int = 48
    text_dim: int = 4096
    text_len: int = 512
    freq_dim: int = 256
    patch_size: tuple = (1, 2, 2)
    eps: float = 1e-6
    num_frame_per_block: int = 3
    local_attn_size: int = 15   # frames kept in the KV cache (sink + window)
    sink_size: int = 3          # frames
    global_sink_size: int = 0   # frames anchored for good (the pipeline sets it to sink_size in multi-shot mode)


class WanRMSNorm(nn.Module):
    """RMS norm over the full model dimension (wan_5b/modules/model.py:82-98)."""

    def __init__(self, dim: int, eps: float = 1e-5) -> None:
        super().__init__()
        self.dim, self.eps = dim, eps
        self.weight = nn.Parameter(torch.ones(dim))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return _native.rms_norm(x, self.weight.data, self.eps)


class WanLayerNorm(nn.LayerNorm):
    def __init__(self, dim: int, eps: float = 1e-6, elementwise_affine: bool = False) -> None:
        super().__init__(dim, elementwise_affine=elementwise_affine, eps=eps)

    def forward(self, x: torch.Tensor, amax_out=None) -> torch.Tensor:
        """``amax_out``: an amax ticket that receives the absolute maximum of the result (device kernel only)."""
        if x.is_cuda and x.dtype == torch.bfloat16 and x.shape[-1] % 8 == 0 and \
                (self.weight is None or self.weight.dtype == torch.bfloat16):
            return _native.layer_norm(x, self.weight, self.bias, self.eps, amax_out=amax_out)
        if amax_out is not None:
            raise ValueError("amax_out needs the device kernel (bfloat16 CUDA input)")
        return super().forward(x).type_as(x)


class QuantizedActivation:
    """An activation that exists only as the NVFP4 operand of the layers that read it (``operand``, built for
    ``layers[0]``'s activation config) together with the shape the bf16 tensor would have had."""

    def __init__(self, operand, shape) -> None:
        self.operand, self.shape = operand, tuple(shape)
        self.device = operand.values.device


def _project_shared(x, layers, amax: torch.Tensor | None = None, amax_outs=None) -> list[torch.Tensor]:
    """Apply several linear layers to the same input.  Quantized layers with the same activation config
    share one quantized operand (bit-identical to quantizing per layer, as the reference does).  ``amax`` is
    the amax ticket that the kernel which produced ``x`` was given; ``amax_outs`` (one entry per layer, ``None``
    for none) are tickets that receive the absolute maximum of a layer's output, which only the quantized path
    can deliver: the return value says whether it did.  ``x`` may be a :class:`QuantizedActivation`."""
    first = layers[0]
    same_config = all(isinstance(m, FourOverSixLinear) for m in layers) and all(
        m.config.get_activation_config() == first.config.get_activation_config() for m in layers)
    if isinstance(x, QuantizedActivation):
        if not same_config:
            raise ValueError("a quantized activation can only feed quantized layers with one activation config")
        outs = FourOverSixLinear.forward_quantized_together(layers, x.operand, amax_outs)
        return [y.reshape(*x.shape[:-1], -1) for y in outs], True
    if same_config:
        xq = first.quantize_input(x.reshape(-1, x.shape[-1]), amax=amax)
        outs = FourOverSixLinear.forward_quantized_together(layers, xq, amax_outs)
        return [y.reshape(*x.shape[:-1], -1) for y in outs], True
    return [m(x) for m in layers], False


def _fused_linear(layer, x: torch.Tensor, *, amax: torch.Tensor | None = None, activation: str | None = None,
                  residual: torch.Tensor | None = None, gate: torch.Tensor | None = None, gate_rows: int = 0,
                  amax_out: torch.Tensor | None = None) -> torch.Tensor | None:
    """``layer(x)`` of a quantized layer with the GEMM epilogue extensions (``residual + y * gate`` etc.);
    ``None`` when the layer is not quantized or the shapes rule the fused epilogue out, so that the caller
    runs the separate operations."""
    if not isinstance(layer, FourOverSixLinear) or layer.out_features % 8 != 0:
        return None
    x2d = x.reshape(-1, x.shape[-1])
    if residual is not None:
        residual = residual.reshape(-1, residual.shape[-1])
        if residual.data_ptr() % 16 or residual.stride(0) % 8 or (gate is not None and (
                gate.data_ptr() % 16 or gate.stride(0) % 8)):
            return None
    out = layer.forward_quantized(layer.quantize_input(x2d, amax=amax), activation, residual=residual, gate=gate,
                                  gate_rows=gate_rows, amax_out=amax_out)
    return out.reshape(*x.shape[:-1], -1)


def _project_out(layer, y: torch.Tensor, amax, residual, gate, gate_rows: int) -> torch.Tensor:
    """``layer(y)``, or ``residual + layer(y) * gate`` (gate [G, C], row ``m // gate_rows``; plain sum without a
    gate) when a residual is given: in the GEMM epilogue for a quantized layer, else as separate operations
    with the same roundings."""
    if residual is None:
        out = _fused_linear(layer, y, amax=amax)
        return layer(y) if out is None else out
    out = _fused_linear(layer, y, amax=amax, residual=residual, gate=gate, gate_rows=gate_rows)
    if out is not None:
        return out
    out = layer(y)
    if gate is None:
        return residual + out
    b, l, c = residual.shape
    return gate_residual(residual, out.contiguous(), gate.view(b, -1, 1, c), gate_rows)


class CausalSelfAttention(nn.Module):
    def __init__(self, dim: int, num_heads: int, eps: float = 1e-6) -> None:
        super().__init__()
        self.dim, self.num_heads, self.head_dim = dim, num_heads, dim // num_heads
        self.q, self.k, self.v, self.o = (nn.Linear(dim, dim) for _ in range(4))
        self.norm_q, self.norm_k = WanRMSNorm(dim, eps), WanRMSNorm(dim, eps)
        self.use_relative_rope = False  # set on the module by the pipeline (pipeline/causal_diffusion_inference.py:316)

    def forward(self, x, cos, sin, kv_cache, current_start, sink_tokens, max_attention_size, *, input_amax=None,
                residual=None, gate=None, gate_rows=0, global_sink_tokens=0, rope_fn=None, collect_kv_amax=True,
                keys_only=False):
        """``input_amax``: the amax ticket the producer of ``x`` was given, if any.
        ``keys_only``: the caller reads the cache update only (the chunk's K and V), not the output: everything
        behind the K / V producers is left out and the output is None.
        ``collect_kv_amax``: leave the maxima of the chunk's K and V behind for the cache write (a forward whose
        cache update will not be applied has no use for them, and they cost ~3 us).
        ``global_sink_tokens``: leading tokens of the stream that stay in the cache for good (multi-shot mode).
        ``rope_fn(frames, start_frame) -> (cos, sin)``: needed when ``use_relative_rope`` is set; the positions
        then count frames of the attended window instead of frames of the stream.
        ``residual`` [B, L, C] (with ``gate`` [B*F, C], ``gate_rows`` tokens per gate row) turns the result into
        ``residual + out * gate``, folded into the output projection."""
        b, s = x.shape[:2]
        n, d = self.num_heads, self.head_dim
        # The chunk's K (after norm and RoPE) and V are what the cache quantizes when the chunk is written, after
        # the forward; their producers leave the tensor maxima in two sinks that belong to this layer's cache, so
        # that quantization needs no pass of its own to find them.
        fused_path = b == 1 and d == 128 and not self.use_relative_rope and self.norm_q.eps == self.norm_k.eps
        k_amax = v_amax = None
        if fused_path and collect_kv_amax and isinstance(kv_cache, dict):
            sinks = kv_cache.get("_amax_sinks")
            if sinks is None:
                sinks = kv_cache["_amax_sinks"] = (_native.PrivateAmaxSink(x.device), _native.PrivateAmaxSink(x.device))
            k_amax, v_amax = sinks[0].ticket(), sinks[1].ticket()
        (q, k, v), v_amax_written = _project_shared(x, [self.q, self.k, self.v], amax=input_amax,
                                                    amax_outs=[None, None, v_amax])
        v = v.view(b, s, n, d)
        if self.use_relative_rope:
            if rope_fn is None:
                raise ValueError("use_relative_rope needs rope_fn")
            k = self.norm_k(k).view(b, s, n, d)
            if keys_only:
                return None, kvc.kv_cache_update_only(k, v, kv_cache, current_start, sink_tokens, max_attention_size,
                                                      global_sink_tokens)
            q = self.norm_q(q).view(b, s, n, d)
            out_amax = None
            out, update = kvc.kv_cache_attention_relative(q, k, v, kv_cache, current_start, sink_tokens, rope_fn,
                                                          max_attention_size=max_attention_size,
                                                          global_sink_tokens=global_sink_tokens)
            return _project_out(self.o, out.flatten(2), out_amax, residual, gate, gate_rows), update
        if b == 1 and d == 128:
            # RMSNorm -> RoPE (-> K smoothing) of the reference in one pass over q and k
            if self.norm_q.eps == self.norm_k.eps:
                roped_q, roped_k, smooth_k = _native.qk_norm_rope_pair(
                    q[0], k[0], self.norm_q.weight.data, self.norm_k.weight.data, self.norm_q.eps, cos, sin, n,
                    k_amax_out=k_amax)
            else:
                roped_q = _native.qk_norm_rope(q[0], self.norm_q.weight.data, self.norm_q.eps, cos, sin, n)
                roped_k, smooth_k = _native.qk_norm_rope(k[0], self.norm_k.weight.data, self.norm_k.eps, cos, sin, n,
                                                         smooth=True)
            roped_q, roped_k, smooth_k = roped_q.unsqueeze(0), roped_k.unsqueeze(0), smooth_k.unsqueeze(0)
        else:
            q = self.norm_q(q).view(b, s, n, d)
            k = self.norm_k(k).view(b, s, n, d)
            roped_q = rope_apply(q[0], cos, sin).unsqueeze(0)
            roped_k = rope_apply(k[0], cos, sin).unsqueeze(0)
            smooth_k = None
        if keys_only:
            out, update = None, kvc.kv_cache_update_only(roped_k, v, kv_cache, current_start, sink_tokens,
                                                         max_attention_size, global_sink_tokens)
        else:
            out_amax = _native.amax_ticket(x.device) if isinstance(self.o, FourOverSixLinear) else None
            out, update = kvc.kv_cache_attention(roped_q, roped_k, v, kv_cache, current_start, sink_tokens,
                                                 max_attention_size=max_attention_size, smoothed_key=smooth_k,
                                                 amax_out=out_amax, global_sink_tokens=global_sink_tokens)
        if update[2] is not None:
            update[2]["new_k_amax"] = k_amax
            update[2]["new_v_amax"] = v_amax if v_amax_written else None
        if keys_only:
            return None, update
        return _project_out(self.o, out.flatten(2), out_amax, residual, gate, gate_rows), update


class CrossAttention(nn.Module):
    def __init__(self, dim: int, num_heads: int, eps: float = 1e-6) -> None:
        super().__init__()
        self.dim, self.num_heads, self.head_dim = dim, num_heads, dim // num_heads
        self.q, self.k, self.v, self.o = (nn.Linear(dim, dim) for _ in range(4))
        self.norm_q, self.norm_k = WanRMSNorm(dim, eps), WanRMSNorm(dim, eps)

    def forward(self, x, context, crossattn_cache: dict | None = None, *, residual=None, input_amax=None):
        """``residual`` [B, L, C] turns the result into ``residual + out`` (folded into the output projection).
        ``input_amax``: the amax ticket the producer of ``x`` was given, if any.
        ``crossattn_cache`` ({"is_init": bool, "k": ..., "v": ...}, the reference's interface,
        wan_5b/modules/causal_model.py:199-206) keeps the projected K / V of a prompt's text context between
        calls; the reference has the argument but recomputes on every call (:229-235), which gives the same
        tensors.  Without a cache K / V are recomputed here too."""
        b, n, d = x.shape[0], self.num_heads, self.head_dim
        q = self.norm_q(_project_shared(x, [self.q], amax=input_amax)[0][0]).view(b, -1, n, d)
        if crossattn_cache is not None and crossattn_cache.get("is_init"):
            k, v = crossattn_cache["k"], crossattn_cache["v"]
        else:
            k, v = _project_shared(context, [self.k, self.v])[0]
            k = self.norm_k(k).view(b, -1, n, d)
            v = v.view(b, -1, n, d)
            if crossattn_cache is not None:
                crossattn_cache.update(is_init=True, k=k, v=v)
        out_amax = _native.amax_ticket(x.device) if isinstance(self.o, FourOverSixLinear) else None
        out = _native.attention_bf16(q[0].contiguous(), k[0].contiguous(), v[0].contiguous(), d ** -0.5,
                                     amax_out=out_amax)
        return _project_out(self.o, out.unsqueeze(0).flatten(2), out_amax, residual, None, 0)


class DiTBlock(nn.Module):
    # normalize and quantize in one launch where a quantized layer reads the result (the same bytes either way)
    fuse_norm_quantize = True

    def __init__(self, dim: int, ffn_dim: int, num_heads: int, eps: float = 1e-6) -> None:
        super().__init__()
        self.dim, self.eps = dim, eps
        self.norm1 = WanLayerNorm(dim, eps)
        self.self_attn = CausalSelfAttention(dim, num_heads, eps)
        self.norm3 = WanLayerNorm(dim, eps, elementwise_affine=True)
        self.cross_attn = CrossAttention(dim, num_heads, eps)
        self.norm2 = WanLayerNorm(dim, eps)
        self.ffn = nn.Sequential(nn.Linear(dim, ffn_dim), nn.GELU(approximate="tanh"), nn.Linear(ffn_dim, dim))
        self.modulation = nn.Parameter(torch.randn(1, 6, dim) / dim ** 0.5)

    def _feed_forward(self, y, y_amax, residual, gate, gate_rows: int) -> torch.Tensor:
        """``residual + ffn(y) * gate`` with ffn = Linear -> GELU(tanh) -> Linear.  With quantized layers the
        GELU runs in the first GEMM's epilogue (which also yields the amax of its result) and the gated
        residual in the second's."""
        up, act, down = self.ffn
        if isinstance(up, FourOverSixLinear) and getattr(act, "approximate", None) == "tanh":
            h_amax = _native.amax_ticket(y.device) if isinstance(down, FourOverSixLinear) else None
            yq = y.operand if isinstance(y, QuantizedActivation) else up.quantize_input(
                y.reshape(-1, y.shape[-1]), amax=y_amax)
            h = up.forward_quantized(yq, activation="gelu_tanh", amax_out=h_amax).reshape(*y.shape[:-1], -1)
        else:
            h, h_amax = act(up(y)), None
        return _project_out(down, h, h_amax, residual, gate, gate_rows)

    def forward(self, x, e, cos, sin, context, kv_cache, current_start, sink_tokens, max_attention_size=None,
                crossattn_cache=None, global_sink_tokens=0, rope_fn=None, collect_kv_amax=True, modulated=None,
                keys_only=False):
        """x [1, L, C]; e [1, F, 6, C]; returns (x, (current_end, local_end_index, cache_update_info)).
        The tensor amax that each activation quantization needs is produced by the kernel that writes the
        activation wherever that kernel is one of this package's.  ``modulated`` is ``self.modulation.unsqueeze(1)
        + e`` when the caller has already formed it (the model does so for all its blocks in one operation).
        ``keys_only``: the block's output has no reader (last block of a pass that only rewrites the cache):
        the block stops behind the producers of the chunk's K and V and returns ``(None, update)``."""
        num_frames, frame_seqlen = e.shape[1], x.shape[1] // e.shape[1]
        e = (self.modulation.unsqueeze(1) + e if modulated is None else modulated).chunk(6, dim=2)
        gates = [g.reshape(-1, g.shape[-1]) for g in (e[2], e[5])]  # [B*F, C] views, one row per frame
        sa = self.self_attn
        y, y_amax = self._normalized_for([sa.q, sa.k, sa.v], x, scale=e[1], shift=e[0], frame_seqlen=frame_seqlen)
        x, update = self.self_attn(y, cos, sin, kv_cache, current_start, sink_tokens, max_attention_size,
                                   input_amax=y_amax, residual=x, gate=gates[0], gate_rows=frame_seqlen,
                                   global_sink_tokens=global_sink_tokens, rope_fn=rope_fn,
                                   collect_kv_amax=collect_kv_amax, keys_only=keys_only)
        if keys_only:
            return None, update
        y, y_amax = self._normalized_for([self.cross_attn.q], x, norm=self.norm3)
        x = self.cross_attn(y, context, crossattn_cache, residual=x, input_amax=y_amax)
        up = self.ffn[0]
        fused_ffn = isinstance(up, FourOverSixLinear) and getattr(self.ffn[1], "approximate", None) == "tanh"
        y, y_amax = self._normalized_for([up], x, scale=e[4], shift=e[3], frame_seqlen=frame_seqlen,
                                         operand_ok=fused_ffn)
        x = self._feed_forward(y, y_amax, x, gates[1], frame_seqlen)
        return x, update

    def _normalized_for(self, layers, x, *, scale=None, shift=None, frame_seqlen=0, norm=None, operand_ok=True):
        """The adaLN modulation of ``x`` (``scale`` / ``shift`` given) or ``norm(x)`` as input of ``layers``:
        ``(activation, amax ticket)``.  When the layers are quantized with one activation config, the activation
        is produced directly as their NVFP4 operand (a :class:`QuantizedActivation`, no ticket) where the
        one-launch kernel takes the shapes; else as a bf16 tensor whose maximum the ticket carries."""
        first = layers[0]
        quantized = isinstance(first, FourOverSixLinear)
        if (quantized and operand_ok and self.fuse_norm_quantize and all(isinstance(m, FourOverSixLinear)
                and m.config.get_activation_config() == first.config.get_activation_config() for m in layers)):
            if norm is None:
                xq = first.quantize_normalized_input(x, scale=scale, shift=shift, frame_seqlen=frame_seqlen,
                                                     eps=self.eps)
            else:
                xq = first.quantize_normalized_input(x, weight=norm.weight, bias=norm.bias, eps=norm.eps)
            if xq is not None:
                return QuantizedActivation(xq, x.shape), None
        ticket = _native.amax_ticket(x.device) if quantized else None
        if norm is None:
            return adaln_modulate(x, scale, shift, frame_seqlen, eps=self.eps, amax_out=ticket), ticket
        return norm(x, amax_out=ticket), ticket


class CausalHead(nn.Module):
    def __init__(self, dim: int, out_dim: int, patch_size, eps: float = 1e-6) -> None:
        super().__init__()
        self.norm = WanLayerNorm(dim, eps)
        self.head = nn.Linear(dim, math.prod(patch_size) * out_dim)
        self.modulation = nn.Parameter(torch.randn(1, 2, dim) / dim ** 0.5)

    def forward(self, x, e):
        num_frames, frame_seqlen = e.shape[1], x.shape[1] // e.shape[1]
        e = (self.modulation.unsqueeze(1) + e).chunk(2, dim=2)
        if x.is_cuda and x.dtype == torch.bfloat16 and x.is_contiguous() and e[0].dtype == torch.bfloat16:
            # norm(x) * (1 + e[1]) + e[0] is the adaLN modulation of the blocks, with the same bf16 roundings
            y = adaln_modulate(x, e[1], e[0], frame_seqlen, eps=self.norm.eps)
            return self.head(y.unflatten(1, (num_frames, frame_seqlen)))
        return self.head(self.norm(x).unflatten(1, (num_frames, frame_seqlen)) * (1 + e[1]) + e[0])


def sinusoidal_embedding_1d(dim: int, position: torch.Tensor) -> torch.Tensor:
    half = dim // 2
    position = position.to(torch.float64)
    sinusoid = torch.outer(position, torch.pow(10000, -torch.arange(half, device=position.device).to(position).div(half)))
    return torch.cat([torch.cos(sinusoid), torch.sin(sinusoid)], dim=1)


class CausalDiT(nn.Module):
    def __init__(self, cfg: DiTConfig) -> None:
        super().__init__()
        self.cfg = cfg
        self.patch_embedding = nn.Conv3d(cfg.in_dim, cfg.dim, kernel_size=cfg.patch_size, stride=cfg.patch_size)
        self.text_embedding = nn.Sequential(nn.Linear(cfg.text_dim, cfg.dim), nn.GELU(approximate="tanh"),
                                            nn.Linear(cfg.dim, cfg.dim))
        self.time_embedding = nn.Sequential(nn.Linear(cfg.freq_dim, cfg.dim), nn.SiLU(), nn.Linear(cfg.dim, cfg.dim))
        self.time_projection = nn.Sequential(nn.SiLU(), nn.Linear(cfg.dim, cfg.dim * 6))
        self.blocks = nn.ModuleList([DiTBlock(cfg.dim, cfg.ffn_dim, cfg.num_heads, cfg.eps) for _ in range(cfg.num_layers)])
        self.head = CausalHead(cfg.dim, cfg.out_dim, cfg.patch_size, cfg.eps)
        self.rope_angles = build_rope_angles(cfg.dim // cfg.num_heads)
        self.global_sink_size = cfg.global_sink_size  # frames; the generator overrides it like the reference pipeline
        self.rope_temporal_offset = 0.0               # frames added to every temporal position (causal_model.py:1097)
        self.kv_quant_config = None
        self._rope_cache: dict = {}
        self._time_cache: dict = {}
        self.init_weights()

    def init_weights(self) -> None:
        """Xavier for linears, N(0, 0.02) for the text / time MLPs, zero output head
        (wan_5b/modules/causal_model.py:1860-1882), with a small non-zero head so that random-init
        runs produce non-trivial outputs."""
        for m in self.modules():
            if isinstance(m, nn.Linear):
                nn.init.xavier_uniform_(m.weight)
                if m.bias is not None:
                    nn.init.zeros_(m.bias)
        nn.init.xavier_uniform_(self.patch_embedding.weight.flatten(1))
        for seq in (self.text_embedding, self.time_embedding):
            for m in seq:
                if isinstance(m, nn.Linear):
                    nn.init.normal_(m.weight, std=0.02)
        nn.init.normal_(self.head.head.weight, std=0.02)

    def _rope(self, f: int, h: int, w: int, start_frame: int, device, temporal_offset: float = 0.0):
        key = (f, h, w, start_frame, str(device), float(temporal_offset))
        if key not in self._rope_cache:
            if len(self._rope_cache) > 64:
                self._rope_cache.clear()
            self._rope_cache[key] = rope_cos_sin(self.rope_angles, f, h, w, start_frame, device,
                                                 temporal_offset=float(temporal_offset))
        return self._rope_cache[key]

    def patch_embed(self, x: torch.Tensor):
        """x [C_in, F, H, W] -> tokens [1, f*h*w, dim] and the grid (f, h, w).  The patch embedding is a Conv3d whose
        kernel equals its stride (wan_5b/modules/causal_model.py:1052-1053, 1535): every output token is a linear map
        of one patch, so it runs as one matrix product over the flattened patches (c, pt, ph, pw), the order of the
        convolution weight, instead of a convolution."""
        pt, ph, pw = self.cfg.patch_size
        c, fr, hh, ww = x.shape
        f, h, w = fr // pt, hh // ph, ww // pw
        patches = x[:, :f * pt, :h * ph, :w * pw].reshape(c, f, pt, h, ph, w, pw).permute(1, 3, 5, 0, 2, 4, 6)
        patches = patches.reshape(f * h * w, c * pt * ph * pw)
        weight = self.patch_embedding.weight.reshape(self.patch_embedding.weight.shape[0], -1)
        return torch.nn.functional.linear(patches, weight, self.patch_embedding.bias).unsqueeze(0), (f, h, w)

    def unpatchify(self, x: torch.Tensor, grid) -> torch.Tensor:
        c = self.cfg.out_dim
        f, h, w = grid
        u = x[: f * h * w].view(f, h, w, *self.cfg.patch_size, c)
        u = torch.einsum("fhwpqrc->cfphqwr", u)
        return u.reshape(c, *[i * j for i, j in zip(grid, self.cfg.patch_size)])

    def _stacked_modulation(self) -> torch.Tensor:
        """The blocks' modulation parameters as one [blocks, 1, 6, C] tensor, rebuilt when a parameter has been
        replaced or written (inference keeps it)."""
        key = tuple((b.modulation.data_ptr(), b.modulation._version) for b in self.blocks)
        cached = getattr(self, "_modulation_stack", None)
        if cached is None or cached[0] != key:
            cached = (key, torch.stack([b.modulation.detach() for b in self.blocks]))
            self._modulation_stack = cached
        return cached[1]

    @torch.no_grad()
    def _time_conditioning(self, t: torch.Tensor, like: torch.Tensor, timestep_key):
        """(e, e0, modulated) of the timesteps t [1, F]: the time embedding, its projection to the six modulation
        vectors per frame (wan_5b/modules/causal_model.py:1554-1564) and modulation + e0 of every block in one
        operation (the same additions and roundings as block by block, :862-863).  A sampler evaluates the model at
        a handful of timestep values over and over; with ``timestep_key`` (a hashable that names the values of t,
        for instance ``(250.0, 3)``) the three tensors are computed once per value and kept until a parameter they
        depend on is replaced or written."""
        cfg = self.cfg
        params = [p for seq in (self.time_embedding, self.time_projection) for p in seq.parameters()] + \
                 [b.modulation for b in self.blocks]
        version = tuple((p.data_ptr(), p._version) for p in params)
        if self._time_cache.get("version") != version:
            self._time_cache = {"version": version}
        key = None if timestep_key is None else (timestep_key, tuple(t.shape), like.dtype, str(like.device))
        if key is not None and key in self._time_cache:
            return self._time_cache[key]
        e = self.time_embedding(sinusoidal_embedding_1d(cfg.freq_dim, t.flatten()).unflatten(0, t.shape).type_as(like))
        e0 = self.time_projection(e).unflatten(2, (6, cfg.dim))
        modulated = self._stacked_modulation().unsqueeze(2) + e0.unsqueeze(0)   # [blocks, 1, F, 6, C]
        if key is not None:
            if len(self._time_cache) > 32:
                self._time_cache = {"version": version}
            self._time_cache[key] = (e, e0, modulated)
        return e, e0, modulated

    @torch.no_grad()
    def forward(self, x: torch.Tensor, t: torch.Tensor, context: torch.Tensor, kv_cache: list[dict],
                current_start: int, apply_cache_updates: bool = True,
                crossattn_cache: list[dict] | None = None, timestep_key=None, cache_only: bool = False):
        """x [C_in, F, H, W] latents of one chunk, t [1, F] timesteps, context [L, text_dim];
        returns the flow prediction [C_out, F, H, W] and updates the KV cache like the reference
        (all layers' updates applied after the last block).  ``crossattn_cache``: one dictionary per layer
        holding the projected text K / V of the current prompt (filled on first use).  ``timestep_key``: a
        hashable naming the values of ``t``; the time conditioning is then computed once per key.
        ``cache_only``: the caller runs the pass for its cache update and does not read the prediction (the
        clean-context pass of the chunk loop, pipeline/causal_diffusion_inference.py:639-647).  The last block then
        stops behind its K / V producers and the head is left out - nothing that reaches the cache depends on them -
        and the return value is None."""
        cfg = self.cfg
        x, (f, h, w) = self.patch_embed(x)
        frame_seqlen = h * w
        e, e0, modulated = self._time_conditioning(t, x, timestep_key)
        if crossattn_cache is not None and all(c.get("is_init") for c in crossattn_cache):
            ctx = None  # every layer holds the projected K / V of this prompt: the text embedding has no reader
        else:
            ctx = torch.cat([context, context.new_zeros(cfg.text_len - context.size(0), context.size(1))]).unsqueeze(0)
            ctx = self.text_embedding(ctx)
        # the multi-shot phase offset applies to absolute positions only (causal_model.py:478-486, 1588)
        cos, sin = self._rope(f, h, w, current_start // frame_seqlen, x.device, self.rope_temporal_offset)
        sink_tokens = cfg.sink_size * frame_seqlen
        max_attn = cfg.local_attn_size * frame_seqlen
        updates = []
        for i, block in enumerate(self.blocks):
            x, upd = block(x, e0, cos, sin, ctx, kv_cache[i], current_start, sink_tokens, max_attn,
                           None if crossattn_cache is None else crossattn_cache[i],
                           global_sink_tokens=self.global_sink_size * frame_seqlen,
                           rope_fn=lambda frames, first: self._rope(frames, h, w, first, x.device),
                           collect_kv_amax=apply_cache_updates, modulated=modulated[i],
                           keys_only=cache_only and i == len(self.blocks) - 1)
            updates.append(upd)
        if apply_cache_updates:
            for i, (cur_end, loc_end, info) in enumerate(updates):
                kvc.apply_cache_update(kv_cache[i], cur_end, loc_end, info, self.kv_quant_config)
        if cache_only:
            return None
        x = self.head(x, e.unsqueeze(2))
        return self.unpatchify(x[0].flatten(0, 1) if x.dim() == 4 else x[0], (f, h, w))
