"""FourOverSixLinear: W4A4 replacement for nn.Linear, inference forward
(mirror of fouroversix/src/fouroversix/model/modules/linear.py:153-355; the autograd backward of
the reference is a training feature and is not provided)."""
from __future__ import annotations

from typing import Any

import torch
import torch.nn as nn

from ...matmul import fp4_matmul
from ...quantize import QuantizationConfig, QuantizedTensor, quantize_to_fp4
from ..config import ModuleQuantizationConfig
from ..quantize import QuantizedModule


@QuantizedModule.register(nn.Linear)
class FourOverSixLinear(nn.Linear):
    """Activations are quantized to NVFP4 on the fly, the weight is held pre-quantized in the
    buffers ``quantized_weight_{values,scale_factors,amax,metadata}`` (same names, dtypes and
    shapes as the reference, so packed NVFP4 checkpoints load with ``load_state_dict``)."""

    _INT32_MAX = 2_147_483_647

    def __init__(self, module: nn.Linear, config: ModuleQuantizationConfig) -> None:
        super().__init__(module.in_features, module.out_features, module.bias is not None,
                         module.weight.device, module.weight.dtype)
        self.weight = module.weight
        self.bias = module.bias
        self.config = config
        if not self.config.keep_master_weights:
            dev = module.weight.device
            self.register_buffer("quantized_weight_values",
                                 torch.zeros(self.out_features, self.in_features // 2, dtype=torch.uint8, device=dev))
            self.register_buffer("quantized_weight_scale_factors",
                                 torch.zeros(self.out_features * self.in_features // config.dtype.block_size(),
                                             dtype=config.dtype.scale_dtype(), device=dev))
            self.register_buffer("quantized_weight_amax", torch.zeros(1, dtype=torch.float32, device=dev))
            self.register_buffer("quantized_weight_metadata", torch.zeros(4, dtype=torch.int32, device=dev))

    # ------------------------------------------------------------------ weight materialisation
    @property
    def parameters_to_quantize(self) -> tuple[str, ...]:
        return ("weight",)

    def get_element_size(self, parameter_name: str) -> float:
        return {"quantized_weight_values": 0.5, "weight": 9 / 16}.get(
            parameter_name, getattr(self, parameter_name).element_size())

    def get_quantized_parameters(self, parameter_name: str, parameter: torch.Tensor,
                                 include_transposed: bool = False) -> dict[str, Any]:
        if parameter_name != "weight":
            raise ValueError(f"Unsupported high-precision parameter: {parameter_name}")
        if include_transposed:
            raise ValueError("transposed weight caches are a training feature and are not supported")
        cfg = QuantizationConfig(backend=self.config.quantize_backend, block_scale_2d=self.config.weight_scale_2d,
                                 dtype=self.config.dtype, scale_rule=self.config.weight_scale_rule)
        return self._serialize_quantized_weight("quantized_weight", quantize_to_fp4(parameter, cfg))

    @staticmethod
    def _serialize_quantized_weight(prefix: str, q: QuantizedTensor) -> dict[str, torch.Tensor]:
        return {
            f"{prefix}_values": q.values,
            f"{prefix}_scale_factors": q.scale_factors,
            f"{prefix}_amax": q.amax,
            f"{prefix}_metadata": torch.tensor([*q.original_shape, *q.padded_shape], dtype=torch.int32),
        }

    def _build_quantized_weight(self, prefix: str) -> QuantizedTensor | None:
        parts = [getattr(self, f"{prefix}_{n}", None) for n in ("values", "scale_factors", "amax", "metadata")]
        if any(p is None for p in parts):
            return None
        values, scale_factors, amax, metadata = parts
        meta = metadata.tolist()
        return QuantizedTensor(values.data, scale_factors.data, amax.data, self.config.dtype, tuple(meta[:2]),
                               self.config.weight_scale_rule, tuple(meta[2:]))

    def quantized_weight(self) -> QuantizedTensor | torch.Tensor:
        if not hasattr(self, "_quantized_weight"):
            if self.config.keep_master_weights:
                return self.weight
            self._quantized_weight = self._build_quantized_weight("quantized_weight")
        return self._quantized_weight

    def quantized_weight_transposed(self) -> None:
        return None

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys,
                              error_msgs) -> None:
        """State dicts written by the reference's module load as they are: after quantization the reference holds
        the tensor amax as a 0-dim tensor (it registers a [1] buffer, linear.py:203-206, and replaces it with
        ``QuantizedTensor.amax``), and values / scale factors in the padded shape (rows to 128, columns to 64)
        where the freshly swapped module registered the unpadded one.  Buffers are brought to the incoming
        shapes before the regular copy, so ``strict=True`` holds for such checkpoints."""
        amax_key = prefix + "quantized_weight_amax"
        own_amax = getattr(self, "quantized_weight_amax", None)
        incoming = state_dict.get(amax_key)
        if isinstance(incoming, torch.Tensor) and isinstance(own_amax, torch.Tensor) and incoming.numel() == 1 \
                and incoming.shape != own_amax.shape:
            state_dict[amax_key] = incoming.reshape(own_amax.shape)
        for name in ("quantized_weight_values", "quantized_weight_scale_factors"):
            own, incoming = getattr(self, name, None), state_dict.get(prefix + name)
            if isinstance(own, torch.Tensor) and isinstance(incoming, torch.Tensor) and own.shape != incoming.shape \
                    and own.dtype == incoming.dtype and incoming.numel() >= own.numel():
                setattr(self, name, torch.zeros(incoming.shape, dtype=own.dtype, device=own.device))
        for attr in ("_quantized_weight", "_quantized_weight_transposed"):
            if hasattr(self, attr):
                delattr(self, attr)
        super()._load_from_state_dict(state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys,
                                      error_msgs)

    # ------------------------------------------------------------------ forward
    def forward(self, input: torch.Tensor) -> torch.Tensor:
        if input.requires_grad and torch.is_grad_enabled():
            raise NotImplementedError("FourOverSixLinear on gfx950 is inference-only; run under torch.no_grad()")
        x2d = input.reshape(-1, input.shape[-1])
        if x2d.shape[0] * x2d.shape[1] > self._INT32_MAX:  # same guard as the reference: two halves
            mid = x2d.shape[0] // 2
            out = torch.cat([self._forward_2d(x2d[:mid]), self._forward_2d(x2d[mid:])], dim=0)
        else:
            out = self._forward_2d(x2d)
        return out.reshape(*input.shape[:-1], out.shape[-1])

    def _forward_2d(self, x2d: torch.Tensor) -> torch.Tensor:
        return self.forward_quantized(self.quantize_input(x2d))

    def quantize_input(self, x2d: torch.Tensor, amax=None) -> QuantizedTensor:
        """The activation operand exactly as ``forward`` would build it from a 2-D input.  ``amax`` is
        the amax ticket of the kernel that produced ``x2d``, if it was given one."""
        return quantize_to_fp4(x2d, self.config.get_activation_config(), amax=amax)

    def quantize_normalized_input(self, x: torch.Tensor, *, scale=None, shift=None, frame_seqlen: int = 0,
                                  weight=None, bias=None, eps: float = 1e-6) -> QuantizedTensor | None:
        """``quantize_input`` of the adaLN modulation of ``x`` [B, L, C] (``scale`` / ``shift`` [B, F, 1, C] given:
        ``LayerNorm(x) * (1 + scale) + shift``) or of its LayerNorm with optional ``weight`` / ``bias``, flattened
        to 2-D, as one launch that never writes the normalized tensor (an extension; the reference runs the
        normalization and the layer's quantization separately, wan_5b/modules/causal_model.py:869-878, 892-906,
        909-918).  The bytes are those of the separate operations.  ``None`` when that launch does not take the
        input or the activation config, and the caller runs the separate operations."""
        from .... import _native
        from ...quantize.frontend import _unsupported

        config = self.config.get_activation_config()
        if not (x.is_cuda and x.dtype == torch.bfloat16 and x.ndim == 3 and x.is_contiguous()) or \
                _unsupported(x[0], config) is not None:
            return None
        rule = config.scale_rule.value
        if scale is not None:
            if scale.dtype != torch.bfloat16 or shift.dtype != torch.bfloat16:
                return None
            out = _native.adaln_quantize(x, scale, shift, frame_seqlen, rule, eps=eps)
        else:
            if any(t is not None and t.dtype != torch.bfloat16 for t in (weight, bias)):
                return None
            out = _native.layer_norm_quantize(x, weight, bias, rule, eps=eps)
        if out is None:
            return None
        shape = (x.shape[0] * x.shape[1], x.shape[2])
        return QuantizedTensor(*out, config.dtype, shape, config.scale_rule, _native.padded_shape(shape))

    @staticmethod
    def forward_quantized_together(layers, xq: QuantizedTensor, amax_outs=None) -> list[torch.Tensor]:
        """``[m.forward_quantized(xq) for m in layers]`` as one GEMM launch when the layers have the same shape
        (the q / k / v projections of an attention layer): the products are computed exactly as they would be
        alone, only the cost of two launches and of two half-empty rounds of workgroups is saved.  ``amax_outs``:
        one amax ticket or ``None`` per layer."""
        from .... import _native

        amax_outs = amax_outs or [None] * len(layers)
        weights = [m.quantized_weight() for m in layers]
        same = (1 < len(layers) <= 4 and all(isinstance(w, QuantizedTensor) for w in weights)
                and all(w.values.shape == weights[0].values.shape and w.original_shape == weights[0].original_shape
                        and w.dtype == xq.dtype for w in weights)
                and weights[0].original_shape[1] == xq.original_shape[1]
                and all(m.bias is None or m.bias.dtype == torch.bfloat16 for m in layers)
                # two tickets of one sink buffer cannot be served by one launch: the later epoch would hide the earlier
                and len({t.parts.data_ptr() for t in amax_outs if t is not None}) == sum(t is not None for t in amax_outs))
        if not same:
            return [m.forward_quantized(xq, amax_out=t) for m, t in zip(layers, amax_outs)]
        denom = lambda q: float(q.scale_rule.max_allowed_e2m1_value() * q.scale_rule.max_allowed_e4m3_value())
        products = [dict(values=w.values, scales=w.scale_factors, amax=w.amax, denom=denom(w), bias=m.bias, amax_out=t)
                    for m, w, t in zip(layers, weights, amax_outs)]
        return _native.gemm_grouped(xq.values, xq.scale_factors, xq.amax, denom(xq), xq.original_shape[0],
                                    weights[0].original_shape[0], products)

    def forward_quantized(self, xq: QuantizedTensor, activation: str | None = None, *,
                          residual: torch.Tensor | None = None, gate: torch.Tensor | None = None,
                          gate_rows: int = 0, amax_out=None) -> torch.Tensor:
        """``forward`` for an input already quantized with :meth:`quantize_input`.  Several layers that read
        the same tensor with the same activation config (the q / k / v projections) share one quantized
        operand this way; each would otherwise compute the identical bytes again.  The keyword arguments are
        the epilogue extensions of :func:`fp4_matmul` (activation, gated residual, amax of the result).
        Returns [M, out_features]."""
        weight = self.quantized_weight()
        if not isinstance(weight, QuantizedTensor):
            weight = quantize_to_fp4(weight.data, self.config.get_weight_config())
        return fp4_matmul(xq, weight, backend=self.config.matmul_backend, out_dtype=self.config.output_dtype,
                          bias=self.bias, activation=activation, residual=residual, gate=gate, gate_rows=gate_rows,
                          amax_out=amax_out)
