"""LongLive quantization glue on the gfx950 kernels: filtered module swap, weight materialisation
and the NVFP4 KV-cache helpers (mirror of the NVFP4 parts of utils/quant.py:44-131, 477-689, 731-798)."""
from __future__ import annotations

import re
from copy import deepcopy
from dataclasses import dataclass

import torch
import torch.nn as nn

from .. import _native
from ..fouroversix import (ModelQuantizationConfig, QuantizationConfig, QuantizedTensor, quantize_model,
                           quantize_to_fp4)  # noqa: F401  (quantize_to_fp4 is re-exported like the reference)
from ..fouroversix.quantize.quantized_tensor import from_blocked  # noqa: F401

QUANTIZATION_TYPE = {"weight": "weight", "activation": "activation", "kv": "kv"}

DEFAULT_GENERATOR_FILTERED_MODULES = [
    "text_embedding.0", "text_embedding.2", "patch_embedding", "time_projection.1", "time_embedding.0",
    "time_embedding.2", "head.head", "head.modulation",
    "re:.*norm_k$", "re:.*norm_q$", "re:.*norm1$", "re:.*norm2$", "re:.*norm3$",
]
DEFAULT_FILTERED_MODULES = list(DEFAULT_GENERATOR_FILTERED_MODULES)
FILTER_PROFILE_ALIASES = {"generator": "generator", "student": "generator", "real_score": "real_score",
                          "teacher": "real_score", "fake_score": "fake_score", "critic": "fake_score"}


@dataclass
class LongLiveQuantizationConfig(QuantizationConfig):
    """QuantizationConfig tagged with what it quantizes: "weight", "activation" or "kv"."""

    type: str = "weight"

    def __post_init__(self) -> None:
        super().__post_init__()
        if not isinstance(self.type, str):
            raise TypeError("Quantization type must be a string.")
        if self.type not in QUANTIZATION_TYPE:
            allowed = ", ".join(QUANTIZATION_TYPE.keys())
            raise ValueError(f"Unknown quantization type '{self.type}'. Expected one of: {allowed}.")
        self.type = QUANTIZATION_TYPE[self.type]


def _resolve_modules_to_not_convert(model: nn.Module, filtered_modules: list[str] | None) -> list[str]:
    if not filtered_modules:
        return []
    exact, patterns = set(), []
    for pattern in filtered_modules:
        if not isinstance(pattern, str):
            raise TypeError("Each filtered module pattern must be a string.")
        if pattern.startswith("re:"):
            patterns.append(re.compile(pattern[3:]))
        else:
            exact.add(pattern)
    hits = {name for name, _ in model.named_modules()
            if name and (name in exact or any(p.search(name) for p in patterns))}
    return sorted(hits)


def _get_default_filtered_modules(filter_profile: str | None) -> list[str]:
    if filter_profile is None:
        return list(DEFAULT_FILTERED_MODULES)
    if FILTER_PROFILE_ALIASES.get(filter_profile, filter_profile) in ("generator", "real_score", "fake_score"):
        return list(DEFAULT_GENERATOR_FILTERED_MODULES)
    allowed = ", ".join(sorted(FILTER_PROFILE_ALIASES))
    raise ValueError(f"Unknown filter_profile '{filter_profile}'. Expected one of: {allowed}.")


def _materialize_quantized_weights_for_inference(model: nn.Module, target_device=None,
                                                 cache_transposed_weights: bool = False):
    """Quantize every swapped module's master weight into its ``quantized_weight_*`` buffers and
    drop the master weight.  Returns (module names, master bytes, quantized bytes)."""
    if cache_transposed_weights:
        raise ValueError("cache_transposed_weights is a training feature and is not supported")
    names, master_bytes, quant_bytes = [], 0, 0
    for module_name, module in model.named_modules():
        params = getattr(module, "parameters_to_quantize", None)
        if params is None or not hasattr(module, "get_quantized_parameters"):
            continue
        params = params() if callable(params) else params
        done = False
        for pname in params:
            p = getattr(module, pname, None)
            if p is None:
                continue
            tensor = p.data if isinstance(p, nn.Parameter) else p
            master_bytes += tensor.numel() * tensor.element_size()
            for qname, qt in module.get_quantized_parameters(pname, tensor).items():
                existing = getattr(module, qname, None)
                dst_dtype = existing.dtype if isinstance(existing, torch.Tensor) else qt.dtype
                if target_device is not None:
                    dst_device = torch.device(target_device)
                else:
                    dst_device = existing.device if isinstance(existing, torch.Tensor) else qt.device
                qt = qt.to(device=dst_device, dtype=dst_dtype)
                setattr(module, qname, qt)
                quant_bytes += qt.numel() * qt.element_size()
            if isinstance(getattr(module, pname, None), nn.Parameter):
                module.register_parameter(pname, None)
            else:
                setattr(module, pname, None)
            done = True
        if done:
            for attr in ("_quantized_weight", "_quantized_weight_transposed", "_quantized_weights"):
                if hasattr(module, attr):
                    delattr(module, attr)
            if hasattr(module, "config") and hasattr(module.config, "keep_master_weights"):
                module.config.keep_master_weights = False
            names.append(module_name)
    return names, master_bytes, quant_bytes


def quantize_model_with_filter(model: nn.Module, quant_config=None, filtered_modules=None, filter_profile=None,
                               use_default_filtered_modules: bool = False, cast_model_to_bf16: bool = True,
                               materialize_for_inference: bool = False, materialize_target_device=None,
                               use_transformer_engine: bool = False, verbose: bool = True, **kwargs):
    """Swap nn.Linear modules for FourOverSixLinear except those matching ``filtered_modules``
    (exact names or ``re:`` patterns) and, optionally, the built-in generator profile.  Returns
    ``(model, matched_module_names)``."""
    if use_transformer_engine:
        raise ValueError("Transformer Engine is an NVIDIA-only library; use the fouroversix path")
    te_keys = [k for k in kwargs if k.startswith("te_")]
    for k in te_keys:
        kwargs.pop(k)
    if quant_config is None:
        cfg = ModelQuantizationConfig()
    elif isinstance(quant_config, dict):
        cfg = ModelQuantizationConfig(**quant_config)
    elif isinstance(quant_config, ModelQuantizationConfig):
        cfg = deepcopy(quant_config)
    else:
        raise TypeError("quant_config must be ModelQuantizationConfig, dict, or None.")
    patterns = list(filtered_modules or [])
    if use_default_filtered_modules:
        patterns = _get_default_filtered_modules(filter_profile) + patterns
    matched = _resolve_modules_to_not_convert(model, patterns)
    cfg.modules_to_not_convert = sorted(set(cfg.modules_to_not_convert or []) | set(matched))
    if cast_model_to_bf16:
        model.to(torch.bfloat16)
    quantize_model(model, cfg, **kwargs)
    if materialize_for_inference:
        names, mb, qb = _materialize_quantized_weights_for_inference(model, target_device=materialize_target_device)
        if verbose:
            print(f"[quantize_model_with_filter] materialized_modules={len(names)}, "
                  f"master_weight={mb / 1024 ** 3:.3f} GiB, quantized_weight={qb / 1024 ** 3:.3f} GiB")
    if verbose:
        print(f"[quantize_model_with_filter] profile={filter_profile or 'default'}, matched={len(matched)}, "
              f"total_excluded={len(cfg.modules_to_not_convert)}")
    return model, matched


# --------------------------------------------------------------------------- KV-cache helpers
class SlotPointerTable:
    """Device arrays with the addresses of the values / scale_factors / amax buffers of a list of
    cache slots.  Slots are persistent buffers (copy_quantized_into keeps their addresses), so the
    table is built once per cache list and reused by every kernel launch."""

    def __init__(self, slots: list[QuantizedTensor]) -> None:
        dev = slots[0].values.device
        self.key = tuple((s.values.data_ptr(), s.scale_factors.data_ptr(), s.amax.data_ptr()) for s in slots)
        host = torch.tensor([[k[i] for k in self.key] for i in range(3)], dtype=torch.int64)
        self.table = host.to(dev)
        self.values, self.scales, self.amax = self.table[0], self.table[1], self.table[2]

    def matches(self, slots: list[QuantizedTensor]) -> bool:
        return len(slots) == len(self.key) and all(
            s.values.data_ptr() == k[0] and s.scale_factors.data_ptr() == k[1] and s.amax.data_ptr() == k[2]
            for s, k in zip(slots, self.key))


_tables: dict[int, SlotPointerTable] = {}


def slot_pointer_table(slots: list[QuantizedTensor]) -> SlotPointerTable:
    t = _tables.get(id(slots))
    if t is None or not t.matches(slots):
        t = SlotPointerTable(slots)
        _tables[id(slots)] = t
    return t


def dequantize_kv_cache(kv_list, max_blocks, num_heads, block_token_size, dtype, device):
    """List of ``max_blocks`` NVFP4 slots, each [block_token_size*num_heads, 128] ->
    one tensor [1, max_blocks*block_token_size, num_heads, 128] of ``dtype`` (one launch)."""
    slots = kv_list[:max_blocks]
    first = slots[0]
    table = slot_pointer_table(kv_list) if max_blocks == len(kv_list) else SlotPointerTable(slots)
    return _native.kv_dequantize_blocks(table.values, table.scales, table.amax, max_blocks, num_heads,
                                        block_token_size, dtype, first.scale_rule.max_allowed_e2m1_value(),
                                        first.scale_rule.max_allowed_e4m3_value())


def clone_quantized_tensor(qt: QuantizedTensor) -> QuantizedTensor:
    return QuantizedTensor(values=qt.values.clone(), scale_factors=qt.scale_factors.clone(),
                           amax=qt.amax.clone() if qt.amax is not None else None, dtype=qt.dtype,
                           original_shape=qt.original_shape, scale_rule=qt.scale_rule, padded_shape=qt.padded_shape)


def copy_quantized_into(slot: QuantizedTensor, src: QuantizedTensor) -> None:
    """In-place copy into a pre-allocated slot; the slot's buffers keep their addresses."""
    slot.values.copy_(src.values)
    slot.scale_factors.copy_(src.scale_factors)
    if src.amax is not None and slot.amax is not None:
        slot.amax.copy_(src.amax.reshape(slot.amax.shape))


def k_smooth(k: torch.Tensor) -> torch.Tensor:
    return k - k.mean(dim=-1, keepdim=True)
