"""Packed NVFP4 generator checkpoints (mirror of utils/nvfp4_checkpoint.py:18-169 and of the
FourOverSix branch of scripts/save_merged_nvfp4_generator.py:98-239 / utils/inference_utils.py:186-218).

A checkpoint is a ``torch.save`` dictionary ``{"generator": state_dict, "checkpoint_format":
"longlive_generator_nvfp4", "checkpoint_version": 1, "quantization": {...}, ...}`` whose state dict
holds, for every quantized linear, the buffers ``quantized_weight_{values,scale_factors,amax,metadata}``
instead of ``weight``.  TransformerEngine checkpoints are an NVIDIA-only format and are rejected.
"""
from __future__ import annotations

from collections.abc import Mapping

import torch
from torch import nn

from ..fouroversix import ModelQuantizationConfig
from .quant import quantize_model_with_filter

NVFP4_CHECKPOINT_FORMAT = "longlive_generator_nvfp4"
TE_NVFP4_CHECKPOINT_FORMAT = "longlive_generator_te_nvfp4"
NVFP4_CHECKPOINT_VERSION = 1


def is_nvfp4_state_dict(state_dict: object) -> bool:
    """True when the state dict carries materialized ``quantized_weight_values`` buffers."""
    return isinstance(state_dict, Mapping) and any(str(k).endswith("quantized_weight_values") for k in state_dict)


def is_te_nvfp4_checkpoint(checkpoint: object) -> bool:
    return isinstance(checkpoint, Mapping) and checkpoint.get("checkpoint_format") == TE_NVFP4_CHECKPOINT_FORMAT


def unwrap_generator_state_dict(checkpoint: object, use_ema: bool = False) -> object:
    """The generator state dict inside the usual LongLive checkpoint layouts."""
    if not isinstance(checkpoint, Mapping):
        return checkpoint
    if "generator" in checkpoint or "generator_ema" in checkpoint:
        return checkpoint["generator_ema" if use_ema and "generator_ema" in checkpoint else "generator"]
    return checkpoint.get("model", checkpoint)


def clean_fsdp_state_dict_keys(state_dict: Mapping) -> dict:
    return {str(k).replace("_fsdp_wrapped_module.", ""): v for k, v in state_dict.items()}


def build_model_quantization_config(config=None, keep_master_weights: bool = False) -> ModelQuantizationConfig:
    """``model_quant_*`` attributes of a run config -> ModelQuantizationConfig (defaults as the reference:
    scale rule static_6, activation rule = scale rule)."""
    rule = getattr(config, "model_quant_scale_rule", "static_6")
    cfg = ModelQuantizationConfig(
        scale_rule=rule,
        quantize_backend=getattr(config, "model_quant_backend", None),
        activation_scale_rule=getattr(config, "model_quant_activation_scale_rule", rule),
        weight_scale_rule=getattr(config, "model_quant_weight_scale_rule", None),
        gradient_scale_rule=getattr(config, "model_quant_gradient_scale_rule", None),
    )
    cfg.keep_master_weights = keep_master_weights
    return cfg


def quantize_model_for_fouroversix_nvfp4(model: nn.Module, config=None, *, keep_master_weights: bool = False,
                                         verbose: bool = True):
    """Swap the eligible linears for FourOverSixLinear according to the run config (weights are not
    materialized here; see :func:`drop_fouroversix_master_weights` / ``load_state_dict``)."""
    return quantize_model_with_filter(
        model,
        quant_config=build_model_quantization_config(config, keep_master_weights=keep_master_weights),
        filtered_modules=getattr(config, "model_quant_filtered_modules", None),
        use_default_filtered_modules=getattr(config, "model_quant_use_default_filtered_modules", True),
        cast_model_to_bf16=True, materialize_for_inference=False, use_transformer_engine=False, verbose=verbose)


def drop_fouroversix_master_weights(model: nn.Module) -> list[str]:
    """Remove the high-precision ``weight`` of every quantized module (before loading packed buffers)."""
    dropped = []
    for name, module in model.named_modules():
        params = getattr(module, "parameters_to_quantize", None)
        if params is None:
            continue
        params = params() if callable(params) else params
        any_dropped = False
        for pname in params or ():
            if isinstance(getattr(module, pname, None), nn.Parameter):
                module.register_parameter(pname, None)
                any_dropped = True
            elif getattr(module, pname, None) is not None:
                setattr(module, pname, None)
                any_dropped = True
        if not any_dropped:
            continue
        for cache in ("_quantized_weight", "_quantized_weight_transposed", "_quantized_weights"):
            if hasattr(module, cache):
                delattr(module, cache)
        if hasattr(module, "config") and hasattr(module.config, "keep_master_weights"):
            module.config.keep_master_weights = False
        dropped.append(name)
    return dropped


def cpu_state_dict(module: nn.Module) -> dict[str, torch.Tensor]:
    return {k: v.detach().cpu() for k, v in module.state_dict().items()}


def export_nvfp4_checkpoint(generator: nn.Module, *, scale_rule: str = "static_6", model_name: str | None = None,
                            matched_modules=None, materialized_modules=None, **extra) -> dict:
    """Checkpoint dictionary for a generator whose quantized weights are materialized."""
    state = cpu_state_dict(generator)
    if not is_nvfp4_state_dict(state):
        raise ValueError("the generator holds no materialized NVFP4 weights; quantize it with "
                         "materialize_for_inference=True first")
    return {
        "generator": state,
        "checkpoint_format": NVFP4_CHECKPOINT_FORMAT,
        "checkpoint_version": NVFP4_CHECKPOINT_VERSION,
        "model_name": model_name,
        "quantization": {"format": "nvfp4", "backend": "fouroversix", "materialized": True, "dtype": "bfloat16",
                         "scale_rule": scale_rule},
        "matched_modules": list(matched_modules or []),
        "materialized_modules": list(materialized_modules or []),
        **extra,
    }


def save_nvfp4_checkpoint(path, generator: nn.Module, **kwargs) -> dict:
    checkpoint = export_nvfp4_checkpoint(generator, **kwargs)
    torch.save(checkpoint, path)
    return checkpoint


def load_nvfp4_generator(generator: nn.Module, checkpoint, config=None, *, use_ema: bool = False,
                         verbose: bool = False) -> nn.Module:
    """Bring ``generator`` (a bf16 model with plain linears) to NVFP4 from ``checkpoint`` (a dictionary or a
    path): a packed checkpoint is loaded straight into the quantized buffers; a bf16 checkpoint is loaded
    first and its weights are quantized and materialized afterwards."""
    if not isinstance(checkpoint, Mapping):
        checkpoint = torch.load(checkpoint, map_location="cpu", weights_only=True)
    if is_te_nvfp4_checkpoint(checkpoint):
        raise ValueError("TransformerEngine NVFP4 checkpoints are not supported; export a FourOverSix one")
    fmt = checkpoint.get("checkpoint_format")
    version = checkpoint.get("checkpoint_version", NVFP4_CHECKPOINT_VERSION)
    if fmt == NVFP4_CHECKPOINT_FORMAT and version != NVFP4_CHECKPOINT_VERSION:
        raise ValueError(f"unsupported {NVFP4_CHECKPOINT_FORMAT} version {version}")
    state = clean_fsdp_state_dict_keys(unwrap_generator_state_dict(checkpoint, use_ema=use_ema))
    if is_nvfp4_state_dict(state):
        # The packed weights were produced under one scale rule, and the rule fixes the denominator of their
        # dequantization (6 * 256 for the four-over-six rules, 6 * 448 / 4 * 448 for the static ones): loading them
        # under another rule would silently scale every weight.  The checkpoint records its rule; refuse a mismatch.
        recorded = (checkpoint.get("quantization") or {}).get("scale_rule")
        qcfg = build_model_quantization_config(config)
        wanted = qcfg.weight_scale_rule or qcfg.scale_rule
        wanted = getattr(wanted, "value", wanted)
        if recorded is not None and str(recorded) != str(wanted):
            raise ValueError(f"the checkpoint's weights were quantized with scale rule {recorded!r}, the run "
                             f"configuration asks for {wanted!r} (model_quant_scale_rule / "
                             "model_quant_weight_scale_rule): they must agree")
        generator, _ = quantize_model_for_fouroversix_nvfp4(generator, config, keep_master_weights=False,
                                                            verbose=verbose)
        drop_fouroversix_master_weights(generator)
        generator.load_state_dict(state, strict=True)
    else:
        generator.load_state_dict(state, strict=not use_ema)
        generator, _ = quantize_model_with_filter(
            generator, quant_config=build_model_quantization_config(config),
            filtered_modules=getattr(config, "model_quant_filtered_modules", None),
            use_default_filtered_modules=getattr(config, "model_quant_use_default_filtered_modules", True),
            cast_model_to_bf16=True, materialize_for_inference=True, verbose=verbose)
    return generator
