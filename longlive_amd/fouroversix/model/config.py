"""Module / model quantization configuration
(mirror of fouroversix/src/fouroversix/model/config.py:17-194)."""
from __future__ import annotations

import hashlib
import json
from dataclasses import dataclass, field
from typing import Any

from ..quantize import QuantizationConfig
from ..utils import DataType, MatmulBackend, QuantizeBackend, RoundStyle, ScaleRule


@dataclass
class ModuleQuantizationConfig:
    """Per-module options.  ``scale_rule`` is the fallback for the activation / weight / gradient
    rules.  Gradient options are kept for configuration compatibility (training is not part of
    this inference path)."""

    activation_scale_rule: ScaleRule | None = None
    dtype: DataType = DataType.nvfp4
    gradient_round_style: RoundStyle = RoundStyle.stochastic
    gradient_scale_rule: ScaleRule | None = None
    keep_master_weights: bool = False
    matmul_backend: MatmulBackend | None = None
    output_dtype: DataType = DataType.bfloat16
    quantize_backend: QuantizeBackend | None = None
    scale_rule: ScaleRule = ScaleRule.mse
    weight_scale_2d: bool = False
    weight_scale_rule: ScaleRule | None = None
    activation_chunk_size: int | None = None

    def __post_init__(self) -> None:
        def conv(value, enum):
            return enum(value) if isinstance(value, str) else value

        self.activation_scale_rule = conv(self.activation_scale_rule, ScaleRule)
        self.dtype = conv(self.dtype, DataType)
        self.gradient_round_style = conv(self.gradient_round_style, RoundStyle)
        self.gradient_scale_rule = conv(self.gradient_scale_rule, ScaleRule)
        self.matmul_backend = conv(self.matmul_backend, MatmulBackend)
        self.output_dtype = conv(self.output_dtype, DataType)
        self.quantize_backend = conv(self.quantize_backend, QuantizeBackend)
        self.scale_rule = conv(self.scale_rule, ScaleRule)
        self.weight_scale_rule = conv(self.weight_scale_rule, ScaleRule)
        self.activation_scale_rule = self.activation_scale_rule or self.scale_rule
        self.gradient_scale_rule = self.gradient_scale_rule or self.scale_rule
        self.weight_scale_rule = self.weight_scale_rule or self.scale_rule

    def get_activation_config(self, **kwargs: Any) -> QuantizationConfig:
        return QuantizationConfig(backend=self.quantize_backend, dtype=self.dtype,
                                  scale_rule=self.activation_scale_rule, **kwargs)

    def get_gradient_config(self, **kwargs: Any) -> QuantizationConfig:
        return QuantizationConfig(backend=self.quantize_backend, dtype=self.dtype,
                                  round_style=self.gradient_round_style, scale_rule=self.gradient_scale_rule,
                                  **kwargs)

    def get_weight_config(self, **kwargs: Any) -> QuantizationConfig:
        return QuantizationConfig(backend=self.quantize_backend, block_scale_2d=self.weight_scale_2d,
                                  dtype=self.dtype, scale_rule=self.weight_scale_rule, **kwargs)


@dataclass
class ModelQuantizationConfig(ModuleQuantizationConfig):
    """Model-wide options plus per-module overrides and the list of modules left unquantized."""

    module_config_overrides: dict[str, ModuleQuantizationConfig] = field(default_factory=dict)
    modules_to_not_convert: list[str] = field(default_factory=lambda: ["lm_head"])

    def __post_init__(self) -> None:
        super().__post_init__()
        if self.module_config_overrides is not None:
            for name, cfg in self.module_config_overrides.items():
                if isinstance(cfg, dict):
                    self.module_config_overrides[name] = ModuleQuantizationConfig(**cfg)

    def get_module_config(self, module_name: str) -> ModuleQuantizationConfig:
        if self.module_config_overrides is None:
            return self
        return self.module_config_overrides.get(module_name, self)

    def __hash__(self) -> str:
        return hashlib.sha256(json.dumps(self.__dict__, sort_keys=True, default=str).encode()).hexdigest()
