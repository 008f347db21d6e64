"""Module-swap registry and quantize_model
(mirror of fouroversix/src/fouroversix/model/quantize.py:13-127)."""
from __future__ import annotations

from typing import TYPE_CHECKING, Any, Callable, ClassVar

import torch.nn as nn

if TYPE_CHECKING:
    from .config import ModelQuantizationConfig


class QuantizedModule:
    """Registry: high-precision module class -> quantized replacement class."""

    _registry: ClassVar[dict[type[nn.Module], type[nn.Module]]] = {}
    _replace_in_model: ClassVar[dict[type[nn.Module], bool]] = {}

    @classmethod
    def is_quantized_module_type(cls, module_type: type[nn.Module]) -> bool:
        return module_type in cls._registry.values()

    @classmethod
    def get_cls(cls, high_precision_cls: type[nn.Module]) -> type[nn.Module] | None:
        return cls._registry.get(high_precision_cls)

    @classmethod
    def should_replace_existing_modules_in_model(cls, module_type: type[nn.Module]) -> bool:
        return cls._replace_in_model.get(module_type, False)

    @classmethod
    def register(
        cls,
        high_precision_cls: type[nn.Module],
        *,
        replace_existing_modules_in_registry: bool = False,
        replace_existing_modules_in_model: bool = True,
    ) -> Callable[[type[nn.Module]], type[nn.Module]]:
        if high_precision_cls in cls._registry and not replace_existing_modules_in_registry:
            raise ValueError(f"High-precision module {high_precision_cls} is already registered.")
        stale = []
        for registered in cls._registry:
            if high_precision_cls is not None and issubclass(high_precision_cls, registered):
                if not replace_existing_modules_in_registry:
                    raise TypeError(f"High-precision module {high_precision_cls} is a subclass of {registered}, "
                                    "which is already registered.")
                stale.append(registered)
        for registered in stale:
            del cls._registry[registered]

        def wrap(quantized_cls: type[nn.Module]) -> type[nn.Module]:
            cls._registry[high_precision_cls] = quantized_cls
            cls._replace_in_model[high_precision_cls] = replace_existing_modules_in_model
            return quantized_cls

        return wrap


def quantize_model(model: nn.Module, config: "ModelQuantizationConfig", **kwargs: Any) -> None:
    """Replace every registered module type (exact type match) outside
    ``config.modules_to_not_convert`` by its quantized counterpart, in place."""
    for name, module in list(model.named_modules()):
        if name == "" or name in config.modules_to_not_convert:
            continue
        quantized_cls = QuantizedModule.get_cls(type(module))
        if quantized_cls is None or not QuantizedModule.should_replace_existing_modules_in_model(type(module)):
            continue
        model.set_submodule(name, quantized_cls(module, config.get_module_config(name), **kwargs))
