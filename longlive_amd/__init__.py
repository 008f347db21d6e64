"""MI355X (gfx950) implementation of LongLive 2.0's NVFP4 inference hot path.

``longlive_amd.fouroversix`` mirrors the reference's ``fouroversix`` package
(quantize_to_fp4, fp4_matmul, QuantizedTensor, FourOverSixLinear, quantize_model);
``longlive_amd.utils`` mirrors the LongLive-level helpers (KV-cache interface, RoPE,
adaLN).  Everything runs through hand-written HIP kernels in ``csrc/`` behind the C ABI
in ``include/ll_nvfp4.h``; :func:`install_as_fouroversix` registers the mirror under the
reference's import name.
"""
from __future__ import annotations

import sys

__version__ = "0.1.0"


def install_as_fouroversix() -> None:
    """Make ``import fouroversix`` (and the submodules LongLive imports from) resolve to this
    implementation, so the reference's ``utils/quant.py`` imports work unchanged."""
    import importlib

    prefix = __name__ + ".fouroversix"
    importlib.import_module(prefix)
    for name, module in list(sys.modules.items()):
        if name == prefix or name.startswith(prefix + "."):
            sys.modules["fouroversix" + name[len(prefix):]] = module
