"""Writes tests/golden/fouroversix_linear_state.npz: the state dict that the reference's own FourOverSixLinear
(fouroversix/src/fouroversix/model/modules/linear.py:153-355) produces for two small nn.Linear layers, and the
output of its forward on a fixed input.  Run in the development container only (it reads /root/reference); the
fixture it writes is committed and is what tests/test_gpu_gemm.py loads into this package's FourOverSixLinear with
strict=True.

Only data is stored: weights and inputs chosen here, and the buffers / outputs the reference computes from them
(`quantized_weight_values`, `_scale_factors`, `_amax`, `_metadata`, linear.py:182-216, 271-307).  The reference's
package __init__ needs distribution metadata and GPU-only back ends, so its modules are imported as submodules of
stub parent packages with the pure-PyTorch back ends wired in (as make_golden.py does).
"""
from __future__ import annotations

import os
import sys

import numpy as np
import torch
import torch.nn as nn

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import make_golden as mg  # noqa: E402


def load_reference_linear():
    ref_quantize, QuantizedTensor, PyTorchMatmulBackend, DataType, ScaleRule = mg.load_reference()
    import fouroversix.quantize as q_pkg
    import fouroversix.matmul as m_pkg
    from fouroversix.quantize.pytorch.backend import PyTorchQuantizeBackend

    def quantize_to_fp4(x, config=None):
        config = config or q_pkg.QuantizationConfig()
        return PyTorchQuantizeBackend.quantize_to_fp4(x, config)

    def fp4_matmul(input, other, *, backend=None, input_config=None, other_config=None, out_dtype=DataType.bfloat16):
        return PyTorchMatmulBackend.fp4_matmul(input, other, out_dtype=out_dtype)

    q_pkg.quantize_to_fp4 = quantize_to_fp4
    m_pkg.fp4_matmul = fp4_matmul
    mg._stub("fouroversix.model", mg.SRC + "/model")
    mg._stub("fouroversix.model.modules", mg.SRC + "/model/modules")
    from fouroversix.model.config import ModuleQuantizationConfig
    from fouroversix.model.modules.linear import FourOverSixLinear

    return FourOverSixLinear, ModuleQuantizationConfig


def bits(t: torch.Tensor) -> np.ndarray:
    return t.detach().contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def main() -> None:
    FourOverSixLinear, ModuleQuantizationConfig = load_reference_linear()
    out = {}
    names = []
    for name, (fin, fout, rows, seed) in {"aligned_192x128": (192, 128, 40, 0), "padded_128x96": (128, 96, 17, 1)}.items():
        g = torch.Generator().manual_seed(seed)
        lin = nn.Linear(fin, fout, bias=True)
        with torch.no_grad():
            lin.weight.copy_(torch.randn(fout, fin, generator=g) * 0.05)
            lin.bias.copy_(torch.randn(fout, generator=g) * 0.1)
        lin = lin.to(torch.bfloat16)
        mod = FourOverSixLinear(lin, ModuleQuantizationConfig(scale_rule="mse"))
        registered = {k: (tuple(v.shape), str(v.dtype)) for k, v in mod.state_dict().items()}
        params = mod.get_quantized_parameters("weight", mod.weight.data)
        # what the reference's model-level quantization does with them (model/quantize.py): replace the buffers
        for key, val in params.items():
            setattr(mod, key, nn.Parameter(val, requires_grad=False))
        del mod.weight
        mod.weight = None
        x = (torch.randn(rows, fin, generator=g) * torch.where(torch.rand(rows, fin, generator=g) < 0.01, 20.0, 1.0)).bfloat16()
        with torch.no_grad():
            y = mod(x)
        sd = {k: v for k, v in mod.state_dict().items()}
        names.append(name)
        out[f"{name}/weight"] = bits(lin.weight.data)
        out[f"{name}/bias"] = bits(lin.bias.data)
        out[f"{name}/x"] = bits(x)
        out[f"{name}/y"] = bits(y)
        out[f"{name}/state_keys"] = np.array(sorted(sd.keys()))
        out[f"{name}/registered_keys"] = np.array(sorted(registered.keys()))
        for k, v in registered.items():
            out[f"{name}/registered_shape/{k}"] = np.array(v[0], dtype=np.int64)
        for k, v in sd.items():
            if v.dtype == torch.float8_e4m3fn:
                out[f"{name}/state/{k}"] = v.view(torch.uint8).numpy().copy()
            elif v.dtype == torch.bfloat16:
                out[f"{name}/state/{k}"] = bits(v)
            else:
                out[f"{name}/state/{k}"] = v.numpy().copy()
            out[f"{name}/state_dtype/{k}"] = np.array(str(v.dtype))
    out["case_names"] = np.array(names)
    path = os.path.join(mg.OUT, "fouroversix_linear_state.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")
    for n in names:
        print(n, list(out[f"{n}/state_keys"]), {k.split('/')[-1]: out[k].shape for k in out if k.startswith(f"{n}/state/")})


if __name__ == "__main__":
    main()
