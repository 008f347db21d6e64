"""Writes the golden vectors under tests/golden/ by running the reference's own
PyTorch (CPU) backend.  Run in the development container only (it reads
/root/reference); the fixtures it writes are committed and are what the tests use.

What is pinned here that nothing else can pin bit-exactly:

* ``select_fouroversix`` (mse / mae / abs_max): the fp32 summation order of the
  per-block error and the strict ``<`` tie rule;
* ``QuantizedTensor.dequantize`` rounding order ``(v*s)*amax/(6*256)``;
* ``PyTorchMatmulBackend.fp4_matmul`` output (bf16) for a small W4A4 product.

The reference package's ``__init__`` needs distribution metadata and GPU-only
back ends, so its pure-PyTorch files are imported as submodules of stub parent
packages (no reference code is copied; only inputs and outputs are stored).
"""
from __future__ import annotations

import os
import sys
import types

import numpy as np
import torch

SRC = "/root/reference/fouroversix/src/fouroversix"
OUT = os.path.dirname(os.path.abspath(__file__))


def _stub(name: str, path: str) -> types.ModuleType:
    m = types.ModuleType(name)
    m.__path__ = [path]
    sys.modules[name] = m
    return m


def load_reference():
    _stub("fouroversix", SRC)
    q = _stub("fouroversix.quantize", SRC + "/quantize")
    _stub("fouroversix.quantize.pytorch", SRC + "/quantize/pytorch")
    _stub("fouroversix.matmul", SRC + "/matmul")
    from fouroversix.quantize.pytorch.reference import quantize_to_fp4 as ref_quantize
    from fouroversix.quantize.quantized_tensor import QuantizedTensor
    from fouroversix.quantize.config import QuantizationConfig
    from fouroversix.utils import DataType, ScaleRule

    q.QuantizedTensor = QuantizedTensor
    q.QuantizationConfig = QuantizationConfig
    from fouroversix.matmul.pytorch import PyTorchMatmulBackend

    return ref_quantize, QuantizedTensor, PyTorchMatmulBackend, DataType, ScaleRule


def make_input(kind: str, shape, seed: int) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    if kind == "zeros":
        return torch.zeros(shape, dtype=torch.bfloat16)
    if kind == "ones":
        return torch.ones(shape, dtype=torch.bfloat16)
    if kind == "rand01":
        return torch.rand(shape, generator=g).bfloat16()
    if kind == "randn":
        return torch.randn(shape, generator=g).bfloat16()
    if kind == "randn_outliers":  # activations of the benchmark configs
        x = torch.randn(shape, generator=g)
        mask = torch.rand(shape, generator=g) < 1e-3
        return torch.where(mask, x * 20, x).bfloat16()
    if kind == "weights":
        return (torch.randn(shape, generator=g) * 0.02).bfloat16()
    if kind == "smallblocks":  # blocks far below amax: sub-normal / zero e4m3 scales, |y| >= 7 codes
        x = torch.randn(shape, generator=g)
        rowscale = torch.logspace(-7, 0, shape[0]).unsqueeze(1)
        x = x * rowscale
        x[0, 0] = 300.0
        x[1, :16] = -0.0
        return x.bfloat16()
    raise ValueError(kind)


def make_adversarial(ScaleRule) -> torch.Tensor:
    """[128, 1024] bf16: element (0,0) fixes amax = 64; the other 8191 blocks are drawn from a
    large random pool and kept only if the 4-vs-6 choice made with torch's own ``sum`` differs
    from the choice a left-to-right loop would make (first half: mse, second half: mae)."""
    from fouroversix.quantize.pytorch import reference as R

    g = torch.Generator().manual_seed(7)
    amax = torch.tensor(64.0)
    picked = {"mse": [], "mae": []}
    need = {"mse": 4096, "mae": 4095}
    while any(len(torch.cat(v)) < need[k] if v else True for k, v in picked.items()):
        x = torch.randn(1 << 20, 16, generator=g) * torch.rand(1 << 20, 1, generator=g) * 8
        x = x.bfloat16().float().clamp(-60, 60)
        b6, s6 = R.quantize_to_nvfp4(x, amax, scale_rule=ScaleRule.mse)
        b4, s4 = R.quantize_to_nvfp4(x, amax, scale_rule=ScaleRule.mse, scale_expansion_factor=1.5)
        d6 = R.fake_quantize_to_e2m1(b6) * s6.unsqueeze(1).float() * amax / torch.tensor(1536.0)
        d4 = R.fake_quantize_to_e2m1(b4) * s4.unsqueeze(1).float() * amax / torch.tensor(1536.0)
        for rule, t4, t6 in (("mse", (d4 - x) ** 2, (d6 - x) ** 2), ("mae", (d4 - x).abs(), (d6 - x).abs())):
            ref_pick = t4.sum(-1) < t6.sum(-1)
            a4 = torch.zeros(x.shape[0])
            a6 = torch.zeros(x.shape[0])
            for j in range(16):
                a4 = a4 + t4[:, j]
                a6 = a6 + t6[:, j]
            picked[rule].append(x[ref_pick != (a4 < a6)])
    blocks = torch.cat([torch.cat(picked["mse"])[:4096], torch.cat(picked["mae"])[:4095]])
    first = torch.zeros(1, 16)
    first[0, 0] = 64.0
    return torch.cat([first, blocks]).reshape(128, 1024).bfloat16()


def bits(x: torch.Tensor) -> np.ndarray:
    return x.view(torch.int16).numpy().view(np.uint16).copy()


def main() -> None:
    torch.manual_seed(0)
    ref_quantize, QuantizedTensor, Matmul, DataType, ScaleRule = load_reference()
    cases = [
        ("randn_outliers", (256, 1024), 0),
        ("randn", (128, 512), 1),
        ("weights", (256, 512), 2),
        ("rand01", (128, 256), 3),
        ("smallblocks", (128, 128), 4),
        ("ones", (128, 64), 5),
        ("zeros", (128, 64), 6),
    ]
    rules = ["static_6", "static_4", "mae", "mse", "abs_max"]
    blob: dict[str, np.ndarray] = {}
    names = []
    for kind, shape, seed in cases:
        x = make_input(kind, shape, seed)
        key = f"{kind}_{shape[0]}x{shape[1]}_s{seed}"
        names.append(key)
        blob[f"{key}/x"] = bits(x)
        for rule in rules:
            values, scales, amax = ref_quantize(x, scale_rule=ScaleRule(rule))
            blob[f"{key}/{rule}/values"] = values.numpy().copy()
            blob[f"{key}/{rule}/scales"] = scales.view(torch.uint8).numpy().copy()
            blob[f"{key}/{rule}/amax"] = amax.reshape(1).numpy().copy()
            if kind in ("randn", "weights") and rule in ("mse", "static_6"):
                qt = QuantizedTensor(values, scales, amax, DataType.nvfp4, tuple(shape), ScaleRule(rule))
                blob[f"{key}/{rule}/deq_f32"] = qt.dequantize(torch.float32).numpy().copy()
                blob[f"{key}/{rule}/deq_bf16"] = bits(qt.dequantize(torch.bfloat16))
    # adversarial case: only blocks whose 4-vs-6 decision differs between the reduction order the
    # reference's CPU run uses and a plain left-to-right fp32 sum (mse and mae halves)
    adv = make_adversarial(ScaleRule)
    names.append("adversarial_128x1024_s7")
    blob["adversarial_128x1024_s7/x"] = bits(adv)
    for rule in rules:
        values, scales, amax = ref_quantize(adv, scale_rule=ScaleRule(rule))
        blob[f"adversarial_128x1024_s7/{rule}/values"] = values.numpy().copy()
        blob[f"adversarial_128x1024_s7/{rule}/scales"] = scales.view(torch.uint8).numpy().copy()
        blob[f"adversarial_128x1024_s7/{rule}/amax"] = amax.reshape(1).numpy().copy()
    # one W4A4 product: X [128, 512] (randn, seed 1) times W [256, 512] (weights, seed 2), rule mse
    xq = ref_quantize(make_input("randn", (128, 512), 1), scale_rule=ScaleRule.mse)
    wq = ref_quantize(make_input("weights", (256, 512), 2), scale_rule=ScaleRule.mse)
    a = QuantizedTensor(*xq, DataType.nvfp4, (128, 512), ScaleRule.mse)
    b = QuantizedTensor(*wq, DataType.nvfp4, (256, 512), ScaleRule.mse)
    y = Matmul.fp4_matmul(a, b, out_dtype=DataType.bfloat16)
    blob["matmul/randn_128x512_s1__weights_256x512_s2/mse/out_bf16"] = bits(y)
    blob["case_names"] = np.array(names)
    blob["torch_cpu_capability"] = np.array([torch.backends.cpu.get_cpu_capability()])
    np.savez_compressed(os.path.join(OUT, "nvfp4_reference_vectors.npz"), **blob)
    print("wrote", len(blob), "arrays; cpu capability", torch.backends.cpu.get_cpu_capability())


if __name__ == "__main__":
    main()
