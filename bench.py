#!/usr/bin/env python
"""Benchmark of the NVFP4 W4A4 hot path on one MI355X.

Workload (BASELINE.json configs[1]): the Wan2.2-TI2V-5B transformer-block linear set in NVFP4 W4A4 for
one 3-latent-frame chunk (M = 2640 tokens): q/k/v/o and cross q/o (6x K=N=3072), cross k/v on the 512
text tokens (2x), FFN up (N=14336) and FFN down (K=14336).  One step = quantize each activation to
NVFP4 (four-over-six, mse) and run its W4A4 GEMM against the pre-quantized weight: 783.4 GFLOP.
Inputs are synthetic (seed 1) and resident in HBM before the timed region.

Prints one JSON line: whole-step TFLOP/s, plus `roofline` for the dominant kernel (the FFN-up W4A4
GEMM, timed with HIP events on the launch stream) and `cpu_baseline` (the numpy oracle of the same
path timed on the host cores on a bounded sample).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

M_TOKENS, M_TEXT, DIM, FFN = 2640, 512, 3072, 14336
# (name, M, K, N, count)
LINEAR_SET = [
    ("attn_qkvo+cross_qo", M_TOKENS, DIM, DIM, 6),
    ("cross_kv", M_TEXT, DIM, DIM, 2),
    ("ffn_up", M_TOKENS, DIM, FFN, 1),
    ("ffn_down", M_TOKENS, FFN, DIM, 1),
]
PEAK_F16_TFLOPS = 2500.0  # MI355X dense fp16/bf16 MFMA peak (the GEMM runs v_mfma_f32_32x32x16_f16)


def step_flops() -> float:
    return sum(2.0 * m * k * n * c for _, m, k, n, c in LINEAR_SET)


def cpu_baseline() -> dict:
    """Oracle (numpy restatement of the reference's PyTorch path) on config 0's single linear:
    quantize X [2640,3072] and W [3072,3072] (mse), dequantize both, fp32 matmul, round to bf16."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import numpy as np
    import nvfp4_oracle as o
    from helpers import activations, bits_of, weights

    x, w = bits_of(activations((M_TOKENS, DIM), 0)), bits_of(weights((DIM, DIM), 0))
    t0 = time.perf_counter()
    ops = []
    for t in (x, w):
        v, s, a, pad = o.quantize_to_fp4(t, "mse")
        ops.append(dict(values=v, scales=s, amax=a, rule="mse", padded=pad, orig=t.shape))
    y = o.fp4_matmul(ops[0], ops[1])
    dt = time.perf_counter() - t0
    assert np.isfinite(y).all()
    flops = 2.0 * M_TOKENS * DIM * DIM
    return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)),
            "kind": "port", "sample": f"config0 single W4A4 linear M=2640 K=N=3072 incl. quantize of X and W, {dt:.2f} s"}


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (no collectives are part of this path); use --gpus 1")

    import torch

    from helpers import activations, weights
    from longlive_amd.fouroversix import QuantizationConfig, fp4_matmul, quantize_to_fp4

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    dev = torch.device("cuda:0")
    cfg = QuantizationConfig(scale_rule="mse")

    # weights pre-quantized offline, activations resident in HBM
    work = []
    seed = 1
    for name, m, k, n, count in LINEAR_SET:
        for i in range(count):
            wq = quantize_to_fp4(weights((n, k), seed * 1000 + len(work)).to(dev), cfg)
            x = activations((m, k), seed * 2000 + len(work)).to(dev)
            work.append((name, x, wq))
    torch.cuda.synchronize()

    def step():
        for _, x, wq in work:
            xq = quantize_to_fp4(x, cfg)
            fp4_matmul(xq, wq)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps

    # dominant kernel: FFN-up GEMM, HIP events on the launch stream (torch's current stream)
    name, x, wq = next(w for w in work if w[0] == "ffn_up")
    xq = quantize_to_fp4(x, cfg)
    reps = max(args.steps, 10)
    for _ in range(3):
        fp4_matmul(xq, wq)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fp4_matmul(xq, wq)
    e1.record()
    torch.cuda.synchronize()
    gemm_ms = e0.elapsed_time(e1) / reps
    gemm_flops = 2.0 * M_TOKENS * DIM * FFN
    achieved = gemm_flops / (gemm_ms * 1e-3) / 1e12

    # secondary figure: the activation quantizer on the FFN-down input (2640 x 14336), bytes = 2.5625 B/elt
    xbig = next(w for w in work if w[0] == "ffn_down")[1]
    for _ in range(3):
        quantize_to_fp4(xbig, cfg)
    e0.record()
    for _ in range(reps):
        quantize_to_fp4(xbig, cfg)
    e1.record()
    torch.cuda.synchronize()
    q_ms = e0.elapsed_time(e1) / reps
    q_gbs = 2.5625 * xbig.numel() / (q_ms * 1e-3) / 1e9

    out = {
        "metric": "W4A4 GEMM TFLOP/s, Wan2.2-TI2V-5B block linear set (NVFP4 activations quantized on the fly)",
        "value": step_flops() / dt / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": dt * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "nvfp4 operands, f16 MFMA, f32 accumulate",
        "data": "synthetic",
        "config": {"workload": "configs[1]: 10 W4A4 linears of one Wan2.2-TI2V-5B block, M=2640 (512 for cross k/v), "
                               "dim 3072, ffn 14336, rule mse, seed 1", "flop_per_step": step_flops()},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_F16_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_F16_TFLOPS, "traffic": None,
                     "kernel": "gemm_w4a4_kernel M=2640 N=14336 K=3072", "avg_ms": gemm_ms},
        "quantize": {"shape": [M_TOKENS, FFN], "avg_ms": q_ms, "GB_per_s": q_gbs, "frac_of_hbm_8TBs": q_gbs / 8000.0,
                     "note": "amax + quantize kernels, 2.5625 algorithmic bytes per element"},
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
