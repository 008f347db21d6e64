#!/usr/bin/env python
"""Benchmark of the NVFP4 W4A4 hot path on one MI355X.

Workload (benchmark configuration 2, `configs[1]`): the Wan2.2-TI2V-5B transformer-block linear set in NVFP4 W4A4 for
one 3-latent-frame chunk (M = 2640 tokens): q/k/v/o and cross q/o (6x K=N=3072), cross k/v on the 512
text tokens (2x), FFN up (N=14336) and FFN down (K=14336).  One step = quantize each activation to
NVFP4 (four-over-six, mse) and run its W4A4 GEMM against the pre-quantized weight: 783.4 GFLOP.
Inputs are synthetic (seed 1) and resident in HBM before the timed region.

Prints one JSON line: whole-step TFLOP/s, plus `roofline` for the dominant kernel (the FFN-up W4A4
GEMM, timed with HIP events on the launch stream) and `cpu_baseline` (the numpy oracle of the same
step timed once on the host cores).  `--workload attention|block|e2e` run benchmark configurations 3 to 5 (`configs[2..4]`)
alone (one kernel or model under a profiler); the default run reports them under `extras`.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

M_TOKENS, M_TEXT, DIM, FFN, HEADS = 2640, 512, 3072, 14336, 24
# (name, M, K, N, count)
LINEAR_SET = [
    ("attn_qkvo+cross_qo", M_TOKENS, DIM, DIM, 6),
    ("cross_kv", M_TEXT, DIM, DIM, 2),
    ("ffn_up", M_TOKENS, DIM, FFN, 1),
    ("ffn_down", M_TOKENS, FFN, DIM, 1),
]
PEAK_F16_TFLOPS = 2500.0  # MI355X dense fp16/bf16 MFMA peak (the GEMM runs v_mfma_f32_32x32x16_f16)
PEAK_FP8_TFLOPS = 5000.0  # MI355X dense FP8 MFMA peak: the figure BASELINE.json's W4A4 target is quoted against
PEAK_HBM_GBS = 8000.0     # MI355X HBM3E peak
PREWARM_SECONDS = 0.5  # untimed load ahead of the warm-up steps (clock ramp-up), reported as config.prewarm_s
# rocprofv3 counter summary of the FFN-up GEMM launch (FETCH_SIZE / WRITE_SIZE per dispatch and the factors a plain
# copy of known size calibrates); roofline.traffic is computed from the numbers in that file, or null without it
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "gemm_w4a4_ffn_up_hbm_traffic.txt")


def measured_traffic_bytes():
    """HBM bytes of one FFN-up GEMM launch = FETCH_SIZE x fetch factor + WRITE_SIZE x write factor, read from the
    `key = value` lines of the counter summary under profiles/ (None when the file or a key is missing)."""
    keys = {"fetch_size_kib_per_launch": None, "fetch_scale": None, "write_size_kib_per_launch": None, "write_scale": None}
    try:
        with open(TRAFFIC_PROFILE) as f:
            for line in f:
                name, sep, value = line.partition("=")
                if sep and name.strip() in keys:
                    keys[name.strip()] = float(value.split()[0])
    except (OSError, ValueError):
        return None
    if any(v is None for v in keys.values()):
        return None
    return (keys["fetch_size_kib_per_launch"] * keys["fetch_scale"]
            + keys["write_size_kib_per_launch"] * keys["write_scale"]) * 1024.0


def live_traffic_bytes():
    """The same figure measured now: four child runs of this file under `rocprofv3 --pmc` (FETCH_SIZE and WRITE_SIZE,
    each for the linear set and for a device copy of known size that calibrates the counter), started before this
    process touches the GPU.  Returns (bytes, details) or (None, reason)."""
    import csv
    import shutil
    import subprocess
    import tempfile

    if shutil.which("rocprofv3") is None:
        return None, "rocprofv3 not found"
    out = tempfile.mkdtemp(prefix="ll_traffic_", dir=os.environ.get("TMPDIR", "/tmp"))
    env = dict(os.environ, TMPDIR=os.environ.get("TMPDIR", "/tmp"))

    def counter(name, workload, kernel):
        d = os.path.join(out, f"{name}_{workload}")
        cmd = ["rocprofv3", "--pmc", name, "--output-format", "csv", "-d", d, "-o", "p", "--", sys.executable,
               os.path.abspath(__file__), "--no-cpu-baseline", "--no-extras", "--workload", workload, "--steps", "5", "--warmup", "2"]
        subprocess.run(cmd, env=env, cwd=ROOT, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL, timeout=150, check=True)
        values = []
        with open(os.path.join(d, "p_counter_collection.csv")) as f:
            for row in csv.DictReader(f):
                if row["Counter_Name"] == name and kernel(row):
                    values.append(float(row["Counter_Value"]))
        if not values:
            raise RuntimeError(f"no {name} rows for {workload}")
        return sum(values) / len(values)

    ffn_up = lambda r: "gemm_w4a4_asm_kernel<4, 2>" in r["Kernel_Name"] and r["Grid_Size"] == "315392"
    copy = lambda r: "copyBuffer" in r["Kernel_Name"]
    try:
        fetch, write = counter("FETCH_SIZE", "linears", ffn_up), counter("WRITE_SIZE", "linears", ffn_up)
        fetch_copy, write_copy = counter("FETCH_SIZE", "copy", copy), counter("WRITE_SIZE", "copy", copy)
    except (OSError, subprocess.SubprocessError, RuntimeError, KeyError, ValueError) as e:
        return None, f"{type(e).__name__}: {e}"
    finally:
        shutil.rmtree(out, ignore_errors=True)
    copied_kib = 256.0 * 1024.0  # the copy workload moves 256 MiB each way
    details = {"fetch_size_kib_per_launch": fetch, "fetch_scale": copied_kib / fetch_copy,
               "write_size_kib_per_launch": write, "write_scale": copied_kib / write_copy}
    return (fetch * details["fetch_scale"] + write * details["write_scale"]) * 1024.0, details


def physical_cores() -> int:
    """Physical cores this process may use: distinct (package, core) pairs of /proc/cpuinfo among the CPUs of the
    affinity mask, capped by OMP_NUM_THREADS (the share of the machine a one-GPU job is given)."""
    try:
        allowed = os.sched_getaffinity(0)
    except AttributeError:
        allowed = set(range(os.cpu_count() or 1))
    cores, cpu, phys = set(), None, "0"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                key, _, val = line.partition(":")
                key, val = key.strip(), val.strip()
                if key == "processor":
                    cpu, phys = int(val), "0"
                elif key == "physical id":
                    phys = val
                elif key == "core id" and cpu in allowed:
                    cores.add((phys, val))
    except OSError:
        pass
    n = len(cores) or len(allowed)
    cap = os.environ.get("OMP_NUM_THREADS")
    return max(1, min(n, int(cap)) if cap and cap.isdigit() else n)


def step_flops() -> float:
    return sum(2.0 * m * k * n * c for _, m, k, n, c in LINEAR_SET)


def cpu_baseline(work) -> dict:
    """Oracle (numpy restatement of the reference's PyTorch path) over one whole step: each of the ten
    activations quantized (mse), both operands dequantized, fp32 matmul, result rounded to bf16.  The
    weights are the same pre-quantized operands the GPU step uses, copied to the host beforehand."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import numpy as np
    import nvfp4_oracle as o
    import torch
    from longlive_amd.utils.synthetic import bits_of

    from threadpoolctl import threadpool_limits

    cores = physical_cores()
    host = []
    for _, x, wq in work:
        wd = dict(values=wq.values.cpu().numpy(), scales=wq.scale_factors.cpu().view(torch.uint8).numpy(),
                  amax=np.float32(wq.amax.item()), rule="mse", padded=tuple(wq.padded_shape), orig=tuple(wq.original_shape))
        host.append((bits_of(x.cpu()), wd))
    n_steps = 0
    with threadpool_limits(limits=cores):  # BLAS threads of the fp32 matmul = physical cores; the rest is numpy
        t0 = time.perf_counter()
        while n_steps < 1 or (time.perf_counter() - t0 < 10.0 and n_steps < 8):  # about 10-30 s of CPU work
            for xb, wd in host:
                v, sc, a, pad = o.quantize_to_fp4(xb, "mse")
                y = o.fp4_matmul(dict(values=v, scales=sc, amax=a, rule="mse", padded=pad, orig=xb.shape), wd)
            n_steps += 1
        dt = time.perf_counter() - t0
    assert np.isfinite(y).all()
    return {"value": n_steps * step_flops() / dt / 1e12, "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": f"{n_steps} whole step(s) of the same workload (10 linears, 783.4 GFLOP each, weights "
                      f"pre-quantized), {dt:.1f} s; BLAS threads limited to the {cores} physical cores of the "
                      "process's CPU share, the element-wise numpy part of the oracle is single-threaded"}


def _time_events(torch, fn, n, warm=10, repeats=3):
    """HIP-event time per call over n calls, best of `repeats` (the secondary figures share the process with
    host-heavy set-up, and a forward is only ~3x longer on the GPU than on the host).  The warm-up is long
    enough for the clocks to come up after the set-up that precedes it."""
    for _ in range(warm):
        fn()
    best = float("inf")
    for _ in range(repeats):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        best = min(best, e0.elapsed_time(e1) / n)
    return best


def _filled_cache(torch, dev, g):
    """Benchmark configuration 3 (`configs[2]`): a 5-slot FP4 cache of 2640-token blocks with slots 0..3 written
    (sink + three window blocks) by four streaming steps, so the next chunk attends 13200 keys."""
    from longlive_amd.fouroversix import QuantizationConfig
    from longlive_amd.utils import kv_cache as kvc

    kv_cfg = QuantizationConfig(scale_rule="mse")
    cache = kvc.initialize_kv_cache(1, M_TOKENS, 5, HEADS, 128, kv_cfg, dev)[0]
    for chunk in range(4):
        q, k, v = (torch.randn(1, M_TOKENS, HEADS, 128, generator=g).bfloat16().to(dev) for _ in range(3))
        _, (g_end, l_end, info) = kvc.kv_cache_attention(q, k, v, cache, chunk * M_TOKENS, sink_tokens=M_TOKENS)
        kvc.apply_cache_update(cache, g_end, l_end, info, kv_cfg)
    return cache, kv_cfg


def run_attention(torch, dev, steps):
    """configs[2]: 24 heads x 128, 2640 queries over 10560 cached FP4 keys + the 2640-token bf16 chunk."""
    from longlive_amd.utils import kv_cache as kvc

    g = torch.Generator().manual_seed(2)
    cache, kv_cfg = _filled_cache(torch, dev, g)
    q, k, v = (torch.randn(1, M_TOKENS, HEADS, 128, generator=g).bfloat16().to(dev) for _ in range(3))
    from longlive_amd.utils.quant import k_smooth
    ks = k_smooth(k)  # the block gets the smoothed key from its norm + RoPE kernel; only the attention launch is timed
    ms = _time_events(torch, lambda: kvc.kv_cache_attention(q, k, v, cache, 4 * M_TOKENS, sink_tokens=M_TOKENS,
                                                            smoothed_key=ks), steps)
    flops = 4.0 * M_TOKENS * (5 * M_TOKENS) * 128 * HEADS
    info = dict(action="direct_insert", local_start_index=4 * M_TOKENS, local_end_index=5 * M_TOKENS, new_k=k, new_v=v)
    wms = _time_events(torch, lambda: kvc.apply_cache_update(cache, 5 * M_TOKENS, 5 * M_TOKENS, info, kv_cfg), steps)
    return {"attention_ms": ms, "attention_TFLOPs": flops / ms / 1e9, "attention_frac_of_bf16_peak": flops / ms / 1e9 / PEAK_F16_TFLOPS,
            "kv_write_ms": wms, "kv_write_GBs": 2 * 2.5625 * M_TOKENS * HEADS * 128 / wms / 1e6,
            "workload": "configs[2]: Lq=2640, Lk=13200 (4 FP4 slots + bf16 chunk), 24 heads x 128, 428.2 GFLOP"}


def run_block(torch, dev, steps):
    """configs[3]: one DiT block (dim 3072, ffn 14336, 24 heads) on the cache of configs[2]."""
    from longlive_amd.dit import DiTBlock
    from longlive_amd.fouroversix import ModelQuantizationConfig
    from longlive_amd.utils.quant import quantize_model_with_filter
    from longlive_amd.utils.rope import build_rope_angles, rope_cos_sin

    g = torch.Generator().manual_seed(3)
    cache, _ = _filled_cache(torch, dev, g)
    torch.manual_seed(3)
    block = DiTBlock(DIM, FFN, HEADS).to(dev)
    block, _ = quantize_model_with_filter(block, ModelQuantizationConfig(), use_default_filtered_modules=True,
                                          materialize_for_inference=True, verbose=False)
    x = torch.randn(1, M_TOKENS, DIM, generator=g).bfloat16().to(dev)
    e0 = torch.randn(1, 3, 6, DIM, generator=g).bfloat16().to(dev)
    ctx = torch.randn(1, M_TEXT, DIM, generator=g).bfloat16().to(dev)
    cos, sin = rope_cos_sin(build_rope_angles(128), 3, 22, 40, 12, dev)
    with torch.no_grad():
        # no cache update follows these forwards, so they do not ask for the K / V maxima (collect_kv_amax)
        ms = _time_events(torch, lambda: block(x, e0, cos, sin, ctx, cache, 4 * M_TOKENS, sink_tokens=M_TOKENS,
                                               collect_kv_amax=False), steps)
    return {"block_ms": ms, "block_TFLOPs": 1228.2 / ms,
            "workload": "configs[3]: one NVFP4 DiT block forward, 1228.2 GFLOP (783.4 linears + 428.2 self-attn + 16.6 cross-attn)"}


def run_block_release(torch, dev, steps):
    """One DiT block at the shapes of the reference's released NVFP4 configuration (chunks of 8 latent frames =
    7040 tokens, window of 32 frames = 4 cache blocks, sink 8 frames): the chunk attends the sink block, two
    cached blocks and itself, 28160 keys.  Not one of the benchmark configurations; reported beside them."""
    from longlive_amd.dit import DiTBlock
    from longlive_amd.fouroversix import ModelQuantizationConfig, QuantizationConfig
    from longlive_amd.utils import kv_cache as kvc
    from longlive_amd.utils.quant import quantize_model_with_filter
    from longlive_amd.utils.rope import build_rope_angles, rope_cos_sin

    tokens, blocks = 8 * 880, 4
    g = torch.Generator().manual_seed(5)
    kv_cfg = QuantizationConfig(scale_rule="mse")
    cache = kvc.initialize_kv_cache(1, tokens, blocks, HEADS, 128, kv_cfg, dev)[0]
    for chunk in range(blocks):
        q, k, v = (torch.randn(1, tokens, HEADS, 128, generator=g).bfloat16().to(dev) for _ in range(3))
        _, (g_end, l_end, info) = kvc.kv_cache_attention(q, k, v, cache, chunk * tokens, sink_tokens=tokens)
        kvc.apply_cache_update(cache, g_end, l_end, info, kv_cfg)
    torch.manual_seed(5)
    block = DiTBlock(DIM, FFN, HEADS).to(dev)
    block, _ = quantize_model_with_filter(block, ModelQuantizationConfig(), use_default_filtered_modules=True,
                                          materialize_for_inference=True, verbose=False)
    x = torch.randn(1, tokens, DIM, generator=g).bfloat16().to(dev)
    e0 = torch.randn(1, 8, 6, DIM, generator=g).bfloat16().to(dev)
    ctx = torch.randn(1, M_TEXT, DIM, generator=g).bfloat16().to(dev)
    cos, sin = rope_cos_sin(build_rope_angles(128), 8, 22, 40, 32, dev)
    with torch.no_grad():
        ms = _time_events(torch, lambda: block(x, e0, cos, sin, ctx, cache, blocks * tokens, sink_tokens=tokens,
                                               collect_kv_amax=False), steps)
    gflop = (2.0 * tokens * (8 * DIM * DIM + 2 * DIM * FFN) - 2 * 2.0 * (tokens - M_TEXT) * DIM * DIM  # k/v of cross-attention run on the text
             + 4.0 * tokens * (blocks * tokens) * 128 * HEADS + 4.0 * tokens * M_TEXT * 128 * HEADS) / 1e9
    return {"block_ms": ms, "block_TFLOPs": gflop / ms, "gflop": gflop,
            "workload": "released configuration: one NVFP4 DiT block forward, 7040 tokens, 28160 keys (3 FP4 slots + bf16 chunk)"}


def run_e2e(torch, dev):
    """configs[4]: 30 blocks, 10 chunks of 3 latent frames, 4 denoising forwards + 1 cache-rewrite forward each."""
    from longlive_amd.dit import DiTConfig, StreamingGenerator

    gen = StreamingGenerator(DiTConfig(), dev, seed=4)
    g = torch.Generator().manual_seed(4)
    noise = torch.randn(1, 30, 48, 44, 80, generator=g).bfloat16().to(dev)
    ctx = torch.randn(M_TEXT, 4096, generator=g).bfloat16().to(dev)
    marks = []

    def on_chunk(_):
        torch.cuda.synchronize()
        marks.append(time.perf_counter())

    gen.generate(noise[:, :6], ctx)  # untimed two-chunk run: first launches (with and without cached slots), allocator growth
    gen.kv_cache = None              # the timed run starts from an empty cache
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    out = gen.generate(noise, ctx, on_chunk)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    per = [marks[0] - t0] + [b - a for a, b in zip(marks, marks[1:])]
    return {"latent_frames_per_s": 30.0 / dt, "seconds_30_frames": dt, "steady_chunk_ms": 1e3 * min(per[5:]),
            "steady_latent_frames_per_s": 3.0 / min(per[5:]), "chunk_ms": [round(1e3 * t, 1) for t in per], "finite": bool(torch.isfinite(out.float()).all().item()),
            "workload": "configs[4]: 30-block NVFP4 generator, 10 chunks x (4 denoising + 1 recache) forwards, FP4 KV cache "
                        "sink 3 + window 12 frames, text K/V projected once per prompt, cache written by the recache forward only (the denoising forwards' writes are dead stores), and that forward stops behind the last layer's K / V (its prediction has no reader); one untimed 6-frame run first; the chunks get slower until the window of 12 frames is full"}


def run_quantize(torch, dev, steps, rule="mse"):
    """The quantize kernel alone on the FFN-down activation (2640 x 14336 bf16, the tensor with the most blocks),
    tensor amax taken from the amax sink its producer filled, as in the DiT block (no reduction pass): the launch
    the `roofline_quantize` record and the instruction-count profile are about."""
    from longlive_amd.utils.synthetic import activations, weights
    from longlive_amd import _native
    from longlive_amd.fouroversix import QuantizationConfig, fp4_matmul, quantize_to_fp4

    cfg = QuantizationConfig(scale_rule=rule)
    # the tensor the DiT block quantizes at this point: the FFN-up GEMM's GELU output, whose amax that GEMM's
    # epilogue leaves in the sink
    xq = quantize_to_fp4(activations((M_TOKENS, DIM), 2008).to(dev), QuantizationConfig(scale_rule="mse"))
    wq = quantize_to_fp4(weights((FFN, DIM), 1008).to(dev), QuantizationConfig(scale_rule="mse"))
    ticket = _native.amax_ticket(dev)
    x = fp4_matmul(xq, wq, activation="gelu_tanh", amax_out=ticket)
    ms = _time_events(torch, lambda: quantize_to_fp4(x, cfg, amax=ticket), steps)
    gbs = 2.5625 * x.numel() / ms / 1e6
    return {"quantize_ms": ms, "GB_per_s": gbs, "frac_of_hbm_8TBs": gbs / PEAK_HBM_GBS, "rule": rule,
            "workload": "quantize_kernel alone, 2640 x 14336 bf16 -> NVFP4, 96.98 MB algorithmic traffic, amax from a sink"}


def run_copy(torch, dev, steps):
    """Plain device-to-device copies, the yardstick for what the memory system gives a streaming kernel: 608 MiB
    (read + write beyond the 256 MB last-level cache, so every byte moves through HBM) and 76 MB (the bytes of the
    FFN-down activation, which stay in the last-level cache between launches)."""
    rows = {}
    for key, n in (("beyond_cache", 304 << 20), ("cached", 75_694_080)):
        src = torch.empty(n, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        ms = _time_events(torch, lambda: dst.copy_(src), steps)
        gbs = 2.0 * n / ms / 1e6
        rows[key] = {"bytes_read_plus_written": 2 * n, "ms": ms, "GB_per_s": gbs, "frac_of_hbm_8TBs": gbs / PEAK_HBM_GBS}
        del src, dst
    return rows


def run_gemm_shapes(torch, dev, work, cfg, steps):
    """The W4A4 GEMM kernel alone on each distinct shape of the linear set (operands already quantized), with the
    vendor library's dense f16 GEMM (torch.matmul) on operands of the same shape beside it: the library kernel
    does the same MFMA work without any FP4 decoding, which makes it the yardstick for the fused kernel."""
    from longlive_amd.fouroversix import fp4_matmul, quantize_to_fp4

    rows, seen = [], set()
    for name, x, wq in work:
        m, k = x.shape
        n = wq.original_shape[0]
        if (m, n, k) in seen:
            continue
        seen.add((m, n, k))
        xq = quantize_to_fp4(x, cfg)
        ms = _time_events(torch, lambda: fp4_matmul(xq, wq), steps)
        a16 = x.to(torch.float16)
        w16 = torch.randn(n, k, device=dev, dtype=torch.float16)
        lib = _time_events(torch, lambda: torch.matmul(a16, w16.t()), steps)
        flops = 2.0 * m * n * k
        rows.append({"linear": name, "M": m, "N": n, "K": k, "w4a4_us": 1e3 * ms, "w4a4_TFLOPs": flops / ms / 1e9,
                     "library_f16_us": 1e3 * lib, "library_f16_TFLOPs": flops / lib / 1e9})
        del a16, w16
    return rows


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true", help="skip the attention / block / end-to-end figures")
    ap.add_argument("--workload", choices=["linears", "attention", "block", "block_release", "e2e", "copy", "quantize", "quantize_static"], default="linears")
    ap.add_argument("--measure-traffic", action="store_true",
                    help="measure roofline.traffic now (four child runs under rocprofv3 --pmc, about a minute) "
                         "instead of reading the committed counter summary")
    ap.add_argument("--separate-norm-quantize", action="store_true",
                    help="block / e2e workloads: adaLN or LayerNorm and the quantization behind it as two launches "
                         "(for comparisons; the default is the one-launch kernel where it applies)")
    ap.add_argument("--gemm-schedule", choices=["auto", "tiles", "tiles_compiled", "persistent"], default="auto",
                    help="which kernel the GEMM entry points run (for comparisons; the default is the library's choice)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (no collectives are part of this path); use --gpus 1")
    live_traffic = live_traffic_bytes() if args.measure_traffic else None  # child processes, before this one uses the GPU

    import torch

    from longlive_amd.utils.synthetic import activations, weights
    from longlive_amd.fouroversix import QuantizationConfig, fp4_matmul, quantize_to_fp4

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    dev = torch.device("cuda:0")
    cfg = QuantizationConfig(scale_rule="mse")
    if args.separate_norm_quantize:
        from longlive_amd.dit import DiTBlock
        DiTBlock.fuse_norm_quantize = False
    if args.gemm_schedule != "auto":
        from longlive_amd import _native
        _native.gemm_schedule(args.gemm_schedule).__enter__()  # for the whole run
    if args.workload == "copy":
        # plain device copy of known size: the yardstick the FETCH_SIZE / WRITE_SIZE counters are scaled by
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        ms = _time_events(torch, lambda: dst.copy_(src), args.steps)
        print(json.dumps({"copy_bytes": src.numel(), "ms": ms, "GBs_read_plus_write": 2 * src.numel() / ms / 1e6}))
        return
    if args.workload != "linears":
        res = {"attention": lambda: run_attention(torch, dev, args.steps), "block": lambda: run_block(torch, dev, args.steps),
               "block_release": lambda: run_block_release(torch, dev, args.steps),
               "quantize": lambda: run_quantize(torch, dev, args.steps),
               "quantize_static": lambda: run_quantize(torch, dev, args.steps, "static_6"),
               "e2e": lambda: run_e2e(torch, dev)}[args.workload]()
        print(json.dumps(res))
        return

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

    # The shader clock needs a few hundred milliseconds of load to leave its idle state (the first launches after
    # an idle period run 10-25 % slower); the same step is therefore run untimed for half a second before the
    # W warm-up steps, so that W and K measure the sustained rate whatever their values.
    t_pre = time.perf_counter()
    while time.perf_counter() - t_pre < PREWARM_SECONDS:
        step()
        torch.cuda.synchronize()
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
    # the same quantization as the DiT block runs it: the tensor is the FFN-up GEMM's own output and its amax
    # comes out of that GEMM's epilogue, so no reduction pass precedes the quantize kernel
    from longlive_amd import _native
    ticket = _native.amax_ticket(dev)
    h = fp4_matmul(xq, wq, activation="gelu_tanh", amax_out=ticket)
    for _ in range(3):
        quantize_to_fp4(h, cfg, amax=ticket)
    e0.record()
    for _ in range(reps):
        quantize_to_fp4(h, cfg, amax=ticket)
    e1.record()
    torch.cuda.synchronize()
    qs_ms = e0.elapsed_time(e1) / reps
    qs_gbs = 2.5625 * h.numel() / (qs_ms * 1e-3) / 1e9
    # the same kernel on inputs that cannot be resident in the 256 MB last-level cache: seven copies of the tensor
    # (530 MB) taken in turn, so every launch reads its 75.7 MB from HBM
    rot = [h] + [h.clone() for _ in range(6)]
    for t in rot:
        quantize_to_fp4(t, cfg, amax=ticket)
    e0.record()
    for i in range(reps):
        quantize_to_fp4(rot[i % len(rot)], cfg, amax=ticket)
    e1.record()
    torch.cuda.synchronize()
    qc_ms = e0.elapsed_time(e1) / reps
    qc_gbs = 2.5625 * h.numel() / (qc_ms * 1e-3) / 1e9
    del rot

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
                               "dim 3072, ffn 14336, rule mse, seed 1", "flop_per_step": step_flops(),
                   "prewarm_s": PREWARM_SECONDS, **({} if args.gemm_schedule == "auto" else {"gemm_schedule": args.gemm_schedule})},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_F16_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_F16_TFLOPS,
                     "traffic": live_traffic[0] if live_traffic and live_traffic[0] else measured_traffic_bytes(),
                     "traffic_source": ("rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE in this run" if live_traffic and live_traffic[0]
                                        else "profiles/gemm_w4a4_ffn_up_hbm_traffic.txt"
                                        + (f" (live measurement failed: {live_traffic[1]})" if live_traffic else "")),
                     "kernel": ("gemm_w4a4_asm_kernel<4, 2>" if args.gemm_schedule in ("auto", "tiles") else
                                "gemm_w4a4_kernel<4, 2>" if args.gemm_schedule == "tiles_compiled" else
                                "gemm_w4a4_persistent_kernel") + " M=2640 N=14336 K=3072", "avg_ms": gemm_ms,
                     "frac_of_fp8_peak": achieved / PEAK_FP8_TFLOPS,
                     "note": "peak = dense f16 MFMA, the instruction the exact scheme runs on; frac_of_fp8_peak is the "
                             "same rate against the 5 PFLOP/s dense FP8 figure"},
        "quantize": {"shape": [M_TOKENS, FFN], "avg_ms": q_ms, "GB_per_s": q_gbs, "frac_of_hbm_8TBs": q_gbs / 8000.0,
                     "note": "amax + quantize kernels, 2.5625 algorithmic bytes per element",
                     "amax_from_producer": {"avg_ms": qs_ms, "GB_per_s": qs_gbs, "frac_of_hbm_8TBs": qs_gbs / 8000.0,
                                            "note": "quantize kernel alone on the FFN-up GEMM's output, tensor amax "
                                                    "left behind by that GEMM's epilogue (how the DiT block runs it)"},
                     "cold_inputs": {"avg_ms": qc_ms, "GB_per_s": qc_gbs, "frac_of_hbm_8TBs": qc_gbs / 8000.0,
                                     "note": "the same kernel rotating over seven copies of its input (530 MB, more "
                                             "than the last-level cache), so every launch reads from HBM"}},
    }
    # the same shape of record for the other two hot kernels (the contract's `roofline` stays the GEMM's)
    q_bytes = 2.5625 * h.numel()
    out["roofline_quantize"] = {"bound": "hbm", "achieved": qs_gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                "frac": qs_gbs / PEAK_HBM_GBS, "traffic": q_bytes,
                                "kernel": "quantize_kernel<mse> 2640x14336 (tensor amax from the producer's epilogue)",
                                "avg_ms": qs_ms, "cold_input_frac": qc_gbs / PEAK_HBM_GBS,
                                "with_amax_pass_frac": q_gbs / PEAK_HBM_GBS,
                                "note": "achieved = 2.5625 algorithmic bytes per element / kernel time; traffic = the "
                                        "same bytes (FETCH_SIZE + WRITE_SIZE of the kernel equal them, profiles/)"}
    # what a plain copy reaches on this box in this run: the ceiling any streaming kernel is measured against
    out["roofline_quantize"]["device_copy"] = run_copy(torch, dev, reps)
    if not args.no_extras:
        extras = {}
        for key, fn in (("gemm_shapes", lambda: run_gemm_shapes(torch, dev, work, cfg, 10)),
                        ("attention", lambda: run_attention(torch, dev, 10)), ("block", lambda: run_block(torch, dev, 10)),
                        ("block_release_shapes", lambda: run_block_release(torch, dev, 5)),
                        ("e2e", lambda: run_e2e(torch, dev))):
            try:
                extras[key] = fn()
            except Exception as exc:  # secondary figures must not lose the main line
                extras[key] = {"error": f"{type(exc).__name__}: {exc}"}
            torch.cuda.empty_cache()
        out["extras"] = extras
        att = extras.get("attention", {})
        if "attention_ms" in att:
            out["roofline_attention"] = {"bound": "mfma", "achieved": att["attention_TFLOPs"], "peak": PEAK_F16_TFLOPS,
                                         "unit": "TFLOP/s", "frac": att["attention_TFLOPs"] / PEAK_F16_TFLOPS,
                                         "traffic": None, "kernel": "kv_attention_kernel Lq=2640 Lk=13200 H=24 (configs[2])",
                                         "avg_ms": att["attention_ms"]}
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(work)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
