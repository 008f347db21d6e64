"""GPU parity: the kernels that normalize (adaLN modulation, affine LayerNorm) and quantize to NVFP4 in one launch.
Bar: packed values, scale bytes and amax bit-identical to the separate operations, each of which is pinned to the
CPU oracle by its own tests; the quantization half is also checked against the oracle directly."""
import numpy as np
import pytest
import torch

import nvfp4_oracle as o
from helpers import bits_of, u8
from longlive_amd import _native

pytestmark = pytest.mark.gpu
RULES = list(o.SCALE_RULES)


def _inputs(dev, L, C, frames, seed, outliers=True):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(1, L, C, generator=g) * (0.5 + 3.0 * torch.rand(1, L, 1, generator=g))
    if outliers:  # a few large channels, as a transformer's residual stream has
        x[:, :, torch.randperm(C, generator=g)[:4]] *= 30.0
    e = torch.randn(1, frames, 2, C, generator=g) * 0.5
    x, e = x.to(dev).bfloat16(), e.to(dev).bfloat16()
    return x, e[:, :, 0:1], e[:, :, 1:2]


def _same(got, want, what):
    assert got is not None, f"{what}: the one-launch kernel refused the shape"
    for name, a, b in zip(("values", "scales", "amax"), got, want):
        a, b = (u8(a), u8(b)) if name != "amax" else (a.cpu().numpy(), b.cpu().numpy())
        assert a.shape == b.shape, f"{what} {name}: shape {a.shape} vs {b.shape}"
        assert np.array_equal(a, b), f"{what} {name}: {(a != b).sum()} of {a.size} differ"


def _separate_adaln(x, scale, shift, fs, rule):
    t = _native.amax_ticket(x.device)
    y = _native.adaln_modulate(x, scale, shift, fs, amax_out=t)
    return y, _native.quantize(y.reshape(-1, y.shape[-1]), rule, amax=t)


@pytest.mark.parametrize("L,C,frames,rule", [
    (2640, 3072, 3, "mse"),     # a 3-frame chunk of the benchmark model
    (3072, 3072, 4, "mse"),     # as many rows as the device holds waves of this kernel
    (48, 128, 3, "mae"),        # fewer rows than one tile of the scale layout, rows shorter than a lane's share
    (1000, 2048, 5, "abs_max"),
    (300, 1536, 2, "static_6"),
    (130, 3072, 1, "static_4"),
])
def test_adaln_and_quantize_in_one_launch_match_the_two_operations(gpu, L, C, frames, rule):
    x, scale, shift = _inputs(gpu, L, C, frames, seed=L + C)
    _, want = _separate_adaln(x, scale, shift, L // frames, rule)
    _same(_native.adaln_quantize(x, scale, shift, L // frames, rule), want, f"adaLN {L}x{C} {rule}")


@pytest.mark.parametrize("rule", RULES)
def test_quantization_half_against_the_oracle(gpu, rule):
    """The modulated tensor as the separate kernel writes it, quantized by the CPU oracle, is what the one launch
    gives: the packed bytes do not depend on the device quantizer being right."""
    L, C, frames = 200, 512, 2
    x, scale, shift = _inputs(gpu, L, C, frames, seed=5)
    y = _native.adaln_modulate(x, scale, shift, L // frames)
    v, s, a, _ = o.quantize_to_fp4(bits_of(y[0]), rule)
    got = _native.adaln_quantize(x, scale, shift, L // frames, rule)
    assert got is not None
    assert float(got[2].cpu()) == float(a)
    assert np.array_equal(u8(got[1]), s)
    assert np.array_equal(u8(got[0]), v)


@pytest.mark.parametrize("weight,bias", [(True, True), (True, False), (False, False)])
def test_layer_norm_and_quantize_in_one_launch_match_the_two_operations(gpu, weight, bias):
    L, C = 2640, 3072
    x, _, _ = _inputs(gpu, L, C, 1, seed=11)
    g = torch.Generator().manual_seed(3)
    w = (1.0 + 0.2 * torch.randn(C, generator=g)).to(gpu).bfloat16() if weight else None
    b = (0.1 * torch.randn(C, generator=g)).to(gpu).bfloat16() if bias else None
    t = _native.amax_ticket(gpu)
    y = _native.layer_norm(x, w, b, amax_out=t)
    want = _native.quantize(y.reshape(-1, C), "mse", amax=t)
    _same(_native.layer_norm_quantize(x, w, b, "mse"), want, "LayerNorm")


@pytest.mark.parametrize("spin_limit", [-1, 0])
def test_a_workgroup_that_stops_waiting_computes_the_same_amax(gpu, spin_limit):
    """spin_limit < 0: no workgroup waits for the others, each computes the tensor maximum itself; 0: one look,
    then the same.  Both end normally with the bytes of the ordinary launch."""
    L, C, frames = 2640, 3072, 3
    x, scale, shift = _inputs(gpu, L, C, frames, seed=21)
    _, want = _separate_adaln(x, scale, shift, L // frames, "mse")
    _same(_native.adaln_quantize(x, scale, shift, L // frames, "mse", spin_limit=spin_limit), want, "adaLN alone")
    y = _native.layer_norm(x, None, None)
    _same(_native.layer_norm_quantize(x, None, None, "mse", spin_limit=spin_limit),
          _native.quantize(y.reshape(-1, C), "mse"), "LayerNorm alone")


def test_all_zero_and_constant_rows(gpu):
    L, C = 256, 256
    x = torch.zeros(1, L, C, device=gpu, dtype=torch.bfloat16)
    x[0, 7] = 3.0            # a constant row normalizes to zero as well
    e = torch.zeros(1, 1, 2, C, device=gpu, dtype=torch.bfloat16)
    _, want = _separate_adaln(x, e[:, :, 0:1], e[:, :, 1:2], L, "mse")
    got = _native.adaln_quantize(x, e[:, :, 0:1], e[:, :, 1:2], L, "mse")
    _same(got, want, "zeros")
    assert float(got[2].cpu()) == 0.0 and not u8(got[0]).any()


def test_shapes_the_one_launch_does_not_take_are_left_to_the_separate_operations(gpu):
    for L, C in ((64, 5120), (64, 96), (7040, 3072)):
        x, scale, shift = _inputs(gpu, L, C, 1, seed=1, outliers=False)
        assert _native.adaln_quantize(x, scale, shift, L, "mse") is None
        assert _native.layer_norm_quantize(x, None, None, "mse") is None


def test_one_launch_recorded_into_a_graph_replays_with_fresh_inputs(gpu):
    """The launch allocates nothing and its epochs advance with the sink's device word, so a recording replays;
    every replay is checked against the eager result, with eager work and synchronization between replays."""
    L, C, frames = 880, 3072, 1
    x, scale, shift = _inputs(gpu, L, C, frames, seed=31)
    sink = _native.ReplayableAmaxSink(gpu)
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        _native.adaln_quantize(x, scale, shift, L, "mse")  # first use outside the recording
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=stream), sink:
            recorded = _native.adaln_quantize(x, scale, shift, L, "mse")
    for seed in (41, 42, 43):
        xn, sn, hn = _inputs(gpu, L, C, frames, seed=seed)
        x.copy_(xn), scale.copy_(sn), shift.copy_(hn)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        _, want = _separate_adaln(x, scale, shift, L, "mse")
        torch.cuda.synchronize()
        _same(recorded, want, f"replay with seed {seed}")


def test_results_hold_while_another_stream_occupies_the_device(gpu):
    """Large matrix products on a side stream compete for the compute units while the one-launch kernel runs: its
    workgroups then do not all start together, some give up waiting and compute the missing rows' maxima
    themselves.  Every launch ends and every result equals the two-launch bytes."""
    L, C, frames = 2640, 3072, 3
    x, scale, shift = _inputs(gpu, L, C, frames, seed=51)
    _, want = _separate_adaln(x, scale, shift, L // frames, "mse")
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    a = torch.randn(8192, 8192, device=gpu, dtype=torch.bfloat16)
    with torch.cuda.stream(side):
        for _ in range(40):
            a @ a
    results = [_native.adaln_quantize(x, scale, shift, L // frames, "mse", spin_limit=2) for _ in range(40)]
    torch.cuda.synchronize()
    for i, got in enumerate(results):
        _same(got, want, f"launch {i} beside the side stream")


def test_batches_of_two_with_strided_scale_and_shift(gpu):
    """B = 2: scale / shift rows are picked by (batch, frame); they arrive as strided views of one [B, F, 6, C]
    tensor, as the block passes them."""
    B, L, C, frames = 2, 192, 512, 3
    g = torch.Generator().manual_seed(61)
    x = (torch.randn(B, L, C, generator=g) * 2).to(gpu).bfloat16()
    e = (torch.randn(B, frames, 6, C, generator=g) * 0.5).to(gpu).bfloat16()
    scale, shift = e[:, :, 4:5], e[:, :, 3:4]
    t = _native.amax_ticket(gpu)
    y = _native.adaln_modulate(x, scale, shift, L // frames, amax_out=t)
    want = _native.quantize(y.reshape(-1, C), "mse", amax=t)
    _same(_native.adaln_quantize(x, scale, shift, L // frames, "mse"), want, "B = 2")
