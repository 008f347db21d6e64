"""GPU parity: NVFP4 quantize / dequantize through the C ABI against the CPU oracle and the golden
vectors.  Bar: bit-exact packed nibbles, scale bytes and amax."""
import numpy as np
import pytest
import torch

import nvfp4_oracle as o
from helpers import activations, bits_of, from_bits, hardware_convert, u8, weights
from longlive_amd import _native
from longlive_amd.fouroversix import QuantizationConfig, QuantizedTensor, quantize_to_fp4

pytestmark = pytest.mark.gpu
RULES = list(o.SCALE_RULES)


def _check(x_bits, rule, dev):
    q = quantize_to_fp4(from_bits(x_bits, dev), QuantizationConfig(scale_rule=rule))
    v, s, a, pad = o.quantize_to_fp4(x_bits, rule)
    assert q.padded_shape == pad
    assert float(q.amax.cpu()) == float(a)
    sg = u8(q.scale_factors)
    assert np.array_equal(sg, s), f"{rule}: {(sg != s).sum()} scale bytes differ"
    vg = u8(q.values)
    assert np.array_equal(vg, v), f"{rule}: {(vg != v).sum()} value bytes differ"
    return q


def test_hardware_e4m3_conversion_matches_software_codec(gpu):
    x = np.concatenate([np.linspace(0, 448, 200001, dtype=np.float32),
                        o.e4m3_decode(np.arange(127, dtype=np.uint8)),
                        np.array([2**-10, 2**-10 * 1.001, 3 * 2**-10, 2**-9 * 2.5, 17.0, 19.0, 27.0], dtype=np.float32)])
    got = hardware_convert(torch.from_numpy(x).to(gpu), 0).cpu().numpy()
    assert np.array_equal(got, o.e4m3_encode(x))


def test_hardware_e2m1_conversion_matches_reference_rounding(gpu):
    x = np.concatenate([np.linspace(-6.9, 6.9, 400001, dtype=np.float32),
                        np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, -0.25, -2.5, -5.0, -0.1, 0.0], dtype=np.float32)])
    got = hardware_convert(torch.from_numpy(x).to(gpu), 1).cpu().numpy()
    ref = o._codes_from_fake_quantized(o._fake_quantize_e2m1(x))
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("rule", RULES)
def test_golden_vectors(golden, gpu, rule):
    for name in golden["case_names"]:
        q = quantize_to_fp4(from_bits(golden[f"{name}/x"], gpu), QuantizationConfig(scale_rule=rule))
        assert float(q.amax.cpu()) == float(golden[f"{name}/{rule}/amax"][0]), name
        assert np.array_equal(u8(q.scale_factors), golden[f"{name}/{rule}/scales"]), name
        assert np.array_equal(u8(q.values), golden[f"{name}/{rule}/values"]), name


@pytest.mark.parametrize("rule", RULES)
@pytest.mark.parametrize("shape,seed", [((128, 64), 0), ((256, 192), 1), ((130, 70), 2), ((1, 16), 3), ((257, 1000), 4)])
def test_random_and_ragged_shapes(gpu, rule, shape, seed):
    _check(bits_of(activations(shape, seed)), rule, gpu)


@pytest.mark.parametrize("rule", ["mse", "static_6"])
def test_input_classes_of_the_reference_test(gpu, rule):
    g = torch.Generator().manual_seed(0)
    for x in (torch.zeros(512, 1024), torch.ones(512, 1024), torch.rand(512, 1024, generator=g),
              torch.randn(1024, 512, generator=g)):
        _check(bits_of(x.bfloat16()), rule, gpu)


def test_edge_values(gpu):
    x = torch.randn(128, 128, generator=torch.Generator().manual_seed(5))
    x[0, :16] = -0.0                      # negative zeros -> code 0
    x[1, :16] = torch.tensor([-1e-4] * 16)  # negatives that round to zero -> code 8
    x[2, :] *= 1e-6                       # blocks with sub-normal / zero e4m3 scales
    x[3, :] *= 3e-5
    x[4, 0] = 250.0                       # sets amax; other blocks far below
    for rule in RULES:
        _check(bits_of(x.bfloat16()), rule, gpu)
    tiny = (torch.randn(128, 64, generator=torch.Generator().manual_seed(6)) * 1e-30).bfloat16()
    huge = (torch.randn(128, 64, generator=torch.Generator().manual_seed(7)) * 1e30).bfloat16()
    for t in (tiny, huge):
        for rule in ("mse", "static_6"):
            _check(bits_of(t), rule, gpu)


def test_benchmark_activation_full_size(gpu):
    """Config 1 activation [2640, 3072], seed 0, rule mse: full-size bit-exact comparison."""
    _check(bits_of(activations((2640, 3072), 0)), "mse", gpu)


@pytest.mark.parametrize("rule", ["mse", "mae"])
def test_ffn_down_activation_full_size_bit_exact(gpu, rule):
    """The activation with the most blocks, [2640, 14336] (2.4 million blocks of 16, the input of the FFN-down
    linear), against the CPU oracle bit for bit: every block whose four-over-six choice the kernel takes from its
    error estimate instead of the reference's arithmetic is one more chance for a wrong confident decision to show."""
    _check(bits_of(activations((2640, 14336), 10)), rule, gpu)


def test_strided_input_and_given_amax(gpu):
    big = activations((200, 512), 8).to(gpu)
    view = big[:, 128:384]  # row stride 512, 256 columns
    q = quantize_to_fp4(view)
    v, s, a, _ = o.quantize_to_fp4(bits_of(view), "mse")
    assert np.array_equal(u8(q.values), v) and np.array_equal(u8(q.scale_factors), s)
    amax = torch.tensor([float(a) * 2], device=gpu)
    vals, sc, am = _native.quantize(view, "mse", amax=amax)
    v2, s2, a2, _ = o.quantize_to_fp4(bits_of(view), "mse", amax=np.float32(float(a) * 2))
    assert np.array_equal(u8(vals), v2) and np.array_equal(u8(sc), s2) and float(am.cpu()) == float(a2)


@pytest.mark.parametrize("rule,factor", [(r, f) for r in ("mse", "mae", "static_6", "abs_max") for f in (1.0, 1.7, 30.0)]
                         + [(r, 0.9) for r in ("mse", "mae", "abs_max")])   # the static rules put the amax itself at 448, the end of e4m3
def test_caller_supplied_amax_bit_exact(gpu, rule, factor):
    """A precomputed amax (quantize/pytorch/reference.py:244) that is the true maximum, larger than it, or a little
    smaller (the blocks above the given amax, here by up to 11 %, get scales above 256 that e4m3 still holds; they
    take the reference's own arithmetic block by block, the others the fast path), against the oracle bit for bit.
    An amax so far below the maximum that block scales leave the e4m3 range (NaN in the reference) is not a
    supported input."""
    x = activations((384, 1024), 23).to(gpu)
    true_amax = float(x.float().abs().max())
    given = np.float32(true_amax * factor)
    vals, sc, am = _native.quantize(x, rule, amax=torch.tensor([given], device=gpu))
    v, s, a, _ = o.quantize_to_fp4(bits_of(x), rule, amax=given)
    assert float(am.cpu()) == float(a) == float(given)
    assert np.array_equal(u8(sc), s)
    assert np.array_equal(u8(vals), v)


def test_rejects_non_bf16_and_cpu_input(gpu):
    with pytest.raises(ValueError, match="bfloat16"):
        quantize_to_fp4(torch.zeros(128, 64, device=gpu))


@pytest.mark.parametrize("rule", ["mse", "static_6", "static_4"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_dequantize_matches_oracle(gpu, rule, dtype):
    x = activations((130, 200), 9)
    q = quantize_to_fp4(x.to(gpu), QuantizationConfig(scale_rule=rule))
    got = q.dequantize(dtype)
    assert got.shape == (130, 200) and got.dtype == dtype
    ref = o.dequantize(u8(q.values), u8(q.scale_factors), np.float32(q.amax.item()), rule, q.padded_shape, (130, 200))
    if dtype == torch.float32:
        assert np.array_equal(got.cpu().numpy(), ref)
    else:
        assert torch.equal(got.cpu(), torch.from_numpy(ref).to(dtype))


def test_dequantize_golden(golden, gpu):
    for name, shape in (("randn_128x512_s1", (128, 512)), ("weights_256x512_s2", (256, 512))):
        v, s, a = (golden[f"{name}/mse/{k}"] for k in ("values", "scales", "amax"))
        qt = QuantizedTensor(torch.from_numpy(v).to(gpu), torch.from_numpy(s).to(gpu).view(torch.float8_e4m3fn),
                             torch.from_numpy(a).to(gpu), "nvfp4", shape, "mse", shape)
        assert np.array_equal(qt.dequantize(torch.float32).cpu().numpy(), golden[f"{name}/mse/deq_f32"])
        assert np.array_equal(bits_of(qt.dequantize(torch.bfloat16)), golden[f"{name}/mse/deq_bf16"])


def test_round_trip_property_at_full_ffn_size(gpu):
    """Size-independent property at the largest benchmark activation [2640, 14336]: dequantize(quantize(x))
    re-quantized with the same amax and a static rule reproduces the same bytes (idempotence), and the
    relative error of the four-over-six result is not worse than plain NVFP4."""
    x = activations((2640, 14336), 10).to(gpu)
    q6 = quantize_to_fp4(x, QuantizationConfig(scale_rule="static_6"))
    d6 = q6.dequantize(torch.float32)
    qm = quantize_to_fp4(x, QuantizationConfig(scale_rule="mse"))
    dm = qm.dequantize(torch.float32)
    e6 = (d6 - x.float()).pow(2).sum().item()
    em = (dm - x.float()).pow(2).sum().item()
    assert em <= e6 * 1.0001
    assert float(qm.amax.cpu()) == float(x.float().abs().max().cpu())
    assert q6.values.shape == (2688, 7168) and not q6.values[2640:].any()


@pytest.mark.parametrize("rule", ["mse", "mae", "abs_max"])
def test_four_over_six_choice_on_ties_and_near_ties(gpu, rule):
    """The kernel decides most blocks from error estimates in units of the block's step and falls back to the
    reference's own arithmetic when the two candidates are close.  Inputs built to make them close or equal:
    values on a coarse lattice (many exact ties), lattice values nudged by one bf16 ulp, blocks repeated at
    many magnitudes, a tensor amax far from the blocks' size, and blocks far below the tensor amax (scale byte 0)."""
    rng = np.random.default_rng(7)
    rows, cols = 1024, 256
    lattice = rng.integers(-12, 13, size=(rows, cols)).astype(np.float32) * 0.25
    nudged = lattice * (1.0 + rng.choice([-2.0 ** -8, 0.0, 2.0 ** -8], size=lattice.shape)).astype(np.float32)
    magn = rng.standard_normal((rows, cols)).astype(np.float32) * np.exp2(rng.integers(-12, 6, size=(rows, 1))).astype(np.float32)
    two_level = np.where(rng.random((rows, cols)) < 0.5, 1.0, 1.5).astype(np.float32) * rng.choice([-1.0, 1.0], size=(rows, cols)).astype(np.float32)
    tiny = rng.standard_normal((rows, cols)).astype(np.float32) * 1e-7
    tiny[0, 0] = 300.0  # tensor amax: the other blocks get scale byte 0 or subnormal scale bytes
    for x in (lattice, nudged, magn, two_level, tiny):
        _check(bits_of(torch.from_numpy(x).bfloat16()), rule, gpu)


@pytest.mark.parametrize("rows,C,rule", [(300, 256, "mse"), (2640, 3072, "mse"), (130, 128, "static_6")])
def test_two_tensors_in_one_launch_equal_the_oracle(gpu, rows, C, rule):
    """The K and V of a chunk go into the cache as one launch (two tensors of one shape, each with the amax its
    producer left in a sink of its own): bytes and amax of both equal the oracle's, i.e. those of two launches."""
    g = torch.Generator().manual_seed(rows + C)
    xs = [(torch.randn(rows, C, generator=g) * s).bfloat16().to(gpu) for s in (1.0, 7.0)]
    sinks = [_native.PrivateAmaxSink(gpu), _native.PrivateAmaxSink(gpu)]
    tickets = [s.ticket() for s in sinks]
    ys = [_native.layer_norm(x, None, None, amax_out=t).reshape(-1, 128) for x, t in zip(xs, tickets)]
    Mp, Kp = _native.padded_shape(tuple(ys[0].shape))
    outs = [(torch.empty((Mp, Kp // 2), dtype=torch.uint8, device=gpu),
             torch.empty(Mp * Kp // 16, dtype=torch.uint8, device=gpu),
             torch.empty(1, dtype=torch.float32, device=gpu)) for _ in range(2)]
    _native.quantize_pair(ys[0], ys[1], rule, tickets[0], tickets[1], outs[0], outs[1])
    for y, (values, scales, amax) in zip(ys, outs):
        v, s, a, _ = o.quantize_to_fp4(bits_of(y), rule)
        assert float(amax.cpu()) == float(a)
        assert np.array_equal(u8(scales), s) and np.array_equal(u8(values), v)
    with pytest.raises(ValueError, match="two sink buffers"):
        t = sinks[0].ticket()
        _native.layer_norm(xs[0], None, None, amax_out=t)
        _native.quantize_pair(ys[0], ys[1], rule, t, t, outs[0], outs[1])
