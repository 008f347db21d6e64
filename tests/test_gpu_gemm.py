"""GPU parity: W4A4 GEMM and the quantized Linear against the oracle's dequantize-then-fp32-matmul.
Bar (floating point): relative Frobenius error <= 1e-3."""
import os

import numpy as np
import pytest
import torch
import torch.nn as nn

import nvfp4_oracle as o
from helpers import activations, bits_of, from_bits, u8, weights
from longlive_amd import _native
from longlive_amd.fouroversix import (FourOverSixLinear, ModelQuantizationConfig, QuantizationConfig,
                                      QuantizedTensor, fp4_matmul, quantize_to_fp4)
from longlive_amd.utils.quant import quantize_model_with_filter

pytestmark = pytest.mark.gpu
TOL = 1e-3


def _as_oracle(q):
    return dict(values=u8(q.values), scales=u8(q.scale_factors), amax=np.float32(q.amax.item()),
                rule=q.scale_rule.value, padded=q.padded_shape, orig=q.original_shape)


def _rel(a, b):
    return float(np.linalg.norm(a.astype(np.float64) - b.astype(np.float64)) / max(np.linalg.norm(b.astype(np.float64)), 1e-30))


def test_integer_special_case_is_exact(gpu):
    """Unit scales and amax = 1536: the product is an exact integer-valued matrix (bf16-representable
    here because entries stay below 256 in magnitude for K = 64 of small codes)."""
    rng = np.random.default_rng(0)
    ca = rng.integers(0, 4, (128, 64)).astype(np.uint8) | (rng.integers(0, 2, (128, 64)).astype(np.uint8) << 3)
    cb = rng.integers(0, 4, (128, 64)).astype(np.uint8) | (rng.integers(0, 2, (128, 64)).astype(np.uint8) << 3)
    va = (ca[:, 0::2] | (ca[:, 1::2] << 4)).astype(np.uint8)
    vb = (cb[:, 0::2] | (cb[:, 1::2] << 4)).astype(np.uint8)
    sc = torch.full((128 * 4,), 0x38, dtype=torch.uint8, device=gpu)
    amax = torch.tensor([1536.0], device=gpu)
    y = _native.gemm(torch.from_numpy(va).to(gpu), sc, torch.from_numpy(vb).to(gpu), sc, 128, 128, amax_a=amax, amax_b=amax)
    expect = o.E2M1_VALUES[ca].astype(np.float64) @ o.E2M1_VALUES[cb].astype(np.float64).T
    assert np.array_equal(y.float().cpu().numpy().astype(np.float64), expect)


def test_golden_matmul(golden, gpu):
    def qt(name, shape):
        v, s, a = (golden[f"{name}/mse/{k}"] for k in ("values", "scales", "amax"))
        return QuantizedTensor(torch.from_numpy(v).to(gpu), torch.from_numpy(s).to(gpu).view(torch.float8_e4m3fn),
                               torch.from_numpy(a).to(gpu), "nvfp4", shape, "mse", shape)

    y = fp4_matmul(qt("randn_128x512_s1", (128, 512)), qt("weights_256x512_s2", (256, 512)))
    ref = o.bf16_to_f32(golden["matmul/randn_128x512_s1__weights_256x512_s2/mse/out_bf16"])
    assert _rel(y.float().cpu().numpy(), ref) <= TOL
    got = y.float().cpu().numpy()
    # elementwise: one bf16 ulp of the value plus fp32 summation-order noise of a K = 512 dot product
    assert (np.abs(got - ref) <= 2.0 ** -7 * np.abs(ref) + 1e-4 * np.abs(ref).max()).all()


@pytest.mark.parametrize("M,N,K,seed", [(128, 128, 64, 0), (200, 192, 256, 1), (130, 70, 200, 2), (1, 3072, 128, 3),
                                        (640, 384, 1152, 4), (300, 1000, 3072, 5), (96, 160, 320, 6), (257, 129, 192, 7)])
def test_against_oracle(gpu, M, N, K, seed):
    x, w = activations((M, K), seed), weights((N, K), seed + 100)
    xq, wq = quantize_to_fp4(x.to(gpu)), quantize_to_fp4(w.to(gpu))
    y = fp4_matmul(xq, wq)
    assert y.shape == (M, N) and y.dtype == torch.bfloat16
    ref = o.fp4_matmul(_as_oracle(xq), _as_oracle(wq))
    assert _rel(y.float().cpu().numpy(), ref) <= TOL


def test_mixed_scale_rules_and_explicit_alpha(gpu):
    x, w = activations((128, 256), 6), weights((256, 256), 7)
    xq = quantize_to_fp4(x.to(gpu), QuantizationConfig(scale_rule="static_6"))
    wq = quantize_to_fp4(w.to(gpu), QuantizationConfig(scale_rule="mse"))
    ref = o.fp4_matmul(_as_oracle(xq), _as_oracle(wq))
    assert _rel(fp4_matmul(xq, wq).float().cpu().numpy(), ref) <= TOL
    alpha = (xq.amax * wq.amax / (2688.0 * 1536.0)).float()
    y = _native.gemm(xq.values, xq.scale_factors, wq.values, wq.scale_factors, 128, 256, alpha=alpha)
    assert _rel(y.float().cpu().numpy(), ref) <= TOL


def _exact_product(xq, wq):
    """The product of the two quantized operands in float64 (no rounding that matters: every factor has at most
    6 significant bits times an fp32 tensor scale), and sum |a||b| for the accumulation bound."""
    def operand(q):
        d = _as_oracle(q)
        Mp, Kp = d["padded"]
        v = o.unpack_e2m1(d["values"]).astype(np.float64)
        s = o.e4m3_decode(o.from_blocked(d["scales"], (Mp, Kp // 16))).astype(np.float64)
        e2, e4 = o.rule_limits(d["rule"])
        return (v * np.repeat(s, 16, axis=1) * float(d["amax"]) / (e2 * e4))[: d["orig"][0], : d["orig"][1]]
    a, b = operand(xq), operand(wq)
    return a @ b.T, np.abs(a) @ np.abs(b).T


@pytest.mark.parametrize("M,N,K,kind,seed", [(130, 1, 16, "tie", 0), (64, 128, 64, "tie", 1), (100, 72, 16, "lattice", 2),
                                             (513, 200, 2048, "tie", 3), (257, 129, 320, "lattice", 4),
                                             (300, 256, 1024, "gauss", 5)])
def test_every_output_is_the_exact_product_rounded_once(gpu, M, N, K, kind, seed):
    """Element-wise bar, tighter than the relative Frobenius norm: each bf16 output lies within half a bf16 ulp of
    the exact product of the quantized operands, plus the fp32 accumulation error (K * 2^-23 * sum |a||b|).  The
    "tie" inputs make one product dominate whose exact value (3 * bf16(0.06)) is a bf16 rounding tie, and the
    lattice inputs produce many such ties: there the fp32 dequantize-then-matmul of the reference may round the
    other way and differ by a whole ulp, so agreement with it in the norm alone would say nothing."""
    g = torch.Generator().manual_seed(seed)
    def make(rows, cols):
        if kind == "tie":
            t = torch.randn(rows, cols, generator=g) * 1e-4
            t[0, 0] = 3.0
        elif kind == "lattice":
            t = torch.randint(-12, 13, (rows, cols), generator=g).float() * 0.25
        else:
            t = torch.randn(rows, cols, generator=g)
        return t
    x, w = make(M, K).bfloat16(), (make(N, K) * 0.02).bfloat16()
    xq, wq = quantize_to_fp4(x.to(gpu)), quantize_to_fp4(w.to(gpu))
    y = fp4_matmul(xq, wq).float().cpu().numpy().astype(np.float64)
    exact, mass = _exact_product(xq, wq)
    top = np.maximum(np.abs(y), np.abs(exact))
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(top, 2.0 ** -126))) - 7)
    bound = 0.5 * ulp + K * 2.0 ** -23 * mass + 2.0 ** -133
    worst = ((np.abs(y - exact) - bound) / ulp).max()
    assert worst <= 0, f"an output is {worst:.3f} bf16 ulp beyond the bound"


def test_high_precision_operands_are_quantized_on_the_fly(gpu):
    x, w = activations((128, 128), 8).to(gpu), weights((128, 128), 9).to(gpu)
    y1 = fp4_matmul(x, w)
    y2 = fp4_matmul(quantize_to_fp4(x), quantize_to_fp4(w))
    assert torch.equal(y1, y2)


def test_config1_single_linear_full_size(gpu):
    """Benchmark configuration 1: X [2640, 3072] seed 0 with outliers, W [3072, 3072] ~ N(0, 0.02), rule mse."""
    x, w = activations((2640, 3072), 0), weights((3072, 3072), 0)
    xq, wq = quantize_to_fp4(x.to(gpu)), quantize_to_fp4(w.to(gpu))
    y = fp4_matmul(xq, wq)
    ref = o.fp4_matmul(_as_oracle(xq), _as_oracle(wq))
    r = _rel(y.float().cpu().numpy(), ref)
    assert r <= TOL, r


def test_ffn_shapes_linearity_property(gpu):
    """Benchmark configuration 2, FFN shapes (too large for a CPU matmul in a unit test): the GEMM is linear in
    the tensor scale of A, so doubling amax_a doubles every output exactly (power of two), and rows of
    A that are zero give zero rows."""
    _ffn_shape_checks(gpu, ((2640, 14336, 3072), (2640, 3072, 14336)))


def test_release_chunk_shapes_linearity_property(gpu):
    """The same checks at the token count of the reference's released configuration (chunks of 8 frames =
    7040 tokens, configs/nvfp4/inference_nvfp4.yaml:5): 55 row tiles of 128 or 27.5 of 256, so other tile
    choices and a ragged last row tile."""
    _ffn_shape_checks(gpu, ((7040, 3072, 3072), (7040, 14336, 3072), (7040, 3072, 14336)))


def _ffn_shape_checks(gpu, shapes):
    for M, N, K in shapes:
        x, w = activations((M, K), 1).to(gpu), weights((N, K), 1).to(gpu)
        x[5] = 0
        xq, wq = quantize_to_fp4(x), quantize_to_fp4(w)
        y = fp4_matmul(xq, wq)
        assert y.shape == (M, N) and torch.isfinite(y.float()).all()
        assert not y[5].any()
        y2 = _native.gemm(xq.values, xq.scale_factors, wq.values, wq.scale_factors, M, N, amax_a=xq.amax * 2,
                          amax_b=wq.amax)
        assert torch.equal(y2.float(), y.float() * 2)
        # spot-check 64 rows against the oracle
        rows = torch.arange(0, M, M // 64)[:64]
        a = _as_oracle(xq)
        b = _as_oracle(wq)
        A = o.dequantize(a["values"], a["scales"], a["amax"], "mse", a["padded"], a["orig"])[rows.numpy()]
        B = o.dequantize(b["values"], b["scales"], b["amax"], "mse", b["padded"], b["orig"])
        ref = o.round_bf16(A @ B.T)
        assert _rel(y[rows.to(gpu)].float().cpu().numpy(), ref) <= TOL


def test_linear_module_with_bias_matches_reference_semantics(gpu):
    torch.manual_seed(0)
    lin = nn.Linear(256, 384, bias=True).to(gpu).bfloat16()
    model = nn.Sequential(lin)
    model, _ = quantize_model_with_filter(model, ModelQuantizationConfig(), materialize_for_inference=True, verbose=False)
    q = model[0]
    assert isinstance(q, FourOverSixLinear) and q.weight is None
    x = activations((2, 50, 256), 3).to(gpu)
    with torch.no_grad():
        y = q(x)
    assert y.shape == (2, 50, 384)
    xq = quantize_to_fp4(x.reshape(-1, 256))
    ref = o.fp4_matmul(_as_oracle(xq), _as_oracle(q.quantized_weight()))
    ref = o.round_bf16(ref + q.bias.detach().float().cpu().numpy()[None, :])  # bf16 add after the bf16 GEMM result
    got = y.reshape(-1, 384).float().cpu().numpy()
    assert _rel(got, ref) <= TOL
    # state-dict round trip: packed buffers reload into a fresh swapped module (out_features is a
    # multiple of 128, as for every Wan linear, so the registered buffer shapes equal the padded ones)
    fresh = nn.Sequential(nn.Linear(256, 384, bias=True).to(gpu).bfloat16())
    fresh, _ = quantize_model_with_filter(fresh, ModelQuantizationConfig(), verbose=False)
    fresh[0].weight = None
    fresh.load_state_dict(model.state_dict(), strict=True)
    with torch.no_grad():
        assert torch.equal(fresh[0](x), y)


def test_gelu_epilogue_matches_separate_gelu(gpu):
    """The GEMM with the GELU(tanh) epilogue against the plain GEMM followed by torch's GELU on the bf16
    result: the same function evaluated as x / (1 + exp(-2u)) instead of 0.5 x (1 + tanh(u)), so results may
    differ by one bf16 ulp on a small fraction of the elements."""
    from longlive_amd.fouroversix import QuantizationConfig, fp4_matmul, quantize_to_fp4
    cfg = QuantizationConfig(scale_rule="mse")
    x = activations((300, 512), 31).to(gpu)
    w = (weights((640, 512), 32) * 40).to(gpu)  # outputs spread over roughly [-8, 8]
    bias = (torch.randn(640, generator=torch.Generator().manual_seed(33)) * 0.5).bfloat16().to(gpu)
    xq, wq = quantize_to_fp4(x, cfg), quantize_to_fp4(w, cfg)
    plain = fp4_matmul(xq, wq, bias=bias)
    fused = fp4_matmul(xq, wq, bias=bias, activation="gelu_tanh")
    want = torch.nn.functional.gelu(plain, approximate="tanh")
    assert plain.float().abs().max() > 4
    # one bf16 ulp where the result is not tiny; far in the negative tail 1 + tanh cancels in torch's formula
    # and the two evaluations differ relatively (not absolutely): results there are below 1e-5
    f, w_ = fused.float(), want.float()
    assert bool(((f - w_).abs() <= torch.maximum(w_.abs() * 2 ** -7, torch.tensor(2e-6, device=gpu))).all())
    body = plain.float().abs() < 3
    assert float((f[body] != w_[body]).float().mean()) < 0.02
    # the oracle's formula in float64
    ref = o.gelu_tanh(plain.float().cpu().numpy().astype(np.float64))
    assert np.abs(fused.float().cpu().numpy() - ref).max() <= 2 ** -8 * max(1.0, np.abs(ref).max())
    with pytest.raises(ValueError):
        fp4_matmul(xq, wq, activation="relu")


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K,frame", [(264, 384, 256, 88), (300, 640, 512, 100), (64, 72, 128, 16)])
def test_gated_residual_epilogue_is_bit_identical_to_the_separate_operations(gpu, M, N, K, frame):
    """residual + y * gate and residual + y inside the GEMM epilogue against the GEMM followed by the two
    bf16 operations of the reference (causal_model.py:889, 906), which the oracle restates."""
    from longlive_amd.fouroversix import QuantizationConfig, fp4_matmul, quantize_to_fp4
    cfg = QuantizationConfig(scale_rule="mse")
    x = activations((M, K), 41).to(gpu)
    w = weights((N, K), 42).to(gpu)
    gen = torch.Generator().manual_seed(43)
    bias = (torch.randn(N, generator=gen) * 0.5).bfloat16().to(gpu)
    residual = torch.randn(M, N, generator=gen).bfloat16().to(gpu)
    frames = M // frame
    e = torch.randn(frames, 6, N, generator=gen).bfloat16().to(gpu)
    gate = e[:, 2]  # rows strided by 6 N, as the chunked modulation tensor of the block hands them over
    xq, wq = quantize_to_fp4(x, cfg), quantize_to_fp4(w, cfg)
    plain = fp4_matmul(xq, wq, bias=bias)
    fused = fp4_matmul(xq, wq, bias=bias, residual=residual, gate=gate, gate_rows=frame)
    want = o.gate_residual(residual.float().cpu().numpy(), plain.float().cpu().numpy(), gate.float().cpu().numpy(),
                           frame)
    assert np.array_equal(fused.float().cpu().numpy(), want)
    assert torch.equal(fused, residual + (plain.view(frames, frame, N) * gate[:, None]).view(M, N))
    summed = fp4_matmul(xq, wq, bias=bias, residual=residual)
    assert torch.equal(summed, residual + plain)
    with pytest.raises(ValueError):
        fp4_matmul(xq, wq, gate=gate, gate_rows=frame)


@pytest.mark.gpu
def test_amax_sink_of_the_epilogue_feeds_the_next_quantization(gpu):
    """The absolute maximum a GEMM leaves in the amax sink makes the following quantization produce the bytes
    of a quantization that reduces the tensor itself; a later use of the sink with smaller values is not
    disturbed by what earlier epochs left there."""
    from longlive_amd import _native
    from longlive_amd.fouroversix import QuantizationConfig, fp4_matmul, quantize_to_fp4
    cfg = QuantizationConfig(scale_rule="mse")
    x = activations((300, 512), 51).to(gpu)
    wq = quantize_to_fp4(weights((640, 512), 52).to(gpu), cfg)
    for scale in (8.0, 1.0, 0.01):  # decreasing maxima: stale slots of older epochs hold larger values
        xq = quantize_to_fp4(x * scale, cfg)
        for act in (None, "gelu_tanh"):
            ticket = _native.amax_ticket(gpu)
            y = fp4_matmul(xq, wq, activation=act, amax_out=ticket)
            via_sink = quantize_to_fp4(y, cfg, amax=ticket)
            direct = quantize_to_fp4(y, cfg)
            assert torch.equal(via_sink.amax, direct.amax) and float(direct.amax) == float(y.abs().max())
            assert torch.equal(via_sink.values, direct.values)
            assert torch.equal(via_sink.scale_factors.view(torch.uint8), direct.scale_factors.view(torch.uint8))


@pytest.mark.parametrize("M,N,K,n", [(264, 384, 256, 3), (300, 200, 192, 2), (64, 128, 64, 4), (2640, 3072, 3072, 3),
                                     (512, 3072, 3072, 2)])
def test_products_that_share_their_input_in_one_launch_equal_the_separate_launches(gpu, M, N, K, n):
    """ll_nvfp4_gemm_tnt_grouped (the q / k / v projections of one activation): every product - own weight, tensor
    scale, bias and amax sink - is bit for bit what the single call computes, at ragged and at full sizes; the
    quantized linear layers take that path through forward_quantized_together.  (With one summation order for every
    shape: a single 2640 x 3072 product would otherwise take the kernel that sums the halves of K separately,
    three of them in one launch the large tiles.)"""
    from longlive_amd import _native
    with _native.gemm_schedule("tiles_compiled"):
        _grouped_equals_separate(gpu, M, N, K, n)


def _grouped_equals_separate(gpu, M, N, K, n):
    cfg = QuantizationConfig(scale_rule="mse")
    xq = quantize_to_fp4(activations((M, K), 61).to(gpu), cfg)
    ws = [quantize_to_fp4((weights((N, K), 62 + i) * (1 + i)).to(gpu), cfg) for i in range(n)]
    biases = [None if i == 1 else (torch.randn(N, generator=torch.Generator().manual_seed(70 + i)) * 0.1).bfloat16().to(gpu)
              for i in range(n)]
    alone, alone_tickets = [], []
    for w, b in zip(ws, biases):
        t = _native.amax_ticket(gpu)
        y = fp4_matmul(xq, w, bias=b, amax_out=t)
        alone.append(y)
        alone_tickets.append(float(quantize_to_fp4(y, cfg, amax=t).amax))
    tickets = [_native.PrivateAmaxSink(gpu) for _ in range(n)]   # each product needs a sink of its own here: one launch
    products = [dict(values=w.values, scales=w.scale_factors, amax=w.amax, denom=1536.0, bias=b, amax_out=s.ticket())
                for w, b, s in zip(ws, biases, tickets)]
    together = _native.gemm_grouped(xq.values, xq.scale_factors, xq.amax, 1536.0, M, N, products)
    for i in range(n):
        assert torch.equal(together[i], alone[i]), i
        got = float(quantize_to_fp4(together[i], cfg, amax=products[i]["amax_out"]).amax)
        assert got == alone_tickets[i] == float(alone[i].abs().max())
    with pytest.raises(ValueError):     # more than four products
        _native.gemm_grouped(xq.values, xq.scale_factors, xq.amax, 1536.0, M, N, [dict(p, amax_out=None) for p in products] * 3)
    with pytest.raises(ValueError):     # two products on one sink buffer
        _native.gemm_grouped(xq.values, xq.scale_factors, xq.amax, 1536.0, M, N,
                             [dict(p, amax_out=tickets[0].ticket()) for p in products[:2]])


def test_quantized_layers_with_one_input_run_as_one_launch(gpu):
    lin = [nn.Linear(256, 384).to(gpu).bfloat16() for _ in range(3)]
    holder = nn.Sequential(*lin)
    holder, _ = quantize_model_with_filter(holder, ModelQuantizationConfig(), use_default_filtered_modules=False,
                                           materialize_for_inference=True, verbose=False)
    layers = list(holder)
    assert all(isinstance(m, FourOverSixLinear) for m in layers)
    x = activations((130, 256), 81).to(gpu)
    xq = layers[0].quantize_input(x)
    together = FourOverSixLinear.forward_quantized_together(layers, xq)
    for m, y in zip(layers, together):
        assert torch.equal(y, m.forward_quantized(xq)) and torch.equal(y, m(x))


@pytest.mark.gpu
def test_ffn_down_full_size_fused_epilogue_and_sink(gpu):
    """The FFN pair at the benchmark size: GELU + amax sink in the up projection, gated residual in the down
    projection, against the same GEMMs followed by the separate operations (bit-identical), and the sink-fed
    quantization against the one that reduces the tensor itself (identical bytes)."""
    from longlive_amd import _native
    from longlive_amd.fouroversix import QuantizationConfig, fp4_matmul, quantize_to_fp4
    cfg = QuantizationConfig(scale_rule="mse")
    M, D, F, frame = 2640, 3072, 14336, 880
    x = activations((M, D), 61).to(gpu)
    w_up, w_down = quantize_to_fp4(weights((F, D), 62).to(gpu), cfg), quantize_to_fp4(weights((D, F), 63).to(gpu), cfg)
    gen = torch.Generator().manual_seed(64)
    residual = torch.randn(M, D, generator=gen).bfloat16().to(gpu)
    gate = torch.randn(M // frame, 6, D, generator=gen).bfloat16().to(gpu)[:, 5]
    xq = quantize_to_fp4(x, cfg)
    ticket = _native.amax_ticket(gpu)
    h = fp4_matmul(xq, w_up, activation="gelu_tanh", amax_out=ticket)
    assert torch.equal(h, fp4_matmul(xq, w_up, activation="gelu_tanh"))
    hq, hq_ref = quantize_to_fp4(h, cfg, amax=ticket), quantize_to_fp4(h, cfg)
    assert torch.equal(hq.amax, hq_ref.amax) and torch.equal(hq.values, hq_ref.values)
    assert torch.equal(hq.scale_factors.view(torch.uint8), hq_ref.scale_factors.view(torch.uint8))
    y = fp4_matmul(hq, w_down)
    fused = fp4_matmul(hq, w_down, residual=residual, gate=gate, gate_rows=frame)
    assert torch.equal(fused, residual + (y.view(M // frame, frame, D) * gate[:, None]).view(M, D))


# --------------------------------------------------------------------------- reference-written module state
def _fixture_state(fx, name, device):
    state = {}
    for key in fx[f"{name}/state_keys"]:
        arr, dt = fx[f"{name}/state/{key}"], str(fx[f"{name}/state_dtype/{key}"])
        if dt == "torch.bfloat16":
            t = torch.from_numpy(arr.view(np.int16).copy()).view(torch.bfloat16)
        elif dt == "torch.float8_e4m3fn":
            t = torch.from_numpy(arr.copy()).view(torch.float8_e4m3fn)
        else:
            t = torch.from_numpy(arr.copy())
        state[str(key)] = t.to(device)
    return state


@pytest.mark.parametrize("name", ["aligned_192x128", "padded_128x96"])
def test_state_dict_written_by_the_reference_module_loads_and_runs(gpu, name):
    """tests/golden/fouroversix_linear_state.npz holds the state dict of the reference's own FourOverSixLinear
    (fouroversix/src/fouroversix/model/modules/linear.py:182-216, 271-307; written by
    tests/golden/make_linear_golden.py) for two nn.Linear layers, one of them with an output dimension that is not a
    multiple of 128, and the reference's forward on a fixed input.  (1) Quantizing the same master weight with this
    package gives the same buffers, bit for bit.  (2) The reference's state dict loads into this package's module
    with strict=True.  (3) The forward on the loaded module matches the reference's output (relative Frobenius
    <= 1e-3, the GEMM bar) and the oracle's."""
    from longlive_amd.fouroversix import FourOverSixLinear, ModuleQuantizationConfig
    from longlive_amd.utils.quant import _materialize_quantized_weights_for_inference

    fx = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fouroversix_linear_state.npz"))
    assert name in list(fx["case_names"])
    w = from_bits(fx[f"{name}/weight"], gpu)
    fout, fin = w.shape

    def fresh(weight, bias):
        lin = torch.nn.Linear(fin, fout, bias=True).to(gpu).to(torch.bfloat16)
        with torch.no_grad():
            lin.weight.copy_(weight)
            lin.bias.copy_(bias)
        mod = FourOverSixLinear(lin, ModuleQuantizationConfig(scale_rule="mse"))
        assert sorted(mod.state_dict().keys()) == sorted(str(k) for k in fx[f"{name}/registered_keys"])
        for k, v in mod.state_dict().items():
            assert tuple(v.shape) == tuple(fx[f"{name}/registered_shape/{k}"]), k
        holder = torch.nn.Sequential(mod)
        _materialize_quantized_weights_for_inference(holder)
        return holder[0]

    ref_state = _fixture_state(fx, name, gpu)
    # (1) own quantization of the same weight
    own = fresh(w, from_bits(fx[f"{name}/bias"], gpu))
    own_state = own.state_dict()
    assert sorted(own_state.keys()) == sorted(ref_state.keys())
    for k, v in ref_state.items():
        a, b = own_state[k], v
        assert a.dtype == b.dtype and a.numel() == b.numel(), k
        assert torch.equal(a.reshape(-1).view(torch.uint8), b.reshape(-1).view(torch.uint8)), k
    # (2) strict load into a module built from other weights
    other = fresh(torch.zeros_like(w), torch.zeros(fout, dtype=torch.bfloat16, device=gpu))
    result = other.load_state_dict(ref_state, strict=True)
    assert not result.missing_keys and not result.unexpected_keys
    # the same into a freshly swapped module whose master weight was dropped without quantizing it: its buffers
    # still have the registered (unpadded) shapes, the load brings them to the checkpoint's
    lin = torch.nn.Linear(fin, fout, bias=True).to(gpu).to(torch.bfloat16)
    bare = FourOverSixLinear(lin, ModuleQuantizationConfig(scale_rule="mse"))
    bare.register_parameter("weight", None)
    result = bare.load_state_dict(ref_state, strict=True)
    assert not result.missing_keys and not result.unexpected_keys
    for k, v in ref_state.items():
        assert torch.equal(bare.state_dict()[k].reshape(-1).view(torch.uint8), v.reshape(-1).view(torch.uint8)), k
    # (3) forward
    x = from_bits(fx[f"{name}/x"], gpu)
    with torch.no_grad():
        y = other(x)
        y_own = own(x)
        assert torch.equal(bare(x), y)
    assert torch.equal(y, y_own)
    y_ref = from_bits(fx[f"{name}/y"]).float().numpy()
    got = y.float().cpu().numpy()
    assert got.shape == y_ref.shape
    assert np.linalg.norm(got - y_ref) / np.linalg.norm(y_ref) <= 1e-3
    xv, xs, xa, xpad = o.quantize_to_fp4(fx[f"{name}/x"], "mse")
    qw = other.quantized_weight()
    oy = o.fp4_matmul(dict(values=xv, scales=xs, amax=xa, rule="mse", padded=xpad, orig=fx[f"{name}/x"].shape),
                      dict(values=u8(qw.values), scales=u8(qw.scale_factors), amax=np.float32(qw.amax.item()),
                           rule="mse", padded=tuple(qw.padded_shape), orig=tuple(qw.original_shape)))
    oy = o.round_bf16(oy + from_bits(fx[f"{name}/bias"]).float().numpy()[None, :])
    assert np.linalg.norm(got - oy) / np.linalg.norm(oy) <= 1e-3


def _ulp_close(a, b, frac=1e-3):
    """Two bf16 results of the same fp32 sums added up in another order: equal except where the fp32 sums round to
    neighbouring bf16 values, on a small fraction of the elements."""
    a, b = a.float(), b.float()
    diff = (a - b).abs()
    assert bool((diff <= torch.maximum(a.abs(), b.abs()) * 2 ** -7 + 1e-30).all())
    assert float((diff != 0).float().mean()) <= frac


@pytest.mark.parametrize("M,N,K,groups", [
    (2640, 3072, 3072, 1),    # the projections of the DiT block: 252 tiles of 128 x 256
    (2640, 3072, 14336, 1),   # FFN-down
    (1300, 5000, 640, 1),     # ragged M and N (waves without output rows), five K steps
    (2100, 2100, 512, 1),     # waves without output columns, four K steps
    (880, 3072, 1024, 3),     # three products in one launch
])
def test_one_workgroup_per_unit_with_k_split_between_its_halves(gpu, M, N, K, groups):
    """Shapes that give at most one 128 x 256 tile per compute unit (and fill more than half of the units) run as
    one workgroup of eight waves per tile, the two halves of every K step summed separately and added through LDS:
    the same exact products as the other tile kernels added in another order.  Against the compiled kernel within
    one bf16 ulp of the fp32 sum, twice for identical bits, against the oracle (1e-3 relative Frobenius) where it
    finishes in seconds; bias, GELU, gated residual and the amax sinks go through the same epilogue."""
    cfg = QuantizationConfig(scale_rule="mse")
    xq = quantize_to_fp4(activations((M, K), 15).to(gpu), cfg)
    ws = [quantize_to_fp4((weights((N, K), 16 + i) * (1 + i)).to(gpu), cfg) for i in range(groups)]
    gen = torch.Generator().manual_seed(17)
    bias = (torch.randn(N, generator=gen) * 0.1).to(gpu).bfloat16()
    frame = M // 4 if M % 4 == 0 else M
    residual = torch.randn(M, N, generator=gen).bfloat16().to(gpu)
    gate = torch.randn(M // frame, 6, N, generator=gen).bfloat16().to(gpu)[:, 2]
    out = {}
    for sched in ("tiles_compiled", "tiles", "tiles"):
        with _native.gemm_schedule(sched):
            if groups == 1:
                t = _native.amax_ticket(gpu)
                y = [fp4_matmul(xq, ws[0], bias=bias, activation="gelu_tanh", amax_out=t)]
                amax = [float(quantize_to_fp4(y[0], cfg, amax=t).amax)]
                if N % 8 == 0:
                    y.append(fp4_matmul(xq, ws[0], bias=bias, residual=residual, gate=gate, gate_rows=frame))
                y.append(fp4_matmul(xq, ws[0]))
            else:
                sinks = [_native.PrivateAmaxSink(gpu) for _ in range(groups)]
                products = [dict(values=w.values, scales=w.scale_factors, amax=w.amax, denom=1536.0, bias=bias if i != 1 else None,
                                 amax_out=s.ticket()) for i, (w, s) in enumerate(zip(ws, sinks))]
                y = list(_native.gemm_grouped(xq.values, xq.scale_factors, xq.amax, 1536.0, M, N, products))
                amax = [float(quantize_to_fp4(yi, cfg, amax=pr["amax_out"]).amax) for yi, pr in zip(y, products)]
        out.setdefault(sched, []).append((y, amax))
    (want, _), = out["tiles_compiled"]
    (got, amax), (again, amax_again) = out["tiles"]
    for a, b in zip(got, again):
        assert torch.equal(a, b)
    assert amax == amax_again
    for a, b in zip(got, want):
        _ulp_close(a, b, frac=5e-3)
    n_sinks = 1 if groups == 1 else groups
    assert amax == [float(yi.float().abs().max()) for yi in got[:n_sinks]]
    if M * N * K <= 3e10 and groups == 1:
        ref = o.fp4_matmul(_as_oracle(xq), _as_oracle(ws[0]))
        assert _rel(got[-1].float().cpu().numpy(), ref) <= TOL


def test_eight_wave_kernel_recorded_into_a_graph(gpu):
    """The eight-wave kernel allocates nothing and waits for no other workgroup: recorded into a graph it replays
    with fresh operands, every replay equal to the eager result bit for bit."""
    cfg = QuantizationConfig(scale_rule="mse")
    M, N, K = 2640, 3072, 1024
    x = activations((M, K), 61).to(gpu)
    wq = quantize_to_fp4(weights((N, K), 62).to(gpu), cfg)
    xq = quantize_to_fp4(x, cfg)
    fp4_matmul(xq, wq)  # first use outside the recording
    side = torch.cuda.Stream(device=gpu)
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        out = fp4_matmul(xq, wq)
    for seed in (63, 64, 65):
        fresh = quantize_to_fp4(activations((M, K), seed).to(gpu), cfg)
        xq.values.copy_(fresh.values), xq.scale_factors.copy_(fresh.scale_factors), xq.amax.copy_(fresh.amax)
        torch.cuda.synchronize()
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, fp4_matmul(xq, wq))


@pytest.mark.parametrize("M,N,K", [(300, 1100, 5120), (2640, 3072, 3072), (130, 513, 12800), (1000, 2048, 14336)])
def test_persistent_schedule_against_the_oracle_and_the_tile_schedule(gpu, M, N, K):
    """The persistent launch (one workgroup per compute unit, 128 x 512 tiles, the K range of the tiles behind the
    whole rounds shared between workgroups and summed from fp32 partial tiles) against the oracle (1e-3 relative
    Frobenius) and against the one-workgroup-per-tile kernel, which adds the same exact products in another order;
    twice for identical bits (the order in which parts arrive must not show).  Shapes: ragged M and N with
    overhanging tiles; the projection shape, whose 126 tiles are all split; 4 tiles of 100 steps over 256 workgroups
    (every tile cut into some sixty parts); a long K with 32 tiles of 112 steps."""
    cfg = QuantizationConfig(scale_rule="mse")
    xq = quantize_to_fp4(activations((M, K), 81).to(gpu), cfg)
    wq = quantize_to_fp4(weights((N, K), 82).to(gpu), cfg)
    cus = torch.cuda.get_device_properties(gpu).multi_processor_count
    assert _native.gemm_plan(M, N, K, compute_units=cus, schedule="persistent")["persistent"]
    with _native.gemm_schedule("tiles"):
        tiles = fp4_matmul(xq, wq)
    with _native.gemm_schedule("persistent"):
        pers = fp4_matmul(xq, wq)
        again = fp4_matmul(xq, wq)
    assert torch.equal(pers, again)
    _ulp_close(pers, tiles)
    if M * N * K <= 3e10:
        ref = o.fp4_matmul(_as_oracle(xq), _as_oracle(wq))
        assert _rel(pers.float().cpu().numpy(), ref) <= TOL
    assert _native.load().ll_nvfp4_gemm_get_schedule() == -1


def test_persistent_schedule_with_every_epilogue_and_grouped_products(gpu):
    """Bias, GELU, gated residual, amax sink and several products in one launch under the persistent schedule: the
    epilogue is the same code behind either kernel, so each result equals the tile schedule's up to the order of
    the fp32 additions, and the amax left in the sink is the maximum of the result written."""
    cfg = QuantizationConfig(scale_rule="mse")
    M, N, K, frame = 528, 1024, 5120, 176
    xq = quantize_to_fp4(activations((M, K), 91).to(gpu), cfg)
    ws = [quantize_to_fp4((weights((N, K), 92 + i) * (1 + i)).to(gpu), cfg) for i in range(3)]
    gen = torch.Generator().manual_seed(93)
    bias = (torch.randn(N, generator=gen) * 0.5).bfloat16().to(gpu)
    residual = torch.randn(M, N, generator=gen).bfloat16().to(gpu)
    gate = torch.randn(M // frame, 6, N, generator=gen).bfloat16().to(gpu)[:, 2]
    results = {}
    for sched in ("tiles", "persistent"):
        with _native.gemm_schedule(sched):
            t1, t2 = _native.amax_ticket(gpu), None
            gelu = fp4_matmul(xq, ws[0], bias=bias, activation="gelu_tanh", amax_out=t1)
            amax_gelu = float(quantize_to_fp4(gelu, cfg, amax=t1).amax)
            gated = fp4_matmul(xq, ws[1], bias=bias, residual=residual, gate=gate, gate_rows=frame)
            sinks = [_native.PrivateAmaxSink(gpu) for _ in range(3)]
            products = [dict(values=w.values, scales=w.scale_factors, amax=w.amax, denom=1536.0, bias=bias if i != 1 else None,
                             amax_out=s.ticket()) for i, (w, s) in enumerate(zip(ws, sinks))]
            grouped = _native.gemm_grouped(xq.values, xq.scale_factors, xq.amax, 1536.0, M, N, products)
            amax_grouped = [float(quantize_to_fp4(y, cfg, amax=pr["amax_out"]).amax) for y, pr in zip(grouped, products)]
            results[sched] = (gelu, amax_gelu, gated, grouped, amax_grouped)
    cus = torch.cuda.get_device_properties(gpu).multi_processor_count
    assert _native.gemm_plan(M, N, K, 3, cus, "persistent")["persistent"] and _native.gemm_plan(M, N, K, 1, cus, "persistent")["persistent"]
    (g0, a0, r0, gr0, ag0), (g1, a1, r1, gr1, ag1) = results["tiles"], results["persistent"]
    _ulp_close(g1, g0, frac=5e-3)
    _ulp_close(r1, r0)
    assert a1 == float(g1.float().abs().max())
    for y0, y1, am in zip(gr0, gr1, ag1):
        _ulp_close(y1, y0)
        assert am == float(y1.float().abs().max())
    with pytest.raises(ValueError):
        _native.gemm_schedule("fastest")


def test_persistent_schedule_on_a_capturing_stream(gpu):
    """A GEMM launch recorded into a graph never allocates: on a stream the library holds no memory for, a shape
    the automatic choice would run persistently takes the one-workgroup-per-tile kernel instead; after
    ll_nvfp4_gemm_reserve on that stream the persistent launch is recorded, and replays reproduce the eager
    result bit for bit."""
    cfg = QuantizationConfig(scale_rule="mse")
    M, N, K = 640, 1024, 6400
    xq = quantize_to_fp4(activations((M, K), 95).to(gpu), cfg)
    wq = quantize_to_fp4(weights((N, K), 96).to(gpu), cfg)
    with _native.gemm_schedule("persistent"):
        eager_p = fp4_matmul(xq, wq)
        with _native.gemm_schedule("tiles"):
            eager_t = fp4_matmul(xq, wq)
        side = torch.cuda.Stream(device=gpu)
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            out = fp4_matmul(xq, wq)
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager_t)          # no memory on that stream: the kernel that needs none
        side2 = torch.cuda.Stream(device=gpu)
        side2.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side2):
            _native.gemm_reserve(M, N, K)
        side2.synchronize()
        graph2 = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph2, stream=side2):
            out2 = fp4_matmul(xq, wq)
        for _ in range(3):
            out2.zero_()
            graph2.replay()
            torch.cuda.synchronize()
            assert torch.equal(out2, eager_p)
            fp4_matmul(xq, wq)
        with torch.cuda.stream(side2):
            _native.release_stream_memory()


@pytest.mark.parametrize("M,N,K,groups", [
    (2640, 14336, 3072, 1),   # 256 x 128 tiles: FFN-up
    (2688, 4096, 128, 1),     # one K step
    (513, 14336, 256, 1),     # ragged M, two steps
    (7040, 3072, 1024, 1),    # the projections at the released chunk size
    (2600, 14300, 1152, 1),   # 256 x 128 tiles, ragged M and N, an odd number of steps
    (12763, 379, 384, 1),     # 128 x 256 tiles, ragged M and N
    (2640, 3072, 3072, 3),    # 128 x 256 tiles: q, k, v in one launch
    (300, 1100, 1152, 2),     # two products, ragged
])
def test_hand_scheduled_main_loop_is_bit_identical_to_the_compiled_one(gpu, M, N, K, groups):
    """The one-workgroup-per-tile kernels with tiles of 256 x 128 and 128 x 256 run their main loop as a generated
    instruction sequence wherever K is a multiple of 128; every accumulator receives the same products in the same
    order as in the compiler's loop, so outputs and the amax left in the sinks are equal bit for bit.  (Shapes that
    take the eight-wave kernel, whose sums are formed in another order, have a test of their own.)"""
    cfg = QuantizationConfig(scale_rule="mse")
    xq = quantize_to_fp4(activations((M, K), 5).to(gpu), cfg)
    ws = [quantize_to_fp4((weights((N, K), 6 + i) * (1 + i)).to(gpu), cfg) for i in range(groups)]
    bias = (torch.randn(N, generator=torch.Generator().manual_seed(7)) * 0.1).to(gpu).bfloat16()
    out = {}
    for sched in ("tiles_compiled", "tiles"):
        with _native.gemm_schedule(sched):
            if groups == 1:
                t = _native.amax_ticket(gpu)
                y = [fp4_matmul(xq, ws[0], bias=bias, activation="gelu_tanh", amax_out=t)]
                amax = [float(quantize_to_fp4(y[0], cfg, amax=t).amax)]
            else:
                sinks = [_native.PrivateAmaxSink(gpu) for _ in range(groups)]
                products = [dict(values=w.values, scales=w.scale_factors, amax=w.amax, denom=1536.0, bias=bias if i != 1 else None,
                                 amax_out=s.ticket()) for i, (w, s) in enumerate(zip(ws, sinks))]
                y = _native.gemm_grouped(xq.values, xq.scale_factors, xq.amax, 1536.0, M, N, products)
                amax = [float(quantize_to_fp4(yi, cfg, amax=pr["amax_out"]).amax) for yi, pr in zip(y, products)]
        out[sched] = (y, amax)
    for got, want in zip(out["tiles"][0], out["tiles_compiled"][0]):
        assert torch.equal(got, want)
    assert out["tiles"][1] == out["tiles_compiled"][1]
    assert out["tiles"][1] == [float(yi.float().abs().max()) for yi in out["tiles"][0]]
