"""CPU pins of the oracle functions the KV-cache and DiT-block checks lean on: kv_dequantize, k_smooth and
gelu_tanh.  Each is checked against something that is not the oracle's own numpy expression: exact rational
arithmetic, torch's CPU kernels on real bf16 / float8 tensors, an algebraically different closed form, and the
golden-pinned dequantize."""
import math
from fractions import Fraction

import numpy as np
import pytest
import torch

import nvfp4_oracle as o
from helpers import bits_of, from_bits

E2M1 = [Fraction(v).limit_denominator(2) for v in (0, 0.5, 1, 1.5, 2, 3, 4, 6)]
AMAXES = [1.0, 1536.0, 3.140625, 0.00390625, 7.53125, 21.875, 1e-3, 250.0, 4.8125, 1.0000001, 5.9999995, 1537.25]


def _fl32(q: Fraction) -> np.float32:
    """Correctly rounded (nearest-even) fp32 of a rational, independent of numpy's float32 arithmetic:
    float(Fraction) is correctly rounded to double, and a double that is not within 2^-29 relative of an
    fp32 rounding boundary rounds to the same fp32 as the rational; the other cases are decided exactly."""
    d = float(q)
    f = np.float32(d)
    lo, hi = np.nextafter(f, np.float32(-np.inf)), np.nextafter(f, np.float32(np.inf))
    best = min((abs(Fraction(float(c)) - q), i, c) for i, c in enumerate((lo, f, hi)))
    ties = [c for c in (lo, f, hi) if abs(Fraction(float(c)) - q) == best[0]]
    if len(ties) == 2:  # exact tie: even mantissa
        return [c for c in ties if (c.view(np.uint32) & 1) == 0][0]
    return best[2]


def _all_codes_slot(amax):
    """A [128, 128] slot that holds every (scale byte < 0x7F, e2m1 code) pair: row r uses scale bytes
    8 (r % 16) .. + 7 in its eight blocks (the 127 finite non-negative e4m3 values and one zero), and every block
    holds the 16 codes."""
    codes = np.tile(np.arange(16, dtype=np.uint8), (128, 8))
    values = o._pack(codes)
    sb = ((np.arange(128)[:, None] % 16) * 8 + np.arange(8)[None, :]).astype(np.uint8)
    sb[sb == 0x7F] = 0
    return values, o.to_blocked(sb), np.float32(amax), codes, sb


@pytest.mark.parametrize("path", ["fused", "triton"])
def test_kv_dequantize_is_the_correctly_rounded_reference_expression(path):
    """(code * scale) * gs with gs = RN(amax * RN(1/1536)) [fused CUDA path, kv_dequant_cuda.cu:95,216] or
    RN(amax / 1536) [Triton fallback, utils/quant.py:753-756], in exact rational arithmetic, rounded once to
    fp32 and then to bf16."""
    for amax in AMAXES[:6]:
        values, scales, a, codes, sb = _all_codes_slot(amax)
        got32 = o.kv_dequantize(values, scales, a, "mse", path=path, dtype="f32")
        got16 = o.kv_dequantize(values, scales, a, "mse", path=path)
        fa = Fraction(float(np.float32(amax)))
        if path == "fused":
            gs = _fl32(fa * Fraction(float(np.float32(1.0 / 1536.0))))
        else:
            gs = _fl32(fa / 1536)
        assert gs == o.kv_global_scale(a, "mse", path)
        for r in range(0, 16):  # rows repeat with period 16
            for blk in range(8):
                b = int(sb[r, blk])
                e, m = b >> 3, b & 7
                s = Fraction(m, 512) if e == 0 else Fraction(8 + m, 8) * Fraction(2) ** (e - 7)
                for c in range(16):
                    exact = (-1 if c & 8 else 1) * E2M1[c & 7] * s * Fraction(float(gs))
                    want = _fl32(exact)
                    assert got32[r, blk * 16 + c] == want
                    want16 = bits_of(torch.tensor([float(want)], dtype=torch.float32).bfloat16())[0]
                    assert o.f32_to_bf16(got16[r:r + 1, blk * 16 + c])[0] == want16 or (want == 0)


@pytest.mark.parametrize("path", ["fused", "triton"])
def test_kv_dequantize_matches_torch_evaluation(path):
    """The same expression evaluated by torch's CPU kernels on float8_e4m3fn / float32 / bfloat16 tensors
    (torch's decoders and roundings, not the oracle's)."""
    lut = torch.tensor([0, .5, 1, 1.5, 2, 3, 4, 6, -0.0, -.5, -1, -1.5, -2, -3, -4, -6], dtype=torch.float32)
    rng = np.random.default_rng(5)
    for amax in AMAXES:
        values, scales, a, codes, sb = _all_codes_slot(amax)
        # shuffle codes so that the packing order matters too
        codes = rng.permuted(codes, axis=1)
        values = o._pack(codes)
        sf = torch.from_numpy(sb.copy()).view(torch.float8_e4m3fn).float().repeat_interleave(16, dim=1)
        at = torch.tensor(float(a), dtype=torch.float32)
        if path == "fused":
            gs = at * torch.tensor(1.0 / (6.0 * 256.0), dtype=torch.float64).float()
        else:
            gs = at / torch.tensor(6 * 256, dtype=torch.float32)
        ref = (lut[torch.from_numpy(codes.astype(np.int64))] * sf * gs).bfloat16()
        got = o.kv_dequantize(values, scales, a, "mse", path=path)
        assert np.array_equal(o.f32_to_bf16(got), bits_of(ref))


def test_kv_dequantize_against_golden_pinned_dequantize(golden):
    """QuantizedTensor.dequantize ((v*s)*amax)/1536 is pinned by reference-written vectors.  The cache
    expression differs from it only in where amax meets 1536, so the fp32 values lie within 2 ulp of each
    other and the bf16 values are equal except next to a bf16 rounding boundary, where they are one bf16 step
    apart.  Both reference paths are held to this."""
    n_checked = 0
    for name in golden["case_names"]:
        key = f"{name}/mse"
        if f"{key}/values" not in golden.files:
            continue
        values, scales, amax = golden[f"{key}/values"], golden[f"{key}/scales"], golden[f"{key}/amax"]
        Mp, Kp = values.shape[0], values.shape[1] * 2
        d32 = o.dequantize(values, scales, amax, "mse", (Mp, Kp), (Mp, Kp), "f32")
        d16 = o.f32_to_bf16(o.dequantize(values, scales, amax, "mse", (Mp, Kp), (Mp, Kp), "bf16"))
        for path in ("fused", "triton"):
            k32 = o.kv_dequantize(values, scales, amax, "mse", path=path, dtype="f32")
            k16 = o.f32_to_bf16(o.kv_dequantize(values, scales, amax, "mse", path=path))
            fin = np.isfinite(d32) & np.isfinite(k32)
            ulp = np.abs(k32.view(np.int32).astype(np.int64) - d32.view(np.int32).astype(np.int64))
            assert ulp[fin].max() <= 2
            step = np.abs(k16.astype(np.int32) - d16.astype(np.int32))
            assert step[fin].max() <= 1
            # bf16 values may differ only where the fp32 value sits within 2 ulp of a bf16 tie
            low = d32.view(np.uint32) & np.uint32(0xFFFF)
            near_tie = np.abs(low.astype(np.int64) - 0x8000) <= 2
            assert not np.any((step != 0) & fin & ~near_tie)
            n_checked += int(fin.sum())
    assert n_checked > 100000


def test_fused_and_triton_global_scales_differ_by_at_most_one_ulp():
    rng = np.random.default_rng(11)
    am = np.abs(rng.standard_normal(200000).astype(np.float32)) * np.float32(10.0) ** rng.integers(-3, 3, 200000).astype(np.float32)
    f = np.array([o.kv_global_scale(a, "mse", "fused") for a in am[:20000]])
    t = np.array([o.kv_global_scale(a, "mse", "triton") for a in am[:20000]])
    d = np.abs(f.view(np.int32).astype(np.int64) - t.view(np.int32).astype(np.int64))
    assert d.max() <= 1 and 0 < (d != 0).mean() < 0.5  # they do differ, which is why one has to be chosen


# ------------------------------------------------------------------ k_smooth
@pytest.mark.parametrize("scale,offset", [(1.0, 0.0), (1.0, 3.0), (30.0, 100.0), (1e-3, 1e-3), (0.05, 8.0)])
def test_k_smooth_matches_torch_bf16_bit_for_bit(scale, offset):
    """utils/quant.py:797-798, `k - k.mean(dim=-1, keepdim=True)`, evaluated by torch on bf16 tensors."""
    g = torch.Generator().manual_seed(int(scale * 1000) + int(offset))
    k = (torch.randn(1, 3000, 4, 128, generator=g) * scale + torch.randn(1, 3000, 4, 1, generator=g) * offset).bfloat16()
    ref = bits_of(k - k.mean(dim=-1, keepdim=True))
    got = o.f32_to_bf16(o.k_smooth(k.float().numpy()))
    assert np.array_equal(got, ref)


def test_k_smooth_closed_forms():
    k = np.full((2, 3, 128), 1.5, dtype=np.float32)
    assert np.array_equal(o.k_smooth(k), np.zeros_like(k))  # a constant head is removed entirely
    k = np.zeros((1, 1, 128), dtype=np.float32)
    k[..., 0] = 128.0  # mean 1 exactly
    want = np.full((1, 1, 128), -1.0, dtype=np.float32)
    want[..., 0] = 127.0
    assert np.array_equal(o.k_smooth(k), want)


# ------------------------------------------------------------------ gelu_tanh
def _all_bf16_in(lo, hi):
    allb = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    x = o.bf16_to_f32(allb)
    sel = np.isfinite(x) & (x >= lo) & (x <= hi)
    return allb[sel]


def test_gelu_tanh_matches_torch_on_every_bf16_value():
    """nn.GELU(approximate="tanh") (wan_5b/modules/causal_model.py:822-824) on every bf16 value of [-8, 8].
    torch evaluates 0.5 x (1 + tanh(u)) in fp32; for x < -2.9 the sum 1 + tanh(u) cancels (tanh(u) is within
    2^-12 of -1), so torch's value carries an absolute error of a few |x| 2^-25 there (fp32 tanh is good to a
    few units of 2^-24 next to -1) while the oracle (fp64) does not.  Outside that tail the two must be
    identical; inside it they must agree within that error plus one bf16 step."""
    xb = _all_bf16_in(-8.0, 8.0)
    x = o.bf16_to_f32(xb)
    ref_bits = bits_of(torch.nn.functional.gelu(from_bits(xb), approximate="tanh"))
    got = o.gelu_tanh(x)
    got_bits = o.f32_to_bf16(got)
    tail = x < -2.9
    assert np.array_equal(got_bits[~tail], ref_bits[~tail])
    assert (~tail).sum() > 30000
    ref = o.bf16_to_f32(ref_bits)
    bound = 2.0 * np.abs(x) * 2.0 ** -24 + np.abs(got) * 2.0 ** -7
    assert np.all(np.abs(ref[tail] - got[tail]) <= bound[tail])
    assert tail.sum() < 250  # the tail is the 199 bf16 values of [-8, -2.9)


def test_gelu_tanh_equals_logistic_form_in_fp64():
    """0.5 (1 + tanh(u)) = 1 / (1 + exp(-2u)): a different expression of the same function, which has no
    cancellation in the negative tail; evaluated with Python's math in double."""
    xb = _all_bf16_in(-8.0, 8.0)
    x = o.bf16_to_f32(xb).astype(np.float64)
    c = math.sqrt(2.0 / math.pi)
    want = np.array([v / (1.0 + math.exp(-2.0 * c * (v + 0.044715 * v ** 3))) for v in x])
    got = o.gelu_tanh(x.astype(np.float32)).astype(np.float64)
    # The tanh form cancels in double too, but only at the 2^-53 level: below |x| 2^-53 ~ 1e-15 it returns -0
    # where the logistic form still resolves values down to 1e-21.  Above that floor the bf16 results are equal.
    resolved = (x > -5.0) | (np.abs(want) > 1e-10)
    want_bits = o.f32_to_bf16(want.astype(np.float32))
    got_bits = o.f32_to_bf16(got.astype(np.float32))
    assert np.array_equal(want_bits[resolved], got_bits[resolved]) and resolved.sum() > 33000
    assert np.all(np.abs(want - got) <= np.abs(want) * 2.0 ** -8 + 1e-14)
    # textbook anchors
    assert o.gelu_tanh(np.array([0.0], dtype=np.float32))[0] == 0.0
    big = o.gelu_tanh(np.array([8.0, -8.0], dtype=np.float32))
    assert big[0] == 8.0 and abs(big[1]) < 1e-12


@pytest.mark.parametrize("affine", [True, False])
@pytest.mark.parametrize("rows,C,scale,offset", [(64, 256, 1.0, 0.0), (16, 3072, 3.0, 5.0), (33, 1000, 0.02, -0.5)])
def test_layer_norm_affine_matches_torch_layer_norm(rows, C, scale, offset, affine):
    """dit_oracle.layer_norm_affine (the LayerNorm ahead of cross-attention, wan_5b/modules/model.py:101-111: fp32
    statistics and affine map on the bf16 input, one rounding to bf16) against torch's CPU layer_norm on the same
    values in fp32, rounded to bf16 by torch: identical except where the fp32 result sits within rounding noise of
    a bf16 tie (the oracle forms the statistics in double), there one bf16 ulp apart; and against the bf16 kernel of
    torch (which keeps fp32 internally), to the same bar."""
    import dit_oracle

    g = torch.Generator().manual_seed(rows * 7 + C)
    x = (torch.randn(rows, C, generator=g) * scale + offset).bfloat16()
    w = (1 + 0.2 * torch.randn(C, generator=g)).bfloat16() if affine else torch.ones(C).bfloat16()
    b = (0.3 * torch.randn(C, generator=g)).bfloat16() if affine else torch.zeros(C).bfloat16()
    xn, wn, bn = (t.float().numpy() for t in (x, w, b))
    got = dit_oracle.layer_norm_affine(xn, wn, bn, 1e-6)
    for want in (torch.nn.functional.layer_norm(x.float(), (C,), w.float() if affine else None, b.float() if affine else None, 1e-6).bfloat16(),
                 torch.nn.functional.layer_norm(x, (C,), w if affine else None, b if affine else None, 1e-6)):
        want = want.float().numpy()
        diff = np.abs(got - want)
        # one bf16 ulp of the result, or - where the affine map cancels - of the terms that went into it
        terms = np.abs(want) + np.abs(bn)[None, :]
        assert (diff <= terms * 2.0 ** -7).all(), float((diff / terms).max())
        assert (diff != 0).mean() <= 5e-3   # most on the row set whose mean lies 25 standard deviations from zero (fp32 statistics)
    # closed form: a constant row normalizes to the bias
    const = np.full((2, C), 3.0, dtype=np.float32)
    out = dit_oracle.layer_norm_affine(const, wn, bn, 1e-6)
    assert np.array_equal(out, np.broadcast_to(bn, (2, C)))
