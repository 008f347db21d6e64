"""The HIP quantizer decides the four-over-six choice of most blocks from cheap error estimates and only
falls back to the reference's arithmetic when the candidates are close (quantize.hip, pick_four).  This test
restates that decision rule in numpy float32 and checks it against the oracle's exact errors on millions of
blocks: wherever the rule claims to be sure, the oracle's comparison must agree, and the rule must be sure
almost always (otherwise the fallback would cost the speed it is there to buy)."""
import zlib

import numpy as np
import pytest

import nvfp4_oracle as o

F32 = np.float32
U = F32(2.0 ** -24)


def _estimates(X, amax, rule):
    e2, e4 = o.rule_limits(rule)
    bmax = np.abs(X).max(axis=-1)
    out = []
    for expansion in (None, 1.5):
        y, sb, sf = o._nvfp4_candidate(X, bmax, amax, e2, e4, expansion)
        q = o._fake_quantize_e2m1(y)
        d = (q - y).astype(F32)
        if rule == "mse":
            a = np.zeros(len(X), dtype=F32)
            for i in range(16):
                a = (a + d[:, i] * d[:, i]).astype(F32)
        elif rule == "mae":
            a = np.abs(d).sum(axis=-1, dtype=F32)
        else:
            a = np.abs(d).max(axis=-1)
        d1 = ((sf * amax) / F32(1536)).astype(F32)
        w = (d1 * d1).astype(F32) if rule == "mse" else d1
        if rule == "mse":
            b = None  # the mse margin is formed from the sums below
        elif rule == "mae":
            b = F32(640) * U + F32(32) * U * a
        else:
            b = F32(40) * U + F32(8) * U * a
        out.append(((a * w).astype(F32), None if b is None else b * w, sb, q, sf, w))
    (E6, B6, sb6, q6, sf6, w6), (E4, B4, sb4, q4, sf4, w4) = out
    if rule == "mse":  # quantize.hip, pick_four: 640 u (w4 + w6) + 800 u (E4 + E6)
        margin = ((F32(800) * U) * (E6 + E4) + (F32(640) * U) * (w6 + w4)).astype(F32) + F32(2.0 ** -100)
    else:
        margin = F32(4) * (B6 + B4 + F32(8) * U * (E6 + E4)) + F32(2.0 ** -100)
    same = sb4 == sb6  # identical candidates: the kernel keeps "6" without looking at errors
    sure = ((np.abs(E4 - E6) > margin) & (sb6 != 0)) | same
    # the oracle's own comparison (reference.py:175-239 as restated in quantize_blocks)
    denom = F32(1536)
    d6 = ((q6 * sf6[:, None]) * amax) / denom
    d4 = ((q4 * sf4[:, None]) * amax) / denom
    if rule == "abs_max":
        x4, x6 = np.abs(d4 - X).max(axis=-1), np.abs(d6 - X).max(axis=-1)
    elif rule == "mae":
        x4, x6 = o._seq_sum(np.abs(d4 - X)), o._seq_sum(np.abs(d6 - X))
    else:
        x4, x6 = o._seq_sum((d4 - X) * (d4 - X)), o._seq_sum((d6 - X) * (d6 - X))
    return sure, (E4 < E6) & ~same, x4 < x6, sb6 == 0


def _inputs(kind, n, rng):
    if kind == "normal":
        x = rng.standard_normal((n, 16))
    elif kind == "outliers":
        x = rng.standard_normal((n, 16)) * np.where(rng.random((n, 16)) < 0.001, 20.0, 1.0)
    elif kind == "magnitudes":
        x = rng.standard_normal((n, 16)) * np.exp2(rng.integers(-14, 4, size=(n, 1)))
    else:  # lattice: many exact and near ties
        x = rng.integers(-12, 13, size=(n, 16)) * 0.25 * (1 + rng.choice([-2.0 ** -8, 0, 2.0 ** -8], size=(n, 16)))
    return o.round_bf16(x.astype(F32))


@pytest.mark.parametrize("rule,n", [("mse", 1 << 20), ("mae", 1 << 18)])  # abs_max always takes the exact path
@pytest.mark.parametrize("kind", ["normal", "outliers", "magnitudes", "lattice"])
def test_estimate_rule_never_contradicts_the_reference(rule, n, kind):
    rng = np.random.default_rng(zlib.crc32(f"{rule}/{kind}".encode()))  # the same blocks in every run
    X = _inputs(kind, n, rng)
    amax = F32(np.abs(X).max())
    sure, by_estimate, by_reference, zero_scale = _estimates(X, amax, rule)
    assert np.array_equal(by_estimate[sure], by_reference[sure]), \
        f"{(by_estimate[sure] != by_reference[sure]).sum()} confident decisions differ from the reference"
    if kind != "lattice":
        # the exact fallback stays rare; blocks more than 2^17 below the tensor amax (scale byte 0 for the "6"
        # candidate only) always take it and are left out of the count
        assert (~sure & ~zero_scale).mean() < (3e-3 if rule == "mse" else 5e-3)
