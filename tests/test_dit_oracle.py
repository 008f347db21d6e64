"""Structure of the DiT block oracle, pinned by special cases that a dropped term, a swapped modulation slot or a
transposed operand would fail (the reference ships no vector for a whole block)."""
import numpy as np
import pytest

import dit_oracle
import nvfp4_oracle as o

C, H, L, FS, T = 256, 2, 12, 4, 5      # dim, heads, tokens, tokens per frame, text tokens
F = L // FS
FFN = 512


def qweight(rng, n, k, scale=0.05):
    w = o.round_bf16((rng.standard_normal((n, k)) * scale).astype(np.float32))
    v, s, a, pad = o.quantize_to_fp4(o.f32_to_bf16(w), "mse")
    return dict(values=v, scales=s, amax=a, rule="mse", padded=pad, orig=w.shape)


def zero_weight(n, k):
    w = np.zeros((n, k), np.float32)
    v, s, a, pad = o.quantize_to_fp4(o.f32_to_bf16(w), "mse")
    return dict(values=v, scales=s, amax=a, rule="mse", padded=pad, orig=w.shape)


def params(seed=0):
    rng = np.random.default_rng(seed)
    p = {"modulation": np.zeros((6, C), np.float32)}
    for name in ("self_attn.q", "self_attn.k", "self_attn.v", "self_attn.o", "cross_attn.q", "cross_attn.k",
                 "cross_attn.v", "cross_attn.o"):
        p[name + ".w"] = qweight(rng, C, C)
        p[name + ".b"] = o.round_bf16((rng.standard_normal(C) * 0.02).astype(np.float32))
    p["ffn.0.w"], p["ffn.0.b"] = qweight(rng, FFN, C), o.round_bf16((rng.standard_normal(FFN) * 0.02).astype(np.float32))
    p["ffn.2.w"], p["ffn.2.b"] = qweight(rng, C, FFN), o.round_bf16((rng.standard_normal(C) * 0.02).astype(np.float32))
    for name in ("self_attn.norm_q", "self_attn.norm_k", "cross_attn.norm_q", "cross_attn.norm_k"):
        p[name] = np.ones(C, np.float32)
    p["norm3.w"], p["norm3.b"] = np.ones(C, np.float32), np.zeros(C, np.float32)
    return p, rng


def inputs(rng):
    x = o.round_bf16(rng.standard_normal((L, C)).astype(np.float32))
    ctx = o.round_bf16(rng.standard_normal((T, C)).astype(np.float32))
    cos, sin = o.rope_cos_sin(F, 2, 2, 0)
    return x, ctx, cos, sin


def e0_with(**slots):
    """[F, 6, C] modulation input: slot order shift1, scale1, gate1, shift2, scale2, gate2 (causal_model.py:862-863)."""
    e = np.zeros((F, 6, C), np.float32)
    for name, val in slots.items():
        e[:, ["shift1", "scale1", "gate1", "shift2", "scale2", "gate2"].index(name)] = val
    return e


def silence_cross_attention(p):
    p["cross_attn.o.w"], p["cross_attn.o.b"] = zero_weight(C, C), np.zeros(C, np.float32)


def run(x, e0, ctx, p, cos, sin, ck=None, cv=None):
    return dit_oracle.block_forward(x, e0, ctx, p, cos, sin, ck, cv, H, FS)[0]


def test_closed_gates_and_silent_cross_attention_leave_x_untouched():
    p, rng = params()
    x, ctx, cos, sin = inputs(rng)
    silence_cross_attention(p)
    out = run(x, e0_with(shift1=0.3, scale1=0.2, shift2=-0.1, scale2=0.4), ctx, p, cos, sin)
    assert np.array_equal(out, x)


def test_each_gate_opens_exactly_its_own_branch():
    p, rng = params()
    x, ctx, cos, sin = inputs(rng)
    silence_cross_attention(p)
    g = 0.5
    # gate1 only: x + bf16(attn_out * g), where attn_out does not depend on the gate
    y = o.adaln_modulate(x, np.zeros((F, C), np.float32), np.zeros((F, C), np.float32), FS, 1e-6)
    out1 = run(x, e0_with(gate1=g), ctx, p, cos, sin)
    out2 = run(x, e0_with(gate1=2 * g), ctx, p, cos, sin)
    d1, d2 = out1 - x, out2 - x
    assert np.abs(d1).max() > 0.01
    assert np.abs(d2 - 2 * d1).max() <= 2.0 ** -6 * np.abs(x).max()      # linear in the gate up to bf16 steps of x
    # gate2 only: x + bf16(ffn(adaLN(x)) * g), computed from the pinned pieces
    h = o.gelu_tanh(dit_oracle.linear_w4a4(y, p["ffn.0.w"], p["ffn.0.b"]))
    f = dit_oracle.linear_w4a4(h, p["ffn.2.w"], p["ffn.2.b"])
    want = o.round_bf16(x + o.round_bf16(f * g))
    assert np.array_equal(run(x, e0_with(gate2=g), ctx, p, cos, sin), want)
    # the self-attention gate does not leak into the FFN branch and vice versa
    assert not np.array_equal(out1, want)


def test_scale_and_shift_slots_feed_the_norm_of_their_own_branch():
    p, rng = params()
    x, ctx, cos, sin = inputs(rng)
    silence_cross_attention(p)
    base = run(x, e0_with(gate2=0.5), ctx, p, cos, sin)
    # slots of the first branch are invisible while its gate is closed
    assert np.array_equal(run(x, e0_with(gate2=0.5, shift1=0.7, scale1=-0.3), ctx, p, cos, sin), base)
    # slots of the second branch act as adaLN(x; scale2, shift2)
    sc, sh = 0.25, -0.5
    y = o.adaln_modulate(x, np.full((F, C), sc, np.float32), np.full((F, C), sh, np.float32), FS, 1e-6)
    h = o.gelu_tanh(dit_oracle.linear_w4a4(y, p["ffn.0.w"], p["ffn.0.b"]))
    want = o.round_bf16(x + o.round_bf16(dit_oracle.linear_w4a4(h, p["ffn.2.w"], p["ffn.2.b"]) * 0.5))
    assert np.array_equal(run(x, e0_with(gate2=0.5, scale2=sc, shift2=sh), ctx, p, cos, sin), want)
    # per-frame modulation: changing frame 1's gate changes frame 1's tokens only
    e = e0_with(gate2=0.5)
    e[1, 5] = 0.0
    out = run(x, e, ctx, p, cos, sin)
    assert np.array_equal(out[FS:2 * FS], x[FS:2 * FS]) and np.array_equal(out[:FS], base[:FS])


def test_cross_attention_is_added_without_a_gate_and_mixes_no_tokens():
    p, rng = params()
    x, ctx, cos, sin = inputs(rng)
    out = run(x, e0_with(), ctx, p, cos, sin)                 # both gates closed: x + cross_attn(norm3(x), ctx)
    n3 = dit_oracle.layer_norm_affine(x, p["norm3.w"], p["norm3.b"])
    cq = o.rms_norm(dit_oracle.linear_w4a4(n3, p["cross_attn.q.w"], p["cross_attn.q.b"]), p["cross_attn.norm_q"], 1e-6)
    ck = o.rms_norm(dit_oracle.linear_w4a4(ctx, p["cross_attn.k.w"], p["cross_attn.k.b"]), p["cross_attn.norm_k"], 1e-6)
    cv = dit_oracle.linear_w4a4(ctx, p["cross_attn.v.w"], p["cross_attn.v.b"])
    a = o.attention(cq.reshape(L, H, C // H), ck.reshape(T, H, C // H), cv.reshape(T, H, C // H)).reshape(L, C)
    assert np.array_equal(out, o.round_bf16(x + dit_oracle.linear_w4a4(a, p["cross_attn.o.w"], p["cross_attn.o.b"])))
    # the text keys are a set: their order does not matter
    perm = np.array([3, 0, 4, 1, 2])
    assert np.abs(run(x, e0_with(), ctx[perm], p, cos, sin) - out).max() <= 2.0 ** -6 * np.abs(out).max()


def test_cached_keys_are_attended_together_with_the_chunk():
    p, rng = params()
    x, ctx, cos, sin = inputs(rng)
    silence_cross_attention(p)
    D = C // H
    ck = o.round_bf16(rng.standard_normal((8, H, D)).astype(np.float32))
    cv = o.round_bf16(rng.standard_normal((8, H, D)).astype(np.float32))
    e = e0_with(gate1=1.0)
    with_cache = run(x, e, ctx, p, cos, sin, ck, cv)
    assert not np.array_equal(with_cache, run(x, e, ctx, p, cos, sin))
    perm = rng.permutation(8)                                  # cached keys are a set as well
    again = run(x, e, ctx, p, cos, sin, ck[perm], cv[perm])
    assert np.abs(again - with_cache).max() <= 2.0 ** -6 * np.abs(with_cache).max()
    # a cache whose values equal a constant row c pulls the attention output towards c
    big = np.zeros((8, H, D), np.float32)
    cvc = np.broadcast_to(o.round_bf16(rng.standard_normal((1, H, D)).astype(np.float32)), (8, H, D)).copy()
    q_like = dit_oracle.block_forward(x, e, ctx, p, cos, sin, big, cvc, H, FS)[0]
    assert np.isfinite(q_like).all()


def test_requantization_turns_a_relative_difference_into_about_two_thirds_of_its_square_root():
    """Where the block's end-to-end bar comes from.  Two bf16 tensors a relative Frobenius distance eps apart
    (eps = 1e-3 is the bar of one W4A4 linear against the oracle) quantize to NVFP4 tensors that are about
    0.65 * sqrt(eps) apart: a fraction ~eps / step of the elements lands on the other side of a rounding boundary
    and moves by a whole e2m1 step, a quarter to a third of its value.  A difference that moves the tensor maximum
    re-derives every block scale: one bf16 ulp on that one element puts the quantized tensors 5e-2 apart, and no
    difference can do more than the quantization noise itself (8.7e-2 for Gaussian data).  The block re-quantizes
    its activations three times behind the attention, each time diluted by the residual stream it is added to;
    its bar of 6e-2 on the output is one such re-derivation of the scales (measured: 3.4e-2)."""
    rng = np.random.default_rng(0)
    x = rng.standard_normal((256, 1024)).astype(np.float32)

    def quantized(t):
        bits = o.f32_to_bf16(t)
        v, s, a, pad = o.quantize_to_fp4(bits, "mse")
        return o.dequantize(v, s, a, "mse", pad, t.shape).astype(np.float64)

    base = quantized(x)
    noise_floor = np.linalg.norm(base - x) / np.linalg.norm(x)
    assert 0.08 < noise_floor < 0.095
    big = np.unravel_index(np.argmax(np.abs(x)), x.shape)
    for eps in (1e-4, 3e-4, 1e-3):
        n = rng.standard_normal(x.shape).astype(np.float32)
        n[big] = 0.0  # the tensor maximum stays where it is
        moved = x + eps * n * np.linalg.norm(x) / np.linalg.norm(n)
        r = np.linalg.norm(quantized(moved) - base) / np.linalg.norm(base)
        assert 0.5 * np.sqrt(eps) <= r <= 0.8 * np.sqrt(eps), (eps, r)
    # the tensor maximum alone, moved by one bf16 ulp (2^-8): every block scale is re-derived from it, 92 % of the
    # dequantized values change and the tensors are 5e-2 apart; moved by 5 % they are as far apart as the noise floor
    for factor, lo, hi in ((1.0 + 2.0 ** -8, 0.03, 0.065), (1.05, 0.07, 1.5 * noise_floor)):
        moved = x.copy()
        moved[big] *= factor
        r = np.linalg.norm(quantized(moved) - base) / np.linalg.norm(base)
        assert lo <= r <= hi, (factor, r)
