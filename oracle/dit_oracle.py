"""CPU oracle for one causal DiT block with NVFP4 linears and an FP4 KV cache (TEST INFRASTRUCTURE ONLY).

Composition of the functions in ``nvfp4_oracle`` in the order of the reference block forward
(wan_5b/modules/causal_model.py:862-930, 362-368, 477-487, 557-671, 197-262), with a bf16 rounding
wherever the eager bf16 graph of the reference rounds.  The reference ships no golden vector for a block, so
the composition is **parity unpinned** against the reference itself; what pins it here is that every component is
pinned on its own and that structural special cases hold (tests/test_dit_oracle.py: closed gates are the
identity, each gate opens exactly its own branch, scale / shift slots feed the norm of their own branch and
frame, cross-attention is added ungated and token by token, cached keys are attended as a set) - the cases a
dropped term, a swapped modulation slot or a transposed operand would fail.
"""
from __future__ import annotations

import numpy as np

import nvfp4_oracle as o

F32 = np.float32


def linear_w4a4(x, weight, bias, act_rule="mse"):
    """x fp32 (bf16 values) [M, K]; weight = dict(values, scales, amax, rule, padded, orig)."""
    v, s, a, pad = o.quantize_to_fp4(o.f32_to_bf16(x), act_rule)
    xa = dict(values=v, scales=s, amax=a, rule=act_rule, padded=pad, orig=x.shape)
    y = o.fp4_matmul(xa, weight)
    if bias is not None:
        y = o.round_bf16(y + bias[None, :])
    return y


def layer_norm_affine(x, w, b, eps=1e-6):
    x64 = x.astype(np.float64)
    mu = x64.mean(-1, keepdims=True)
    var = ((x64 - mu) ** 2).mean(-1, keepdims=True)
    return o.round_bf16((((x64 - mu) / np.sqrt(var + eps)) * w + b).astype(F32))


def block_forward(x, e0, context, p, cos, sin, cached_k, cached_v, num_heads, frame_seqlen, eps=1e-6):
    """x [L, C]; e0 [F, 6, C]; context [T, C]; p: parameter dict; cached_k / cached_v: dequantized
    bf16 cache [n, H, D] (or None).  Returns (x_out, roped_k [L,H,D], v [L,H,D])."""
    L, C = x.shape
    H, D = num_heads, C // num_heads
    e = o.round_bf16(p["modulation"][None, :, :] + e0)  # [F, 6, C]
    fidx = np.arange(L) // frame_seqlen
    y = o.adaln_modulate(x, e[:, 1], e[:, 0], frame_seqlen, eps)
    q = o.rms_norm(linear_w4a4(y, p["self_attn.q.w"], p["self_attn.q.b"]), p["self_attn.norm_q"], eps)
    k = o.rms_norm(linear_w4a4(y, p["self_attn.k.w"], p["self_attn.k.b"]), p["self_attn.norm_k"], eps)
    v = linear_w4a4(y, p["self_attn.v.w"], p["self_attn.v.b"]).reshape(L, H, D)
    rq = o.rope_apply(q.reshape(L, H, D), cos, sin)
    rk = o.rope_apply(k.reshape(L, H, D), cos, sin)
    ks = o.k_smooth(rk)
    keys = ks if cached_k is None else np.concatenate([cached_k, ks])
    vals = v if cached_v is None else np.concatenate([cached_v, v])
    a = o.attention(rq, keys, vals).reshape(L, C)
    y = linear_w4a4(a, p["self_attn.o.w"], p["self_attn.o.b"])
    x = o.round_bf16(x + o.round_bf16(y * e[fidx, 2]))
    n3 = layer_norm_affine(x, p["norm3.w"], p["norm3.b"], eps)
    cq = o.rms_norm(linear_w4a4(n3, p["cross_attn.q.w"], p["cross_attn.q.b"]), p["cross_attn.norm_q"], eps)
    ck = o.rms_norm(linear_w4a4(context, p["cross_attn.k.w"], p["cross_attn.k.b"]), p["cross_attn.norm_k"], eps)
    cv = linear_w4a4(context, p["cross_attn.v.w"], p["cross_attn.v.b"])
    T = context.shape[0]
    a = o.attention(cq.reshape(L, H, D), ck.reshape(T, H, D), cv.reshape(T, H, D)).reshape(L, C)
    x = o.round_bf16(x + linear_w4a4(a, p["cross_attn.o.w"], p["cross_attn.o.b"]))
    y = o.adaln_modulate(x, e[:, 4], e[:, 3], frame_seqlen, eps)
    h = o.gelu_tanh(linear_w4a4(y, p["ffn.0.w"], p["ffn.0.b"]))
    y = linear_w4a4(h, p["ffn.2.w"], p["ffn.2.b"])
    x = o.round_bf16(x + o.round_bf16(y * e[fidx, 5]))
    return x, rk, v
