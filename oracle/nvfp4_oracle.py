"""CPU oracle for the NVFP4 inference hot path (TEST INFRASTRUCTURE ONLY).

This module is a numpy restatement of the reference's algorithms.  It is the
checker for the HIP kernels: only ``tests/``, ``__graft_entry__.smoke()`` and
the ``cpu_baseline`` leg of ``bench.py`` may import it.  The product path never
routes through it.

All arithmetic is IEEE binary32 unless stated; every intermediate that the
reference rounds is rounded here in the same place.  bf16 tensors are carried
as ``uint16`` bit patterns (``bf16_to_f32`` / ``f32_to_bf16``).

Reference files followed (paths relative to the reference checkout):

* quantize        fouroversix/src/fouroversix/quantize/pytorch/reference.py:13-368
                  fouroversix/src/fouroversix/quantize/pytorch/backend.py:36-112
* scale layout    fouroversix/src/fouroversix/quantize/utils.py:88-96
                  fouroversix/src/fouroversix/quantize/quantized_tensor.py:10-18
* dequantize      fouroversix/src/fouroversix/quantize/quantized_tensor.py:21-53,184-214
* matmul          fouroversix/src/fouroversix/matmul/pytorch.py:22-41
* KV dequant      utils/kernel/kv_dequant_cuda.cu:59-107, 216 (the path the reference takes when its extension is
                  built), utils/nvfp4_kernel.py:40-176 + utils/quant.py:731-768 (its fallback)
* KV attention    wan_5b/modules/causal_model.py:491-724,781 ; wan_5b/modules/attention.py:260-306
* RoPE            utils/rope_triton.py:36-135 ; wan_5b/modules/model.py:29-36 ;
                  wan_5b/modules/causal_model.py:90-194
* adaLN           utils/adaln_triton.py:36-126
* RMSNorm         wan_5b/modules/model.py:82-98

Pinning status (what independent evidence fixes each function):

* e2m1 / e4m3 codecs          exhaustive enumeration + torch.float8_e4m3fn casts
* to_blocked / from_blocked   brute-force index formula (utils/kernel/kv_dequant_cuda.cu:41-57)
* quantize static_6/static_4  closed forms (zeros / ones / block-max scale bytes), idempotence
* quantize mse/mae/abs_max    selection invariant in fp64 + golden vectors written by the
                              reference's own PyTorch backend (tests/golden/)
* dequantize / matmul         exhaustive code x scale table; fp64 brute force; integer special case
* kv_dequantize               exact rational arithmetic, torch float32/float8/bfloat16 evaluation of the same
                              expression, and the golden-pinned dequantize (within one bf16 ulp, equal away
                              from rounding boundaries)
* k_smooth                    bit-exact against torch's bf16 `k - k.mean(-1, keepdim=True)`
* attention / RoPE / adaLN    fp64 textbook forms, torch library routines (layer_norm,
                              complex multiply), norm preservation
* gate_residual               the two eager bf16 operations
* gelu_tanh                   torch.nn.functional.gelu(approximate="tanh") on every bf16 value of [-8, 8] (equal
                              outside the negative tail, where torch's fp32 `1 + tanh` cancels; there within
                              the cancellation bound) and the algebraically equal logistic form in fp64

Parity unpinned: the reference's production matmul is a CUTLASS kernel (fouroversix/.gitmodules, submodule
absent, no pinned commit) and its attention is flash-attn 2.8.3 (not installed); neither result is
recorded anywhere in the reference's tests.  ``fp4_matmul`` and ``attention`` here follow the reference's
PyTorch matmul backend (pinned by one golden matmul) and the textbook softmax; agreement with the
third-party kernels themselves is not pinned.
"""
from __future__ import annotations

import numpy as np

F32 = np.float32

E2M1_VALUES = np.array(
    [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0],
    dtype=F32,
)

SCALE_RULES = ("static_6", "static_4", "mae", "mse", "abs_max")
# ids used by the native operator schema (fouroversix/src/fouroversix/utils.py:113-122)
RULE_ID = {"static_6": 0, "static_4": 1, "mae": 2, "mse": 3, "abs_max": 4}


def rule_limits(rule: str) -> tuple[int, int]:
    """(max e2m1 value, max e4m3 value) — fouroversix/src/fouroversix/utils.py:124-134."""
    e2 = 4 if rule == "static_4" else 6
    e4 = 448 if rule in ("static_6", "static_4") else 256
    return e2, e4


# --------------------------------------------------------------------------- bf16
def bf16_to_f32(bits: np.ndarray) -> np.ndarray:
    bits = np.asarray(bits, dtype=np.uint16)
    return (bits.astype(np.uint32) << np.uint32(16)).view(F32)


def f32_to_bf16(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even fp32 -> bf16 bit pattern (NaN kept quiet)."""
    x = np.ascontiguousarray(x, dtype=F32)
    u = x.view(np.uint32)
    lsb = (u >> np.uint32(16)) & np.uint32(1)
    r = (u + np.uint32(0x7FFF) + lsb) >> np.uint32(16)
    nan = np.isnan(x)
    r = np.where(nan, (u >> np.uint32(16)) | np.uint32(0x40), r)
    return r.astype(np.uint16)


def round_bf16(x: np.ndarray) -> np.ndarray:
    return bf16_to_f32(f32_to_bf16(x))


# --------------------------------------------------------------------------- e4m3fn
def e4m3_decode(b: np.ndarray) -> np.ndarray:
    """uint8 e4m3fn (bias 7, subnormals, 0x7F/0xFF = NaN) -> fp32, exact."""
    b = np.asarray(b, dtype=np.uint8).astype(np.int32)
    sign = np.where(b & 0x80, F32(-1.0), F32(1.0)).astype(F32)
    e = (b >> 3) & 0xF
    m = b & 0x7
    normal = np.ldexp((8 + m).astype(F32), e - 10).astype(F32)
    sub = np.ldexp(m.astype(F32), -9).astype(F32)
    v = np.where(e == 0, sub, normal).astype(F32)
    v = np.where((e == 15) & (m == 7), F32(np.nan), v)
    return (sign * v).astype(F32)


def e4m3_encode(x: np.ndarray) -> np.ndarray:
    """fp32 -> e4m3fn byte, round-to-nearest-even, |x| > 464 -> NaN (0x7F), like the
    ``.to(torch.float8_e4m3fn)`` cast used at reference.py:157."""
    x = np.ascontiguousarray(x, dtype=F32)
    sign = ((x.view(np.uint32) >> np.uint32(24)) & np.uint32(0x80)).astype(np.uint8)
    a = np.abs(x).astype(np.float64)  # exact widening; rounding done once below
    out = np.zeros(x.shape, dtype=np.uint8)
    # exponent of the target grid: normal numbers 2^-6 .. 2^8, step 2^(e-3); subnormal step 2^-9
    with np.errstate(divide="ignore", invalid="ignore"):
        e = np.floor(np.log2(np.where(a > 0, a, 1.0))).astype(np.int64)
    e = np.clip(e, -6, 8)
    step = np.ldexp(1.0, e - 3)
    n = np.rint(a / step)  # rint = half-to-even; a/step exact (power of two)
    # mantissa overflow (n == 16) moves to the next binade
    bump = n >= 16
    e = np.where(bump, e + 1, e)
    n = np.where(bump, 8, n)
    is_sub = n < 8  # only possible when e == -6
    byte = np.where(is_sub, n, ((e + 7) << 3) + (n - 8)).astype(np.int64)
    nan = (byte > 0x7E) | np.isnan(a)
    byte = np.where(nan, 0x7F, byte)
    out[...] = byte.astype(np.uint8)
    return out | sign


# --------------------------------------------------------------------------- scale layout
def to_blocked(a: np.ndarray) -> np.ndarray:
    """[rows, cols] -> 1-D, 128x4 tiles swizzled as 32x16 (quantize/utils.py:88-96)."""
    rows, cols = a.shape
    assert rows % 128 == 0 and cols % 4 == 0
    t = a.reshape(rows // 128, 128, cols // 4, 4).transpose(0, 2, 1, 3)
    t = t.reshape(-1, 4, 32, 4).transpose(0, 2, 1, 3)
    return np.ascontiguousarray(t).reshape(-1)


def from_blocked(a: np.ndarray, shape: tuple[int, int]) -> np.ndarray:
    """Inverse of :func:`to_blocked` (quantized_tensor.py:10-18)."""
    rows, cols = shape
    t = a.reshape(-1, 32, 4, 4).transpose(0, 2, 1, 3)
    t = np.ascontiguousarray(t).reshape(-1, cols // 4, 128, 4).transpose(0, 2, 1, 3)
    return np.ascontiguousarray(t).reshape(rows, cols)


def blocked_index(r, c, cols):
    """Flat offset of scale (r, c) of a [rows, cols] matrix in the blocked layout
    (closed form; cf. utils/kernel/kv_dequant_cuda.cu:41-57)."""
    rb, ri = np.divmod(r, 128)
    cb, ci = np.divmod(c, 4)
    return ((rb * (cols // 4) + cb) * 32 + (ri % 32)) * 16 + (ri // 32) * 4 + ci


# --------------------------------------------------------------------------- quantize
def _fake_quantize_e2m1(y: np.ndarray) -> np.ndarray:
    """reference.py:13-34 (nearest): grid 0,.5,1,1.5 | 2,3 | 4,6,(8,..) with half-to-even."""
    a = np.abs(y)
    step1 = np.rint(F32(2) * a) / F32(2)
    step2 = np.rint(a)
    step3 = F32(2) * np.rint(a / F32(2))
    m1 = a < F32(2)
    m2 = a < F32(4)
    mag = np.where(m1, step1, np.where(m2, step2, step3)).astype(F32)
    return (np.sign(y).astype(F32) * mag).astype(F32)


def _codes_from_fake_quantized(q: np.ndarray) -> np.ndarray:
    """reference.py:37-63: e2m1 code read from the bf16 bit pattern of q (no clamping;
    |q| >= 8 spills past 4 bits exactly as the int16 arithmetic of the reference does)."""
    bx = f32_to_bf16(q).astype(np.int16)
    s = (bx >> 15) & 0x1
    e = (bx >> 7) & 0xFF
    m = bx & 0x7F
    is_zero = (e == 0) & (m == 0)
    m = (m >> 6) & 1
    is_half = (e == 126) & (m == 0)
    m = np.where(is_half, 1, m)
    e = e - 126
    e = np.where(is_zero, 0, e)
    m = np.where(is_zero, 0, m)
    code = (s << 3) | (e << 1) | m
    return code.astype(np.uint8)


def _pack(codes: np.ndarray) -> np.ndarray:
    """reference.py:66-87: byte j = code[2j] | code[2j+1] << 4 (uint8 wrap-around)."""
    lo = codes[:, 0::2]
    hi = codes[:, 1::2]
    return ((hi << np.uint8(4)) | lo).astype(np.uint8)


def _nvfp4_candidate(X, bmax, amax, e2, e4, expansion):
    """reference.py:121-173.  Returns (y, scale_bytes, scale_f32)."""
    if amax == 0:
        hp = np.zeros(bmax.shape, dtype=F32)
    else:
        enc = F32(e2 * e4) / amax
        hp = (bmax / F32(e2)) * enc
    if expansion is not None:
        hp = hp * F32(expansion)
    sb = e4m3_encode(hp)
    sf = e4m3_decode(sb)
    with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
        dec = F32(1) / (F32(e2 * e4) / amax)
        r = F32(1) / (dec * sf)
        y = np.where((sf != 0)[:, None], X * r[:, None], F32(0)).astype(F32)
    return y, sb, sf


def quantize_blocks(X: np.ndarray, amax: np.float32, rule: str):
    """X: fp32 [nblocks, 16].  Returns (fake-quantized fp32 [nblocks,16], scale bytes [nblocks])."""
    X = np.ascontiguousarray(X, dtype=F32)
    amax = F32(amax)
    e2, e4 = rule_limits(rule)
    bmax = np.abs(X).max(axis=-1)
    if rule in ("static_6", "static_4"):
        y, sb, _ = _nvfp4_candidate(X, bmax, amax, e2, e4, None)
        return _fake_quantize_e2m1(y), sb
    y6, sb6, sf6 = _nvfp4_candidate(X, bmax, amax, e2, e4, None)
    y4, sb4, sf4 = _nvfp4_candidate(X, bmax, amax, e2, e4, 1.5)
    q6 = _fake_quantize_e2m1(y6)
    q4 = _fake_quantize_e2m1(y4)
    denom = F32(6 * 256)
    with np.errstate(invalid="ignore", over="ignore"):
        d6 = ((q6 * sf6[:, None]) * amax) / denom
        d4 = ((q4 * sf4[:, None]) * amax) / denom
        if rule == "abs_max":
            e4_ = np.abs(d4 - X).max(axis=-1)
            e6_ = np.abs(d6 - X).max(axis=-1)
        elif rule == "mae":
            e4_ = _seq_sum(np.abs(d4 - X))
            e6_ = _seq_sum(np.abs(d6 - X))
        elif rule == "mse":
            t4 = d4 - X
            t6 = d6 - X
            e4_ = _seq_sum(t4 * t4)
            e6_ = _seq_sum(t6 * t6)
        else:
            raise ValueError(rule)
    pick4 = e4_ < e6_
    q = np.where(pick4[:, None], q4, q6).astype(F32)
    sb = np.where(pick4, sb4, sb6).astype(np.uint8)
    return q, sb


def _seq_sum(t: np.ndarray) -> np.ndarray:
    """fp32 sum over the 16 block elements in the order torch's CPU reduction uses for a
    contiguous inner dimension of 16 floats: 256-bit lanes, i.e. p[i] = t[i] + t[i+8] for
    i = 0..7, then ((((0 + p[0]) + p[1]) + ...) + p[7]), one rounding per add.  The golden
    vectors under tests/golden (written by the reference itself) pin this order: the
    'adversarial' case holds only blocks whose 4-vs-6 choice flips under a plain
    left-to-right sum."""
    p = (t[:, :8] + t[:, 8:]).astype(F32)
    acc = np.zeros(t.shape[0], dtype=F32)
    for j in range(8):
        acc = (acc + p[:, j]).astype(F32)
    return acc


def quantize_to_fp4(x_bf16: np.ndarray, rule: str = "mse", amax=None):
    """Full entry (pytorch/backend.py:36-112 + reference.py:242-368) for a 2-D bf16 tensor
    given as uint16 bits.  Returns (values u8 [Mp, Kp/2], scales u8 [Mp*Kp/16] blocked,
    amax f32, padded_shape)."""
    x_bf16 = np.asarray(x_bf16, dtype=np.uint16)
    M, K = x_bf16.shape
    Mp = -(-M // 128) * 128
    Kp = -(-K // 64) * 64
    xp = np.zeros((Mp, Kp), dtype=np.uint16)
    xp[:M, :K] = x_bf16
    xf = bf16_to_f32(xp)
    if amax is None:
        amax = F32(np.abs(xf).max()) if xf.size else F32(0)
    amax = F32(amax)
    q, sb = quantize_blocks(xf.reshape(-1, 16), amax, rule)
    codes = _codes_from_fake_quantized(q).reshape(Mp, Kp)
    values = _pack(codes)
    scales = to_blocked(sb.reshape(Mp, Kp // 16))
    return values, scales, amax, (Mp, Kp)


# --------------------------------------------------------------------------- dequantize
def unpack_e2m1(values: np.ndarray) -> np.ndarray:
    """quantized_tensor.py:37-53: low nibble = even column."""
    lo = values & np.uint8(0xF)
    hi = values >> np.uint8(4)
    codes = np.stack([lo, hi], axis=-1).reshape(values.shape[0], values.shape[1] * 2)
    return E2M1_VALUES[codes]


def dequantize(values, scales_blocked, amax, rule, padded_shape, original_shape, dtype="f32"):
    """quantized_tensor.py:184-214.  dtype 'f32' or 'bf16' (returns fp32 holding bf16 values)."""
    Mp, Kp = padded_shape
    v = unpack_e2m1(values)
    s = e4m3_decode(from_blocked(np.asarray(scales_blocked, dtype=np.uint8), (Mp, Kp // 16)))
    res = v * np.repeat(s, 16, axis=1)  # exact in bf16 and fp32 (<= 6 significant bits)
    e2, e4 = rule_limits(rule)
    res = (res * F32(amax)) / F32(e2 * e4)
    if dtype == "bf16":
        res = round_bf16(res)
    return res[: original_shape[0], : original_shape[1]]


def fp4_matmul(a, b, out_bf16=True):
    """matmul/pytorch.py:22-41.  a, b are dicts with values/scales/amax/rule/padded/orig."""
    A = dequantize(a["values"], a["scales"], a["amax"], a["rule"], a["padded"], a["orig"])
    B = dequantize(b["values"], b["scales"], b["amax"], b["rule"], b["padded"], b["orig"])
    out = A @ B.T
    return round_bf16(out) if out_bf16 else out


def kv_global_scale(amax, rule="mse", path="fused"):
    """fp32 per-slot scale of the KV cache.  The reference has two code paths that differ in this one value:

    * "fused"  the CUDA extension, the path taken whenever it is built:
               amax * f32(1.0 / (e2m1_max * e4m3_max)), the reciprocal formed in double on the host
               (utils/kernel/kv_dequant_cuda.cu:95, 216);
    * "triton" the per-block fallback: amax / (e2m1_max * e4m3_max), an fp32 division (utils/quant.py:753-756).

    The two agree except where the rounded reciprocal tips the product over a rounding boundary (1 ulp)."""
    e2, e4 = rule_limits(rule)
    if path == "fused":
        return F32(F32(amax) * F32(1.0 / (e2 * e4)))
    if path == "triton":
        return F32(F32(amax) / F32(e2 * e4))
    raise ValueError(path)


def kv_dequantize(values, scales_blocked, amax, rule="mse", path="fused", dtype="bf16"):
    """One cache slot -> its dequantized values: (f32(e2m1) * f32(scale)) * global_scale, evaluated left to
    right in fp32 and cast (utils/kernel/kv_dequant_cuda.cu:97-106; utils/nvfp4_kernel.py:125-133 has the same
    expression).  The product of code and scale is exact, so the fp32 value carries one rounding.
    ``path`` selects how the global scale is formed (see kv_global_scale); dtype "bf16" or "f32"."""
    Mp = values.shape[0]
    Kp = values.shape[1] * 2
    v = unpack_e2m1(values)
    s = e4m3_decode(from_blocked(np.asarray(scales_blocked, dtype=np.uint8), (Mp, Kp // 16)))
    g = kv_global_scale(amax, rule, path)
    res = ((v * np.repeat(s, 16, axis=1)) * g).astype(F32)
    return round_bf16(res) if dtype == "bf16" else res


# --------------------------------------------------------------------------- attention
def attention(q, k, v, scale=None):
    """softmax(q k^T * scale) v per head, no mask (wan_5b/modules/attention.py:260-306).
    q [Lq,H,D], k/v [Lk,H,D] fp32 holding bf16 values; fp64 accumulation, bf16-rounded output."""
    Lq, H, D = q.shape
    scale = 1.0 / np.sqrt(D) if scale is None else scale
    out = np.empty((Lq, H, D), dtype=F32)
    for h in range(H):
        s = (q[:, h].astype(np.float64) @ k[:, h].astype(np.float64).T) * scale
        s -= s.max(axis=1, keepdims=True)
        p = np.exp(s)
        p /= p.sum(axis=1, keepdims=True)
        out[:, h] = (p @ v[:, h].astype(np.float64)).astype(F32)
    return round_bf16(out)


def k_smooth(k):
    """utils/quant.py:797-798 on bf16 tensors: mean over head_dim (fp32 accumulate, rounded to
    bf16), subtraction rounded to bf16."""
    mean = round_bf16(k.astype(F32).mean(axis=-1, keepdims=True, dtype=F32))
    return round_bf16(k - mean)


# --------------------------------------------------------------------------- RoPE / adaLN / RMSNorm
def rope_table(max_pos: int = 1024, head_dim: int = 128, theta: float = 10000.0):
    """Angles [max_pos, head_dim/2] in fp64: columns split [c-2(c//3), c//3, c//3] for
    (frame, height, width) (wan_5b/modules/model.py:29-36, causal_model.py:1075-1081)."""
    c = head_dim // 2
    parts = [c - 2 * (c // 3), c // 3, c // 3]
    cols = []
    pos = np.arange(max_pos, dtype=np.float64)[:, None]
    for p in parts:
        dim = 2 * p
        inv = 1.0 / np.power(theta, np.arange(0, dim, 2, dtype=np.float64) / dim)
        cols.append(pos * inv[None, :])
    return cols  # three arrays [max_pos, 22], [max_pos, 21], [max_pos, 21]


def rope_cos_sin(f, h, w, start_frame=0, head_dim=128, t_scale=1.0, temporal_offset=0.0):
    """fp32 cos/sin [f*h*w, head_dim/2], token order (f, h, w) row-major
    (causal_model.py:161-178, utils/rope_triton.py:84-91).  Temporal position of frame i:
    (start_frame + i + temporal_offset) * t_scale (utils/position_embedding_utils.py:55-107; the offset is a
    number or one value per frame of the chunk)."""
    tf, th, tw = rope_table(head_dim=head_dim)
    pos = (np.arange(f, dtype=np.float64) + start_frame + np.asarray(temporal_offset, dtype=np.float64)) * t_scale
    inv = tf[1]                      # angle per unit of position
    ang_t = pos[:, None] * inv[None, :]
    ang = np.concatenate(
        [
            np.broadcast_to(ang_t[:, None, None, :], (f, h, w, tf.shape[1])),
            np.broadcast_to(th[:h][None, :, None, :], (f, h, w, th.shape[1])),
            np.broadcast_to(tw[:w][None, None, :, :], (f, h, w, tw.shape[1])),
        ],
        axis=-1,
    ).reshape(f * h * w, -1)
    return np.cos(ang).astype(F32), np.sin(ang).astype(F32)


def rope_apply(x, cos, sin, seq_len=None):
    """utils/rope_triton.py:36-81: x [S,N,D] fp32 holding bf16; pairs (2j,2j+1) rotated in fp32,
    rows >= seq_len copied; bf16-rounded output."""
    S = x.shape[0]
    seq_len = S if seq_len is None else seq_len
    a = x[:seq_len, :, 0::2]
    b = x[:seq_len, :, 1::2]
    c = cos[:, None, :]
    s = sin[:, None, :]
    out = x.copy()
    out[:seq_len, :, 0::2] = (a * c).astype(F32) - (b * s).astype(F32)
    out[:seq_len, :, 1::2] = (a * s).astype(F32) + (b * c).astype(F32)
    return round_bf16(out)


def adaln_modulate(x, scale, shift, frame_seqlen, eps=1e-6):
    """utils/adaln_triton.py:36-86: x [L,C] fp32 holding bf16; scale/shift [F,C] bf16 values."""
    L, C = x.shape
    x = x.astype(F32)
    mean = x.sum(axis=1, keepdims=True, dtype=np.float64) / C
    xc = (x - mean.astype(F32)).astype(F32)
    var = (xc.astype(np.float64) ** 2).sum(axis=1, keepdims=True) / C
    rstd = (1.0 / np.sqrt(var + eps)).astype(F32)
    xn = round_bf16(xc * rstd)
    fidx = np.arange(L) // frame_seqlen
    sc = round_bf16(scale[fidx].astype(F32) + F32(1))
    prod = round_bf16(xn * sc)
    return round_bf16(prod + shift[fidx].astype(F32))


def gate_residual(x, y, gate, frame_seqlen):
    """wan_5b/modules/causal_model.py:889, 919-920: x + y * gate with the product and the sum each rounded
    to bf16.  x, y [L,C] and gate [F,C] hold bf16 values."""
    fidx = np.arange(x.shape[0]) // frame_seqlen
    prod = round_bf16(y.astype(F32) * gate[fidx].astype(F32))
    return round_bf16(x.astype(F32) + prod)


def rms_norm(x, weight, eps=1e-6):
    """wan_5b/modules/model.py:82-98: fp32 x*rsqrt(mean(x^2)+eps) -> bf16, times bf16 weight -> bf16."""
    x = x.astype(F32)
    ms = (x.astype(np.float64) ** 2).mean(axis=-1, keepdims=True)
    n = round_bf16(x * (1.0 / np.sqrt(ms + eps)).astype(F32))
    return round_bf16(n * weight.astype(F32))


def gelu_tanh(x):
    x64 = x.astype(np.float64)
    return round_bf16((0.5 * x64 * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (x64 + 0.044715 * x64**3)))).astype(F32))
