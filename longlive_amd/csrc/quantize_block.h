// Quantization of one block of 16 values to NVFP4 (scale byte and 16 e2m1 codes) under the five scale rules,
// shared by every kernel that writes packed NVFP4.  Arithmetic follows the reference's PyTorch backend
// (fouroversix/src/fouroversix/quantize/pytorch/reference.py:121-368) operation by operation.
//
// Files that include this must be compiled without floating-point contraction.
#pragma once
#include "ll_common.h"

#pragma clang fp contract(off)

namespace ll {

// ----------------------------------------------------------------------------- exact block math
// reference.py:18-34, nearest rounding: the e2m1 grid with half-to-even ties, no clamp at 6.
__device__ __forceinline__ float fake_quantize_e2m1(float y) {
  const float a = fabsf(y);
  float q;
  if (a < 2.0f) {
    q = __builtin_rintf(2.0f * a) / 2.0f;
  } else if (a < 4.0f) {
    q = __builtin_rintf(a);
  } else {
    q = 2.0f * __builtin_rintf(a / 2.0f);
  }
  return y > 0.0f ? q : (y < 0.0f ? -q : 0.0f);  // sign(y) * q with sign(+-0) = 0
}

// reference.py:37-63: the 4-bit code is read from the bf16 bit pattern of q with 16-bit integer
// arithmetic and truncated to 8 bits; values of |q| >= 8 overflow the nibble exactly as there.
__device__ __forceinline__ uint32_t code_from_q(float q) {
  const int32_t bx = (int32_t)(int16_t)f32_to_bf16_bits(q);
  int32_t s = (bx >> 15) & 1;
  int32_t e = (bx >> 7) & 0xFF;
  int32_t m = bx & 0x7F;
  const bool is_zero = (e == 0) && (m == 0);
  m = (m >> 6) & 1;
  if (e == 126 && m == 0) m = 1;
  e -= 126;
  if (is_zero) {
    e = 0;
    m = 0;
  }
  return (uint32_t)((s << 3) | (e << 1) | m) & 0xFFu;
}

struct Candidate {
  float q[16];
  uint32_t scale_byte;
  float scale;
};

// reference.py:121-173 for one block.  hp is the high-precision scale (already expanded by 1.5 for the
// "4" candidate); dec = 1 / (E2*E4 / amax).
__device__ __forceinline__ void make_candidate(const float (&X)[16], float hp, float dec, Candidate& c) {
  c.scale_byte = f32_to_e4m3(hp);
  c.scale = e4m3_to_f32(c.scale_byte);
  const float r = 1.0f / (dec * c.scale);
  const bool nz = c.scale != 0.0f;  // torch.where(scales != 0, x * r, 0); a NaN scale compares != 0
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const float y = nz ? X[i] * r : 0.0f;
    c.q[i] = fake_quantize_e2m1(y);
  }
}

// reference.py:196-225: error of one candidate against the block, summed in the order torch's CPU
// reduction uses for 16 contiguous floats (p[i] = t[i] + t[i+8], then p[0] + p[1] + ... + p[7]).
template <int RULE>
__device__ __forceinline__ float candidate_error(const float (&X)[16], const Candidate& c, float amax) {
  float t[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const float d = ((c.q[i] * c.scale) * amax) / 1536.0f;
    const float e = d - X[i];
    t[i] = (RULE == LL_RULE_MSE) ? e * e : fabsf(e);
  }
  if (RULE == LL_RULE_ABS_MAX) {
    float m = t[0];
#pragma unroll
    for (int i = 1; i < 16; ++i) m = fmaxf(m, t[i]);
    return m;
  }
  float acc = t[0] + t[8];
#pragma unroll
  for (int i = 1; i < 8; ++i) acc = acc + (t[i] + t[i + 8]);
  return acc;
}

// Quantize one block of 16 values; returns the 8 packed bytes (lo, hi) and the scale byte.
// enc = (E2 * E4) / amax and dec = 1 / enc do not depend on the block; the kernel forms them once.
template <int RULE>
__device__ __forceinline__ void quantize_block(const float (&X)[16], float amax, float enc, float dec, uint32_t& lo,
                                               uint32_t& hi, uint32_t& scale_byte) {
  constexpr bool kStatic = (RULE == LL_RULE_STATIC_6 || RULE == LL_RULE_STATIC_4);
  constexpr float E2 = (RULE == LL_RULE_STATIC_4) ? 4.0f : 6.0f;
  float bmax = fabsf(X[0]);
#pragma unroll
  for (int i = 1; i < 16; ++i) bmax = fmaxf(bmax, fabsf(X[i]));
  const float hp = (amax == 0.0f) ? 0.0f : (bmax / E2) * enc;

  Candidate c6;
  make_candidate(X, hp, dec, c6);
  const Candidate* pick = &c6;
  Candidate c4;
  if (!kStatic) {
    make_candidate(X, hp * 1.5f, dec, c4);
    const float e4 = candidate_error<RULE>(X, c4, amax);
    const float e6 = candidate_error<RULE>(X, c6, amax);
    if (e4 < e6) pick = &c4;
  }
  uint32_t b[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const uint32_t cl = code_from_q(pick->q[2 * j]);
    const uint32_t ch = code_from_q(pick->q[2 * j + 1]);
    b[j] = ((ch << 4) | cl) & 0xFFu;  // uint8 arithmetic of reference.py:85-87
  }
  lo = b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24);
  hi = b[4] | (b[5] << 8) | (b[6] << 16) | (b[7] << 24);
  scale_byte = pick->scale_byte;
}

// ----------------------------------------------------------------------------- fast block math
// Same results as quantize_block above, with the per-element divisions and software codecs replaced:
//
//  * everything that depends only on the scale byte s and the tensor amax is tabulated once per
//    workgroup for the 127 finite e4m3 values:  r(s) = 1 / (dec * f32(s)),  d1(s) = ((1 * s) * amax) / 1536,
//    d3(s) = ((1.5 * s) * amax) / 1536, each computed with the reference's operations;
//  * the dequantized value ((q * s) * amax) / 1536 of an e2m1 value q = m * 2^k (m = 1 or 1.5) equals
//    2^k * d1(s) or 2^k * d3(s) exactly (scaling by a power of two commutes with both roundings while
//    nothing under- or overflows, which the caller guarantees by bounding amax);
//  * fp32 -> e4m3 and fp32 -> e2m1 use the gfx950 conversion instructions, which round to nearest even
//    like the reference (checked exhaustively by the test-suite); they saturate, where the reference
//    produces out-of-range codes for |y| >= 7, so such blocks are sent to the exact path;
//  * y = fma(x, r, +0) equals x * r and turns -0 into +0, which is what sign(y) * |q| does there;
//  * bmax / 6 = fma(fma(-6, q0, bmax), 1/6, q0) with q0 = bmax * (1/6) is the correctly rounded
//    quotient for every fp32 bmax (verified exhaustively on the CPU).
struct ScaleEntry {
  float r, d1, d3, w;  // w = d1 * d1
};

typedef float float2v __attribute__((ext_vector_type(2)));

// Codes of one candidate (scale entry e) and, for the rules that choose between candidates, a cheap
// estimate of its error in units of the candidate's own step: sum (q - y)^2, sum |q - y| or max |q - y| with
// y = x * r the scaled value the codes were rounded from.
template <int RULE>
__device__ __forceinline__ float encode_candidate(const float (&X)[16], const ScaleEntry& e, uint32_t& lo,
                                                  uint32_t& hi) {
  float y[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) y[i] = __builtin_fmaf(X[i], e.r, 0.0f);
  lo = 0;
  hi = 0;
#define LL_PACK(dst, base, k) \
  dst = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(dst, y[base + 2 * k], y[base + 2 * k + 1], 1.0f, k)
  LL_PACK(lo, 0, 0);
  LL_PACK(lo, 0, 1);
  LL_PACK(lo, 0, 2);
  LL_PACK(lo, 0, 3);
  LL_PACK(hi, 8, 0);
  LL_PACK(hi, 8, 1);
  LL_PACK(hi, 8, 2);
  LL_PACK(hi, 8, 3);
#undef LL_PACK
  constexpr bool kStatic = (RULE == LL_RULE_STATIC_6 || RULE == LL_RULE_STATIC_4);
  if (kStatic) return 0.0f;
  float acc = 0.0f;
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    float2v q;
    switch (k & 3) {
      case 0: q = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(k < 4 ? lo : hi, 1.0f, 0); break;
      case 1: q = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(k < 4 ? lo : hi, 1.0f, 1); break;
      case 2: q = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(k < 4 ? lo : hi, 1.0f, 2); break;
      default: q = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(k < 4 ? lo : hi, 1.0f, 3); break;
    }
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const float d = q[h] - y[2 * k + h];
      if (RULE == LL_RULE_MSE) {
        acc = __builtin_fmaf(d, d, acc);
      } else if (RULE == LL_RULE_MAE) {
        acc += fabsf(d);
      } else {
        acc = fmaxf(acc, fabsf(d));
      }
    }
  }
  return acc;
}

// The reference's error of a candidate whose codes are lo / hi: dequantize with the reference's operations,
// subtract, square or take the magnitude, reduce in the reference's order.
template <int RULE>
__device__ __forceinline__ float exact_error(const float (&X)[16], const ScaleEntry& e, uint32_t lo, uint32_t hi) {
  float t[16];
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    float2v q;
    switch (k & 3) {
      case 0: q = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(k < 4 ? lo : hi, 1.0f, 0); break;
      case 1: q = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(k < 4 ? lo : hi, 1.0f, 1); break;
      case 2: q = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(k < 4 ? lo : hi, 1.0f, 2); break;
      default: q = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(k < 4 ? lo : hi, 1.0f, 3); break;
    }
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const float qv = q[h];
      const float p = __uint_as_float(__float_as_uint(qv) & 0xFF800000u);  // sign and power of two of q
      const float d = p * ((qv != p) ? e.d3 : e.d1);
      const float err = d - X[2 * k + h];
      t[2 * k + h] = (RULE == LL_RULE_MSE) ? err * err : fabsf(err);
    }
  }
  if (RULE == LL_RULE_ABS_MAX) {
    float m = t[0];
#pragma unroll
    for (int i = 1; i < 16; ++i) m = fmaxf(m, t[i]);
    return m;
  }
  float acc = t[0] + t[8];
#pragma unroll
  for (int i = 1; i < 8; ++i) acc = acc + (t[i] + t[i + 8]);
  return acc;
}

// Four-over-six choice.  The reference compares the two candidates' errors as it computes them in fp32
// (exact_error).  The estimates of encode_candidate, multiplied by the candidate's weight w (the step d1 of the
// candidate, squared for mse), are the same quantities up to rounding.  With u = 2^-24, D the real-number step
// s * amax / 1536 and a* = sum (q - x / D)^2 the real-number error in step units:
//   * y = fl(x * r) carries five roundings (1536 / amax, its reciprocal, the product with s, the reciprocal of
//     that, the product with x) and |y| < 7, so |y - x / D| <= 35 u and the estimate a = sum (q - y)^2, 17 more
//     roundings of its own, lies within 2 * 35 u * sum |q - x / D| + 18 u a* <= 280 u sqrt(a*) + 18 u a* of a*
//     (Cauchy-Schwarz over the 16 terms);
//   * the reference's dequantized value q D (1 + 2u) (q * s is exact, two roundings follow) gives errors
//     D (q - x / D + q eps) with |q eps| <= 12 u, so its sum of squares, 18 more roundings, lies within
//     D^2 (96 u sqrt(a*) + 19 u a*) of D^2 a*;
//   * w = fl(d1 * d1) = D^2 (1 + 5u) and E = fl(a * w) add 6 u E.
// Hence both E and the reference's value lie within B = (320 u sqrt(a) + 32 u a) w + 8 u E of the real-number
// error D^2 a*, and when |E4 - E6| exceeds 2 (B4 + B6) the reference's comparison has the same outcome.  The
// kernel asks for twice that and bounds the square root by 2 sqrt(a) <= 1 + a, which gives the margin
//     mse: 640 u (w4 + w6) + 800 u (E4 + E6)
// (mae, whose terms are |q - y| instead of squares: B = (640 u + 32 u a) w + 8 u E, the same derivation with
// sum |.| <= 16 * 35 u in place of the Cauchy-Schwarz step).  Blocks inside the margin (a few in 10^4 of
// Gaussian data) are decided by exact_error.  `approx_ok` is false when the tensor amax is so small or large
// that squares could leave the normal fp32 range; then every block is decided by exact_error.
template <int RULE>
__device__ __forceinline__ bool pick_four(const float (&X)[16], const ScaleEntry& e6, const ScaleEntry& e4, float a6,
                                          float a4, uint32_t lo6, uint32_t hi6, uint32_t lo4, uint32_t hi4,
                                          bool approx_ok) {
  constexpr float u = 0x1p-24f;
  // abs_max compares two maxima over values that sit on a coarse grid (bf16 inputs): exact ties are common
  // (a few percent of the blocks), so that rule always takes the reference's arithmetic.
  if (RULE != LL_RULE_ABS_MAX) {
    const float w6 = (RULE == LL_RULE_MSE) ? e6.w : e6.d1;
    const float w4 = (RULE == LL_RULE_MSE) ? e4.w : e4.d1;
    const float E6 = a6 * w6, E4 = a4 * w4;
    float margin;
    if (RULE == LL_RULE_MSE) {
      margin = __builtin_fmaf(800.0f * u, E6 + E4, (640.0f * u) * (w6 + w4)) + 0x1p-100f;
    } else {
      const float b6 = 640.0f * u + 32.0f * u * a6, b4 = 640.0f * u + 32.0f * u * a4;
      margin = 4.0f * (b6 * w6 + b4 * w4 + 8.0f * u * (E6 + E4)) + 0x1p-100f;
    }
    if (approx_ok && fabsf(E4 - E6) > margin) return E4 < E6;
  }
  return exact_error<RULE>(X, e4, lo4, hi4) < exact_error<RULE>(X, e6, lo6, hi6);
}

// Returns false when the block has to take the exact path (an element would round past the e2m1 range).
// `bound`: the tensor amax when the caller supplied it (it need not be the true maximum: a block that exceeds it
// would get a scale beyond the e4m3 range, where the hardware conversion saturates and the reference does not),
// infinity when the amax was computed from the tensor.
template <int RULE>
__device__ __forceinline__ bool quantize_block_fast(const float (&X)[16], float enc, const ScaleEntry* tab,
                                                    bool approx_ok, float bound, uint32_t& lo, uint32_t& hi,
                                                    uint32_t& scale_byte) {
  constexpr bool kStatic = (RULE == LL_RULE_STATIC_6 || RULE == LL_RULE_STATIC_4);
  float bmax = fabsf(X[0]);
#pragma unroll
  for (int i = 1; i < 16; ++i) bmax = fmaxf(bmax, fabsf(X[i]));
  if (!(bmax <= bound)) return false;
  float quot;
  if (RULE == LL_RULE_STATIC_4) {
    quot = bmax * 0.25f;
  } else {
    const float c = 1.0f / 6.0f;
    const float q0 = bmax * c;
    quot = __builtin_fmaf(__builtin_fmaf(-6.0f, q0, bmax), c, q0);
  }
  const float hp = quot * enc;
  const uint32_t sb2 = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(hp, hp * 1.5f, 0, false);
  const uint32_t s6 = sb2 & 0xFFu, s4 = (sb2 >> 8) & 0xFFu;
  const ScaleEntry e6 = tab[s6];
  if (!(bmax * e6.r < 7.0f)) return false;
  if (kStatic) {
    encode_candidate<RULE>(X, e6, lo, hi);
    scale_byte = s6;
    return true;
  }
  const ScaleEntry e4 = tab[s4];
  if (!(bmax * e4.r < 7.0f)) return false;
  uint32_t lo4, hi4;
  const float a6 = encode_candidate<RULE>(X, e6, lo, hi);
  const float a4 = encode_candidate<RULE>(X, e4, lo4, hi4);
  // Equal scale bytes (blocks small enough for the subnormal end of e4m3) make the candidates identical: the
  // reference's strict comparison then keeps "6".  A zero scale byte (block far below the tensor amax) has
  // r = 0: its estimate says nothing about the error.
  const bool pick4 = s4 != s6 && pick_four<RULE>(X, e6, e4, a6, a4, lo, hi, lo4, hi4, approx_ok && s6 != 0);
  lo = pick4 ? lo4 : lo;
  hi = pick4 ? hi4 : hi;
  scale_byte = pick4 ? s4 : s6;
  return true;
}

// The fast path's table of the 128 non-negative e4m3 scale bytes for a tensor amax: filled by 256 threads (entry
// threadIdx.x % 128: the lower half of the workgroup fills r, d1 and w, the upper half d3); the caller puts a
// barrier behind it.
template <int RULE>
__device__ __forceinline__ void fill_scale_table(ScaleEntry* tab, float amax, float dec) {
  constexpr bool kStaticRule = (RULE == LL_RULE_STATIC_6 || RULE == LL_RULE_STATIC_4);
  const uint32_t idx = threadIdx.x & 127;
  const float sf = e4m3_to_f32(idx);
  if (threadIdx.x < 128) {
    const float d1 = (sf * amax) / 1536.0f;
    tab[idx].r = (idx == 0 || idx == 127) ? 0.0f : 1.0f / (dec * sf);
    tab[idx].d1 = d1;
    tab[idx].w = d1 * d1;
  } else if (!kStaticRule) {
    tab[idx].d3 = ((1.5f * sf) * amax) / 1536.0f;
  }
}

}  // namespace ll
