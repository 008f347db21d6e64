// Row operations shared by the normalization kernels and by the kernel that normalizes and quantizes in one
// launch: one wave computes one row, a lane holds NCH groups of 8 consecutive elements (group lane + 64 i).
// The order of every floating-point operation is part of the result (the sums are not associative), so every
// kernel that needs a row calls these.
#pragma once
#include "ll_common.h"

#pragma clang fp contract(off)

namespace ll {

__device__ __forceinline__ void unpack8(const uint4& v, float (&f)[8]) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = __uint_as_float(w[i] << 16);
    f[2 * i + 1] = __uint_as_float(w[i] & 0xFFFF0000u);
  }
}
__device__ __forceinline__ uint4 pack8(const float (&f)[8]) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) w[i] = pack_bf16x2(f[2 * i], f[2 * i + 1]);
  return make_uint4(w[0], w[1], w[2], w[3]);
}

// Row kernels: one wave per row (no workgroup barrier; a row's sums are wave reductions), four rows per
// workgroup.  A lane holds NCH groups of 8 elements: NCH = 6 covers C = 3072 exactly, 16 anything up to 8192.
constexpr int kRowThreads = 256;
constexpr int kRowsPerWg = kRowThreads / 64;
constexpr int kMaxChunks = 16;  // 8 elements each: C <= 64 * 16 * 8 = 8192
constexpr int kMaxRowLength = 64 * kMaxChunks * 8;

// adaLN modulation of one row, utils/adaln_triton.py:36-86: LayerNorm without affine in fp32, rounded to bf16,
// times (1 + scale) rounded, plus shift rounded.  `packed[i]` receives the 8 results of group lane + 64 i; the
// return value is the lane's share of the row's absolute maximum.
template <int NCH>
__device__ __forceinline__ float adaln_row(const uint16_t* __restrict__ xr, const uint16_t* __restrict__ scr,
                                           const uint16_t* __restrict__ shr, int C, float eps, int add_one, int lane,
                                           uint4 (&packed)[NCH]) {
  const int nchunks = C >> 3;
  float v[NCH][8];
  uint4 sraw[NCH], hraw[NCH];  // requested up front: their latency runs under the two reductions
  float sum = 0.0f;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = lane + i * 64;
    if (c < nchunks) {
      unpack8(*reinterpret_cast<const uint4*>(xr + c * 8), v[i]);
      sraw[i] = *reinterpret_cast<const uint4*>(scr + c * 8);
      hraw[i] = *reinterpret_cast<const uint4*>(shr + c * 8);
#pragma unroll
      for (int j = 0; j < 8; ++j) sum += v[i][j];
    }
  }
  const float inv_c = 1.0f / (float)C;
  const float mean = wave_sum_dpp(sum) * inv_c;
  float sq = 0.0f;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = lane + i * 64;
    if (c < nchunks) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        v[i][j] -= mean;
        sq += v[i][j] * v[i][j];
      }
    }
  }
  const float var = wave_sum_dpp(sq) * inv_c;
  const float rstd = 1.0f / sqrtf(var + eps);
  float out_max = 0.0f;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = lane + i * 64;
    packed[i] = make_uint4(0u, 0u, 0u, 0u);
    if (c < nchunks) {
      float s8[8], h8[8], y[8];
      unpack8(sraw[i], s8);
      unpack8(hraw[i], h8);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float xn = round_to_bf16(v[i][j] * rstd);
        const float s = add_one ? round_to_bf16(s8[j] + 1.0f) : s8[j];
        const float prod = round_to_bf16(xn * s);
        y[j] = prod + h8[j];
      }
      packed[i] = pack8(y);
      out_max = abs_max_bf16x8(packed[i], out_max);
    }
  }
  return out_max;
}

// LayerNorm with optional weight and bias of one row, wan_5b/modules/model.py:101-111 (nn.LayerNorm on bf16
// tensors: statistics and the affine map in fp32, one rounding to bf16 at the end).
template <int NCH>
__device__ __forceinline__ float layernorm_row(const uint16_t* __restrict__ xr, const uint16_t* __restrict__ w,
                                               const uint16_t* __restrict__ b, int C, float eps, int lane,
                                               uint4 (&packed)[NCH]) {
  const int nchunks = C >> 3;
  float v[NCH][8];
  uint4 wraw[NCH], braw[NCH];  // requested up front: their latency runs under the two reductions
  float sum = 0.0f;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = lane + i * 64;
    if (c < nchunks) {
      unpack8(*reinterpret_cast<const uint4*>(xr + c * 8), v[i]);
      wraw[i] = w ? *reinterpret_cast<const uint4*>(w + c * 8) : make_uint4(0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u);
      braw[i] = b ? *reinterpret_cast<const uint4*>(b + c * 8) : make_uint4(0, 0, 0, 0);
#pragma unroll
      for (int j = 0; j < 8; ++j) sum += v[i][j];
    }
  }
  const float inv_c = 1.0f / (float)C;
  const float mean = wave_sum_dpp(sum) * inv_c;
  float sq = 0.0f;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = lane + i * 64;
    if (c < nchunks) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        v[i][j] -= mean;
        sq += v[i][j] * v[i][j];
      }
    }
  }
  const float var = wave_sum_dpp(sq) * inv_c;
  const float rstd = 1.0f / sqrtf(var + eps);
  float out_max = 0.0f;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = lane + i * 64;
    packed[i] = make_uint4(0u, 0u, 0u, 0u);
    if (c < nchunks) {
      float w8[8], b8[8], y[8];
      unpack8(wraw[i], w8);
      unpack8(braw[i], b8);
#pragma unroll
      for (int j = 0; j < 8; ++j) y[j] = (v[i][j] * rstd) * w8[j] + b8[j];
      packed[i] = pack8(y);
      out_max = abs_max_bf16x8(packed[i], out_max);
    }
  }
  return out_max;
}

}  // namespace ll
