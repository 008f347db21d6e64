// NVFP4 -> bf16 / f16 / f32 dequantization for gfx950 (memory-bound helpers).
//
//  * ll_nvfp4_dequantize      QuantizedTensor.dequantize semantics
//                             (fouroversix/src/fouroversix/quantize/quantized_tensor.py:184-214)
//  * ll_kv_dequantize_blocks  multi-slot KV-cache dequantization
//                             (utils/kernel/kv_dequant_cuda.cu:59-107, utils/nvfp4_kernel.py:125-133)
#include <hip/hip_fp16.h>

#include "ll_common.h"

#pragma clang fp contract(off)

namespace ll {

template <int DT>
__device__ __forceinline__ void store8(void* out, int64_t off, const float (&v)[8]) {
  if (DT == LL_DTYPE_F32) {
    float4* p = reinterpret_cast<float4*>(static_cast<float*>(out) + off);
    p[0] = make_float4(v[0], v[1], v[2], v[3]);
    p[1] = make_float4(v[4], v[5], v[6], v[7]);
  } else {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (DT == LL_DTYPE_BF16) {
        w[i] = pack_bf16x2(v[2 * i], v[2 * i + 1]);
      } else {
        const __half2 h = __floats2half2_rn(v[2 * i], v[2 * i + 1]);
        w[i] = *reinterpret_cast<const uint32_t*>(&h);
      }
    }
    *reinterpret_cast<uint4*>(static_cast<uint16_t*>(out) + off) = make_uint4(w[0], w[1], w[2], w[3]);
  }
}

template <int DT>
__device__ __forceinline__ void store1(void* out, int64_t off, float v) {
  if (DT == LL_DTYPE_F32) {
    static_cast<float*>(out)[off] = v;
  } else if (DT == LL_DTYPE_BF16) {
    static_cast<uint16_t*>(out)[off] = (uint16_t)f32_to_bf16_bits(v);
  } else {
    static_cast<__half*>(out)[off] = __float2half_rn(v);
  }
}

// One thread = 8 consecutive elements (4 packed bytes) of one row.
template <int DT>
__global__ __launch_bounds__(256) void dequantize_kernel(const uint8_t* __restrict__ values,
                                                         const uint8_t* __restrict__ scales,
                                                         const float* __restrict__ amax, float denom, int64_t Kp,
                                                         int64_t M, int64_t K, void* __restrict__ out, int64_t ldo) {
  const int64_t groups_per_row = (K + 7) >> 3;
  const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (g >= M * groups_per_row) return;
  const int64_t r = g / groups_per_row;
  const int64_t c = (g - r * groups_per_row) * 8;
  const uint32_t packed = *reinterpret_cast<const uint32_t*>(values + r * (Kp >> 1) + (c >> 1));
  const float s = e4m3_to_f32(scales[blocked_scale_offset(r, c >> 4, Kp >> 4)]);
  const float a = amax[0];
  float v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float e = kE2M1[(packed >> (4 * i)) & 0xF];
    v[i] = ((e * s) * a) / denom;  // (v * s) exact, then * amax, then / (e2m1_max * e4m3_max)
  }
  const bool aligned = ((ldo & 7) == 0) && ((reinterpret_cast<uintptr_t>(out) & 31) == 0);
  if (c + 8 <= K && aligned) {
    store8<DT>(out, r * ldo + c, v);
  } else {
    for (int i = 0; i < 8 && c + i < K; ++i) store1<DT>(out, r * ldo + c + i, v[i]);
  }
}

// KV cache: slot rows are (token, head) pairs, 128 columns; output [slot*T + token, head, 128].
template <int DT>
__global__ __launch_bounds__(256) void kv_dequantize_kernel(const uint64_t* __restrict__ values_ptrs,
                                                            const uint64_t* __restrict__ scales_ptrs,
                                                            const uint64_t* __restrict__ amax_ptrs,
                                                            int64_t rows_per_slot, int64_t total_groups,
                                                            float inv_denom, void* __restrict__ out) {
  const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;  // group of 8 elements; 16 groups per row
  if (g >= total_groups) return;
  const int64_t grow = g >> 4;
  const int c = (int)(g & 15) * 8;
  const int64_t slot = grow / rows_per_slot;
  const int64_t r = grow - slot * rows_per_slot;
  const uint8_t* values = reinterpret_cast<const uint8_t*>(values_ptrs[slot]);
  const uint8_t* scales = reinterpret_cast<const uint8_t*>(scales_ptrs[slot]);
  const float amax = *reinterpret_cast<const float*>(amax_ptrs[slot]);
  const uint32_t packed = *reinterpret_cast<const uint32_t*>(values + r * 64 + (c >> 1));
  const float s = e4m3_to_f32(scales[blocked_scale_offset(r, c >> 4, 8)]);
  // The slot scale as the reference's fused path forms it: amax * f32(1 / (e2m1_max * e4m3_max))
  // (utils/kernel/kv_dequant_cuda.cu:95, 216), then (code * scale) * gs left to right (:97-106): the first product
  // is exact, so every value carries one fp32 rounding.  kv_attention_kernel decodes with the same expression.
  const float gs = amax * inv_denom;
  float v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = (kE2M1[(packed >> (4 * i)) & 0xF] * s) * gs;
  store8<DT>(out, grow * 128 + c, v);
}

}  // namespace ll

extern "C" int ll_nvfp4_dequantize(const uint8_t* values, const uint8_t* scales, const float* amax, int rule,
                                   int64_t Mp, int64_t Kp, int64_t M, int64_t K, void* out, int out_dtype,
                                   int64_t ldo, void* stream) {
  using namespace ll;
  LL_REQUIRE(values && scales && amax && out, "ll_nvfp4_dequantize: null pointer");
  LL_REQUIRE(Mp % 128 == 0 && Kp % 64 == 0 && M > 0 && K > 0 && M <= Mp && K <= Kp && ldo >= K,
             "ll_nvfp4_dequantize: bad shape Mp=%lld Kp=%lld M=%lld K=%lld ldo=%lld", (long long)Mp, (long long)Kp,
             (long long)M, (long long)K, (long long)ldo);
  LL_REQUIRE(rule >= 0 && rule <= 4, "ll_nvfp4_dequantize: unknown scale rule %d", rule);
  float e2, e4;
  rule_limits(rule, e2, e4);
  const float denom = e2 * e4;
  const int64_t groups = M * ((K + 7) / 8);
  const dim3 grid((unsigned)((groups + 255) / 256));
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (out_dtype) {
    case LL_DTYPE_BF16:
      hipLaunchKernelGGL(dequantize_kernel<LL_DTYPE_BF16>, grid, dim3(256), 0, s, values, scales, amax, denom, Kp, M, K,
                         out, ldo);
      break;
    case LL_DTYPE_F16:
      hipLaunchKernelGGL(dequantize_kernel<LL_DTYPE_F16>, grid, dim3(256), 0, s, values, scales, amax, denom, Kp, M, K,
                         out, ldo);
      break;
    case LL_DTYPE_F32:
      hipLaunchKernelGGL(dequantize_kernel<LL_DTYPE_F32>, grid, dim3(256), 0, s, values, scales, amax, denom, Kp, M, K,
                         out, ldo);
      break;
    default:
      LL_REQUIRE(false, "ll_nvfp4_dequantize: unknown dtype code %d", out_dtype);
  }
  LL_CHECK_LAUNCH("dequantize_kernel");
  return LL_OK;
}

extern "C" int ll_kv_dequantize_blocks(const uint64_t* values_ptrs, const uint64_t* scales_ptrs,
                                       const uint64_t* amax_ptrs, int n_blocks, int num_heads, int block_token_size,
                                       int out_dtype, float e2m1_max, float e4m3_max, void* out, void* stream) {
  using namespace ll;
  LL_REQUIRE(values_ptrs && scales_ptrs && amax_ptrs && out, "ll_kv_dequantize_blocks: null pointer");
  LL_REQUIRE(n_blocks > 0 && num_heads > 0 && block_token_size > 0, "ll_kv_dequantize_blocks: bad sizes");
  LL_REQUIRE(e2m1_max > 0.f && e4m3_max > 0.f, "ll_kv_dequantize_blocks: e2m1_max and e4m3_max must be positive");
  const int64_t rows_per_slot = (int64_t)num_heads * block_token_size;
  const int64_t groups = rows_per_slot * n_blocks * 16;
  const dim3 grid((unsigned)((groups + 255) / 256));
  const float inv_denom = kv_inverse_denominator(e2m1_max, e4m3_max);
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (out_dtype) {
    case LL_DTYPE_BF16:
      hipLaunchKernelGGL(kv_dequantize_kernel<LL_DTYPE_BF16>, grid, dim3(256), 0, s, values_ptrs, scales_ptrs,
                         amax_ptrs, rows_per_slot, groups, inv_denom, out);
      break;
    case LL_DTYPE_F16:
      hipLaunchKernelGGL(kv_dequantize_kernel<LL_DTYPE_F16>, grid, dim3(256), 0, s, values_ptrs, scales_ptrs,
                         amax_ptrs, rows_per_slot, groups, inv_denom, out);
      break;
    case LL_DTYPE_F32:
      hipLaunchKernelGGL(kv_dequantize_kernel<LL_DTYPE_F32>, grid, dim3(256), 0, s, values_ptrs, scales_ptrs,
                         amax_ptrs, rows_per_slot, groups, inv_denom, out);
      break;
    default:
      LL_REQUIRE(false, "ll_kv_dequantize_blocks: unknown dtype code %d", out_dtype);
  }
  LL_CHECK_LAUNCH("kv_dequantize_kernel");
  return LL_OK;
}
