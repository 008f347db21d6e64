// Test-only library (libll_nvfp4_testhooks.so), not part of the product ABI: applies the gfx950 conversion
// instructions the quantizer's fast path relies on to raw floats, so that the GPU tests can compare them with the
// software e4m3 / e2m1 codecs value by value.
#include <hip/hip_runtime.h>
#include <stdint.h>

__global__ void convert_kernel(const float* __restrict__ in, int64_t n, int mode, uint8_t* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const float v = in[i];
  if (mode == 0) {
    out[i] = (uint8_t)(__builtin_amdgcn_cvt_pk_fp8_f32(v, 0.0f, 0, false) & 0xFF);
  } else {
    out[i] = (uint8_t)(__builtin_amdgcn_cvt_scalef32_pk_fp4_f32(0u, v, 0.0f, 1.0f, 0) & 0xF);
  }
}

// mode 0: fp32 -> e4m3 byte (v_cvt_pk_fp8_f32), mode 1: fp32 -> e2m1 nibble (v_cvt_scalef32_pk_fp4_f32).
// Returns 0, -1 for bad arguments, -2 when the launch fails.
extern "C" int ll_test_convert(const float* in, int64_t n, int mode, uint8_t* out, void* stream) {
  if (!in || !out || n <= 0 || (mode != 0 && mode != 1)) return -1;
  hipLaunchKernelGGL(convert_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                     in, n, mode, out);
  return hipGetLastError() == hipSuccess ? 0 : -2;
}
