// Probe (not part of the library): which f16 MFMA shape delivers more under the chip's power limit.
// v_mfma_f32_32x32x16_f16 (32 cycles) against two v_mfma_f32_16x16x32_f16 (16 cycles each) - the same flops - with
// N decode instructions (FP4 conversion / packed multiply, alternating) per 32 MFMA cycles, on every compute unit,
// two waves per SIMD, for a quarter of a second per case; operands are random decoded-FP4 values (e2m1 code x e4m3
// scale as f16) or all zero (same instructions, nothing switching in the multipliers: the issue-bound figure).
// Build: make -C longlive_amd/csrc probes      Run: ./longlive_amd/csrc/probe_mfma_shape
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <vector>
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef float float4v __attribute__((ext_vector_type(4)));
#define CHECK(x) do { hipError_t e__ = (x); if (e__ != hipSuccess) { printf("%s: %s\n", #x, hipGetErrorString(e__)); exit(1); } } while (0)

template <int SHAPE, int NV>
__global__ __launch_bounds__(512) void k(const half8* __restrict__ ops, float* out, int iters) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  half8 a[4], b[4];
  for (int i = 0; i < 4; ++i) { a[i] = ops[(t * 8 + i) & 0xFFFF]; b[i] = ops[(t * 8 + 4 + i) & 0xFFFF]; }
  uint32_t w = __builtin_bit_cast(uint4, a[0]).x, dd[8] = {0, 1, 2, 3, 4, 5, 6, 7};
  float r = 0;
  if (SHAPE == 32) {
    float16v acc[8];
    for (int i = 0; i < 8; ++i) for (int j = 0; j < 16; ++j) acc[i][j] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(acc[i]) : "v"(a[i & 3]), "v"(b[(i >> 1) & 3]));
#pragma unroll
        for (int v = 0; v < NV; ++v) {
          uint32_t& d = dd[(i * NV + v) & 7];
          if (v & 1) asm volatile("v_pk_mul_f16 %0, %1, %1" : "+v"(d) : "v"(w));
          else asm volatile("v_cvt_scalef32_pk_f16_fp4 %0, %1, 1.0" : "+v"(d) : "v"(w));
        }
      }
    }
    for (int i = 0; i < 8; ++i) for (int j = 0; j < 16; ++j) r += acc[i][j];
  } else {
    float4v acc[16];
    for (int i = 0; i < 16; ++i) for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(acc[i]) : "v"(a[i & 3]), "v"(b[(i >> 2) & 3]));
#pragma unroll
        for (int v = (i & 1) * (NV / 2); v < ((i & 1) ? NV : NV / 2); ++v) {
          uint32_t& d = dd[(i * NV + v) & 7];
          if (v & 1) asm volatile("v_pk_mul_f16 %0, %1, %1" : "+v"(d) : "v"(w));
          else asm volatile("v_cvt_scalef32_pk_f16_fp4 %0, %1, 1.0" : "+v"(d) : "v"(w));
        }
      }
    }
    for (int i = 0; i < 16; ++i) for (int j = 0; j < 4; ++j) r += acc[i][j];
  }
  out[t] = r + (float)(dd[0] ^ dd[1] ^ dd[2] ^ dd[3] ^ dd[4] ^ dd[5] ^ dd[6] ^ dd[7]);
}

template <int SHAPE, int NV>
void run(const half8* d, float* o, const char* what, int waves_per_simd) {
  hipEvent_t e0, e1; CHECK(hipEventCreate(&e0)); CHECK(hipEventCreate(&e1));
  const int iters = 20000, launches = 12;   // ~ a quarter of a second
  hipLaunchKernelGGL((k<SHAPE, NV>), dim3(256), dim3(256 * waves_per_simd), 0, 0, d, o, iters);
  CHECK(hipEventRecord(e0));
  for (int l = 0; l < launches; ++l) hipLaunchKernelGGL((k<SHAPE, NV>), dim3(256), dim3(256 * waves_per_simd), 0, 0, d, o, iters);
  CHECK(hipEventRecord(e1)); CHECK(hipEventSynchronize(e1));
  float ms; CHECK(hipEventElapsedTime(&ms, e0, e1));
  const double units = 256.0 * 4 * waves_per_simd * iters * 8.0 * launches;  // units of 32 MFMA cycles = 32768 flops each... per wave
  const double flops = units * 2.0 * 32 * 32 * 16;
  printf("%s %dx%d + %d decode per 32 MFMA cycles, %d wave(s)/SIMD: %.1f ms, %.0f TFLOP/s, %.1f nominal cycles per unit\n", what, SHAPE, SHAPE, NV,
         waves_per_simd, ms, flops / ms / 1e9, ms * 1e-3 * 2.4e9 / (iters * 8.0 * launches * waves_per_simd));
}

int main() {
  const int n = 1 << 16;
  std::vector<_Float16> h(n * 8);
  srand(1);
  const float codes[8] = {0.f, .5f, 1.f, 1.5f, 2.f, 3.f, 4.f, 6.f};
  for (auto& v : h) { float c = codes[rand() & 7] * ((rand() & 1) ? -1.f : 1.f) * (1.0f + (rand() & 7) / 8.0f) * (1 << (rand() % 5)); v = (_Float16)c; }
  half8* d; float* o;
  CHECK(hipMalloc(&d, n * 16)); CHECK(hipMalloc(&o, 256 * 512 * 4));
  CHECK(hipMemcpy(d, h.data(), n * 16, hipMemcpyHostToDevice));
  for (int rep = 0; rep < 2; ++rep) {
    run<32, 0>(d, o, "random", 2); run<16, 0>(d, o, "random", 2);
    run<32, 4>(d, o, "random", 2); run<16, 4>(d, o, "random", 2);
    run<32, 6>(d, o, "random", 2); run<16, 6>(d, o, "random", 2);
    run<32, 8>(d, o, "random", 2); run<16, 8>(d, o, "random", 2);
    run<16, 6>(d, o, "random", 2); run<32, 6>(d, o, "random", 2);
    run<32, 4>(d, o, "random", 1); run<16, 4>(d, o, "random", 1);
  }
  CHECK(hipMemset(d, 0, n * 16));
  run<32, 0>(d, o, "zero", 2); run<16, 0>(d, o, "zero", 2);
  run<32, 6>(d, o, "zero", 2); run<16, 6>(d, o, "zero", 2);
  run<32, 8>(d, o, "zero", 2); run<16, 8>(d, o, "zero", 2);
  return 0;
}
