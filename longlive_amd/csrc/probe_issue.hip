// Probe (not part of the library): what a gfx950 SIMD issues per cycle, measured with hand-placed instructions.
//   * one wave and two waves per SIMD issuing nothing but v_pk_mul_f16, v_cvt_scalef32_pk_f16_fp4 or
//     v_cvt_scalef32_pk_f16_fp8 (independent destinations): cycles per instruction;
//   * v_mfma_f32_32x32x16_f16 on eight independent accumulators with N other vector instructions behind every MFMA
//     (N = 0 .. 8; conversions, packed multiplies, or alternating): cycles per MFMA.
// The W4A4 GEMM decodes its operands in registers (conversion + packed multiply per pair of elements), so the second
// table is the budget that decides the tile shape: how many decode instructions an MFMA can carry.
// Cycles are wall time x the nominal 2.4 GHz; the MFMA-only line shows what that assumption is worth under load.
// Build: make -C longlive_amd/csrc probes      Run: ./longlive_amd/csrc/probe_issue
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
typedef _Float16 half8v __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));

#define REP8(x) x x x x x x x x
__global__ void k_cvt4(int iters, uint32_t* out) {
  uint32_t w = threadIdx.x * 2654435761u, a0, a1, a2, a3, a4, a5, a6, a7;
  for (int it = 0; it < iters; ++it) {
    REP8(asm volatile("v_cvt_scalef32_pk_f16_fp4 %0, %8, 1.0\n v_cvt_scalef32_pk_f16_fp4 %1, %8, 1.0 op_sel:[1,0,0]\n"
                      "v_cvt_scalef32_pk_f16_fp4 %2, %8, 1.0 op_sel:[0,1,0]\n v_cvt_scalef32_pk_f16_fp4 %3, %8, 1.0 op_sel:[1,1,0]\n"
                      "v_cvt_scalef32_pk_f16_fp4 %4, %8, 1.0\n v_cvt_scalef32_pk_f16_fp4 %5, %8, 1.0 op_sel:[1,0,0]\n"
                      "v_cvt_scalef32_pk_f16_fp4 %6, %8, 1.0 op_sel:[0,1,0]\n v_cvt_scalef32_pk_f16_fp4 %7, %8, 1.0 op_sel:[1,1,0]\n"
                      : "=&v"(a0), "=&v"(a1), "=&v"(a2), "=&v"(a3), "=&v"(a4), "=&v"(a5), "=&v"(a6), "=&v"(a7)
                      : "v"(w));)
  }
  out[blockIdx.x * blockDim.x + threadIdx.x] = a0 ^ a1 ^ a2 ^ a3 ^ a4 ^ a5 ^ a6 ^ a7;
}
__global__ void k_mul(int iters, uint32_t* out) {
  uint32_t w = threadIdx.x * 2654435761u, a0, a1, a2, a3, a4, a5, a6, a7;
  for (int it = 0; it < iters; ++it) {
    REP8(asm volatile("v_pk_mul_f16 %0, %8, %8\n v_pk_mul_f16 %1, %8, %8\n v_pk_mul_f16 %2, %8, %8\n v_pk_mul_f16 %3, %8, %8\n"
                      "v_pk_mul_f16 %4, %8, %8\n v_pk_mul_f16 %5, %8, %8\n v_pk_mul_f16 %6, %8, %8\n v_pk_mul_f16 %7, %8, %8\n"
                      : "=&v"(a0), "=&v"(a1), "=&v"(a2), "=&v"(a3), "=&v"(a4), "=&v"(a5), "=&v"(a6), "=&v"(a7)
                      : "v"(w));)
  }
  out[blockIdx.x * blockDim.x + threadIdx.x] = a0 ^ a1 ^ a2 ^ a3 ^ a4 ^ a5 ^ a6 ^ a7;
}
__global__ void k_cvt8(int iters, uint32_t* out) {
  uint32_t w = threadIdx.x * 2654435761u, a0, a1, a2, a3, a4, a5, a6, a7;
  for (int it = 0; it < iters; ++it) {
    REP8(asm volatile("v_cvt_scalef32_pk_f16_fp8 %0, %8, 1.0\n v_cvt_scalef32_pk_f16_fp8 %1, %8, 1.0 op_sel:[1,0,0]\n"
                      "v_cvt_scalef32_pk_f16_fp8 %2, %8, 1.0\n v_cvt_scalef32_pk_f16_fp8 %3, %8, 1.0 op_sel:[1,0,0]\n"
                      "v_cvt_scalef32_pk_f16_fp8 %4, %8, 1.0\n v_cvt_scalef32_pk_f16_fp8 %5, %8, 1.0 op_sel:[1,0,0]\n"
                      "v_cvt_scalef32_pk_f16_fp8 %6, %8, 1.0\n v_cvt_scalef32_pk_f16_fp8 %7, %8, 1.0 op_sel:[1,0,0]\n"
                      : "=&v"(a0), "=&v"(a1), "=&v"(a2), "=&v"(a3), "=&v"(a4), "=&v"(a5), "=&v"(a6), "=&v"(a7)
                      : "v"(w));)
  }
  out[blockIdx.x * blockDim.x + threadIdx.x] = a0 ^ a1 ^ a2 ^ a3 ^ a4 ^ a5 ^ a6 ^ a7;
}
// KIND 0: conversions, 1: packed multiplies, 2: alternating
template <int NV, int KIND>
__global__ __launch_bounds__(512) void k_mix(int iters, uint32_t* out) {
  float16v acc[8];
  for (int a = 0; a < 8; ++a)
    for (int i = 0; i < 16; ++i) acc[a][i] = 0.f;
  half8v opa, opb;
  for (int j = 0; j < 8; ++j) {
    opa[j] = (_Float16)1.0f;
    opb[j] = (_Float16)0.5f;
  }
  uint32_t w = threadIdx.x * 2654435761u, dd[8] = {0, 1, 2, 3, 4, 5, 6, 7};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int a = 0; a < 8; ++a) {
      asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(acc[a]) : "v"(opa), "v"(opb));
#pragma unroll
      for (int v = 0; v < NV; ++v) {
        const int kind = KIND == 2 ? (v & 1) : KIND;
        uint32_t& d = dd[(a * NV + v) & 7];
        if (kind == 0) {
          if (v & 2) asm volatile("v_cvt_scalef32_pk_f16_fp4 %0, %1, 1.0 op_sel:[1,0,0]" : "+v"(d) : "v"(w));
          else asm volatile("v_cvt_scalef32_pk_f16_fp4 %0, %1, 1.0" : "+v"(d) : "v"(w));
        } else {
          asm volatile("v_pk_mul_f16 %0, %1, %1" : "+v"(d) : "v"(w));
        }
      }
    }
  }
  float r = 0;
  for (int a = 0; a < 8; ++a)
    for (int i = 0; i < 16; ++i) r += acc[a][i];
  out[blockIdx.x * blockDim.x + threadIdx.x] = __float_as_uint(r) ^ dd[0] ^ dd[1] ^ dd[2] ^ dd[3] ^ dd[4] ^ dd[5] ^ dd[6] ^ dd[7];
}
template <class F>
float time_ms(F f, int reps = 5) {
  hipEvent_t s, e;
  (void)hipEventCreate(&s);
  (void)hipEventCreate(&e);
  f();
  (void)hipDeviceSynchronize();
  float best = 1e9;
  for (int r = 0; r < reps; ++r) {
    (void)hipEventRecord(s);
    f();
    (void)hipEventRecord(e);
    (void)hipEventSynchronize(e);
    float ms;
    (void)hipEventElapsedTime(&ms, s, e);
    if (ms < best) best = ms;
  }
  return best;
}
int main() {
  uint32_t* out;
  if (hipMalloc(&out, 256 * 512 * 4) != hipSuccess) return 1;
  const double ghz = 2.4;
  for (int i = 0; i < 300; ++i) hipLaunchKernelGGL(k_mul, dim3(256), dim3(256), 0, 0, 2000, out);
  (void)hipDeviceSynchronize();
  for (int per_simd = 1; per_simd <= 2; ++per_simd) {
    const int threads = 256 * per_simd, iters = 4000;
    const float t1 = time_ms([&] { hipLaunchKernelGGL(k_mul, dim3(256), dim3(threads), 0, 0, iters, out); });
    const float t2 = time_ms([&] { hipLaunchKernelGGL(k_cvt4, dim3(256), dim3(threads), 0, 0, iters, out); });
    const float t3 = time_ms([&] { hipLaunchKernelGGL(k_cvt8, dim3(256), dim3(threads), 0, 0, iters, out); });
    const double n = (double)iters * 64 * per_simd;
    printf("%d wave(s) per SIMD: v_pk_mul_f16 %.2f, v_cvt_scalef32_pk_f16_fp4 %.2f, v_cvt_scalef32_pk_f16_fp8 %.2f cycles per instruction (at %.1f GHz)\n",
           per_simd, t1 * 1e-3 * ghz * 1e9 / n, t2 * 1e-3 * ghz * 1e9 / n, t3 * 1e-3 * ghz * 1e9 / n, ghz);
  }
#define MIX(NV, KIND, T)                                                                                                       \
  {                                                                                                                           \
    const int iters = 3000;                                                                                                   \
    const float t = time_ms([&] { hipLaunchKernelGGL((k_mix<NV, KIND>), dim3(256), dim3(T), 0, 0, iters, out); });            \
    printf("MFMA + %d %s, %d wave(s) per SIMD: %.2f cycles per MFMA\n", NV, KIND == 0 ? "conversions" : KIND == 1 ? "packed multiplies" : "decode instructions (alternating)", \
           T / 256, t * 1e-3 * ghz * 1e9 / ((double)iters * 8 * (T / 256)));                                                 \
  }
  MIX(0, 2, 256) MIX(2, 2, 256) MIX(4, 2, 256) MIX(6, 2, 256) MIX(8, 2, 256)
  MIX(0, 2, 512) MIX(2, 2, 512) MIX(4, 2, 512) MIX(6, 2, 512) MIX(8, 2, 512)
  MIX(4, 0, 512) MIX(8, 0, 512) MIX(4, 1, 512) MIX(8, 1, 512)
  return 0;
}
