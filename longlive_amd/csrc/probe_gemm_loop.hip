// Probe (not part of the library): the generated main loop of the persistent W4A4 GEMM (gemm_loop_gfx950.inc) on its
// own - one workgroup per 128 x 512 tile, the whole K range, raw fp32 accumulators out.  It answers three questions
// the kernel design rests on:
//   1. is the instruction sequence right?  every output of a small problem against the exact sum of products
//      computed on the host (random codes and scale bytes);
//   2. how fast is it?  time per launch on a full chip (one tile per compute unit, K = 14336) and on the two FFN shapes;
//   3. what does the chip's clock do under it?  s_memtime counts shader clocks, s_memrealtime a constant 100 MHz,
//      so their ratio over one workgroup's life is the clock the loop ran at; with all-zero operands (same
//      instructions, no switching in the multipliers) the same loop shows what the clock would allow.
// Build: make -C longlive_amd/csrc probes      Run: ./longlive_amd/csrc/probe_gemm_loop
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include <vector>
typedef float float16v __attribute__((ext_vector_type(16)));
#define CHECK(x)                                                                           \
  do {                                                                                     \
    hipError_t e__ = (x);                                                                  \
    if (e__ != hipSuccess) {                                                               \
      printf("HIP error %s at line %d\n", hipGetErrorString(e__), __LINE__);               \
      exit(1);                                                                             \
    }                                                                                      \
  } while (0)
#define V10(a) "v" #a "0", "v" #a "1", "v" #a "2", "v" #a "3", "v" #a "4", "v" #a "5", "v" #a "6", "v" #a "7", "v" #a "8", "v" #a "9"

__global__ __launch_bounds__(256) void loop_kernel(const uint8_t* Av, const uint8_t* As, const uint8_t* Bv, const uint8_t* Bs,
                                                   int Kp, int tiles_m, float* out, int ldo, int write, unsigned long long* clk) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const unsigned long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
  const int tile_m = blockIdx.x % tiles_m, tile_n = blockIdx.x / tiles_m;
  const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int row0 = tile_m * 128, col0 = tile_n * 512;
  const uint32_t row_bytes = (uint32_t)Kp >> 1;
  const uint32_t nk = Kp / 128;
  float16v acc[16];
#pragma unroll
  for (int i = 0; i < 16; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[i][j] = 0.0f;
  const uint32_t swz = (l32 >> 2) & 3;
  const uint32_t voff = (uint32_t)(lane >> 2) * row_bytes + 16u * ((lane & 3) ^ ((lane >> 4) & 3));
  const uint32_t soff = lane * 16u;
  const uint32_t ard = l32 * 64u + 16u * ((lh ^ (swz & 1)) | (swz & 2));
  const uint32_t sard = 40960u + l32 * 16u;
  const uint32_t sh = 16u * lh;
  const uint8_t* sA = Av + (size_t)(row0 + 32 * wave) * row_bytes;
  const uint8_t* sB = Bv + (size_t)(col0 + 128 * wave) * row_bytes;
  const uint32_t rb16 = 16u * row_bytes;
  const uint8_t* sAs = As + (size_t)(row0 / 128) * (Kp / 64) * 512;
  const uint8_t* sBs = Bs + (size_t)(col0 / 128 + wave) * (Kp / 64) * 512;
  __syncthreads();
  asm volatile(
#include "gemm_loop_gfx950.inc"
      : "+a"(acc[0]), "+a"(acc[1]), "+a"(acc[2]), "+a"(acc[3]), "+a"(acc[4]), "+a"(acc[5]), "+a"(acc[6]), "+a"(acc[7]), "+a"(acc[8]),
        "+a"(acc[9]), "+a"(acc[10]), "+a"(acc[11]), "+a"(acc[12]), "+a"(acc[13]), "+a"(acc[14]), "+a"(acc[15])
      : "s"(nk), "v"(voff), "v"(soff), "v"(ard), "v"(sard), "v"(sh), "s"(sA), "s"(sB), "s"(rb16), "s"(sAs), "s"(sBs), "s"(wave)
      : "memory", "scc", "vcc", "v0", "v1", "v2", "v3", "v4", "v5", "v6", "v7", "v8", "v9", V10(1), V10(2), V10(3), V10(4), V10(5),
        V10(6), V10(7), V10(8), V10(9), V10(10), V10(11), V10(12), V10(13), V10(14), V10(15), V10(16), "s56", "s57", "s58", "s59",
        "s60", "s61", "s62", "s63", "s64", "s65", "s66", "s67", "s68", "s69", "s70", "s71", "s72", "s73", "s74", "s75", "s76", "s77",
        "s78", "s79", "s80", "s81", "s82", "s83", "s84", "s85", "s86", "s87");
  if (write) {  // acc[4 g + f][r]: row 32 f + lane % 32, column 128 wave + 32 g + 8 (r / 4) + 4 (lane / 32) + r % 4
#pragma unroll
    for (int g = 0; g < 4; ++g)
#pragma unroll
      for (int f = 0; f < 4; ++f)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          out[(size_t)(row0 + 32 * f + l32) * ldo + col0 + 128 * wave + 32 * g + 8 * (r / 4) + 4 * lh + r % 4] = acc[4 * g + f][r];
  } else if (acc[0][0] == 12345.678f) {
    out[0] = acc[3][1];
  }
  if (clk && threadIdx.x == 0) {
    clk[2 * blockIdx.x] = __builtin_readcyclecounter() - c0;
    clk[2 * blockIdx.x + 1] = __builtin_amdgcn_s_memrealtime() - r0;
  }
}

static float e2m1(int c) {
  static const float t[8] = {0, .5f, 1, 1.5f, 2, 3, 4, 6};
  return (c & 8) ? -t[c & 7] : t[c & 7];
}
static float e4m3(int b) {
  const int e = (b >> 3) & 15, m = b & 7;
  return e == 0 ? m * ldexpf(1.f, -9) : ldexpf(1.f + m / 8.f, e - 7);
}
static size_t blocked(size_t r, size_t c, size_t cols) {
  const size_t rb = r >> 7, ri = r & 127, cb = c >> 2, ci = c & 3;
  return ((rb * (cols >> 2) + cb) * 32 + (ri & 31)) * 16 + (ri >> 5) * 4 + ci;
}

int main() {
  const int kSmem = 92160;
  CHECK(hipFuncSetAttribute((const void*)loop_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kSmem));
  int failures = 0;
  for (int Kp : {128, 256, 384, 1024}) {  // 1, 2, 3 and 8 K steps
    const int M = 256, N = 1024;
    std::vector<uint8_t> av((size_t)M * Kp / 2), as((size_t)M * Kp / 16), bv((size_t)N * Kp / 2), bs((size_t)N * Kp / 16);
    srand(Kp);
    for (auto& x : av) x = rand() & 0xFF;
    for (auto& x : bv) x = rand() & 0xFF;
    for (auto& x : as) x = 0x28 + (rand() % 0x30);  // scales 2^-2 .. 2^3
    for (auto& x : bs) x = 0x28 + (rand() % 0x30);
    uint8_t *dav, *das, *dbv, *dbs;
    float* dout;
    CHECK(hipMalloc(&dav, av.size()));
    CHECK(hipMalloc(&das, as.size()));
    CHECK(hipMalloc(&dbv, bv.size()));
    CHECK(hipMalloc(&dbs, bs.size()));
    CHECK(hipMalloc(&dout, (size_t)M * N * 4));
    CHECK(hipMemcpy(dav, av.data(), av.size(), hipMemcpyHostToDevice));
    CHECK(hipMemcpy(das, as.data(), as.size(), hipMemcpyHostToDevice));
    CHECK(hipMemcpy(dbv, bv.data(), bv.size(), hipMemcpyHostToDevice));
    CHECK(hipMemcpy(dbs, bs.data(), bs.size(), hipMemcpyHostToDevice));
    hipLaunchKernelGGL(loop_kernel, dim3((M / 128) * (N / 512)), dim3(256), kSmem, 0, dav, das, dbv, dbs, Kp, M / 128, dout, N, 1, nullptr);
    CHECK(hipDeviceSynchronize());
    std::vector<float> got((size_t)M * N);
    CHECK(hipMemcpy(got.data(), dout, got.size() * 4, hipMemcpyDeviceToHost));
    std::vector<float> da((size_t)M * Kp), db((size_t)N * Kp);
    for (int m = 0; m < M; ++m)
      for (int k = 0; k < Kp; ++k) {
        const int byte = av[(size_t)m * Kp / 2 + k / 2];
        da[(size_t)m * Kp + k] = e2m1(k & 1 ? byte >> 4 : byte & 15) * e4m3(as[blocked(m, k / 16, Kp / 16)]);
      }
    for (int n = 0; n < N; ++n)
      for (int k = 0; k < Kp; ++k) {
        const int byte = bv[(size_t)n * Kp / 2 + k / 2];
        db[(size_t)n * Kp + k] = e2m1(k & 1 ? byte >> 4 : byte & 15) * e4m3(bs[blocked(n, k / 16, Kp / 16)]);
      }
    double worst = 0;
    for (int m = 0; m < M; ++m)
      for (int n = 0; n < N; ++n) {
        double ref = 0, mag = 0;
        for (int k = 0; k < Kp; ++k) {
          const double p = (double)da[(size_t)m * Kp + k] * db[(size_t)n * Kp + k];
          ref += p;
          mag += fabs(p);
        }
        const double err = fabs(got[(size_t)m * N + n] - ref) / (mag + 1e-30);
        if (err > worst) worst = err;
      }
    printf("exactness Kp=%d: worst |got - exact| / sum |products| = %.3g %s\n", Kp, worst, worst <= 1e-6 ? "ok" : "FAILED");
    failures += worst > 1e-6;
    CHECK(hipFree(dav)); CHECK(hipFree(das)); CHECK(hipFree(dbv)); CHECK(hipFree(dbs)); CHECK(hipFree(dout));
  }
  const int shapes[3][3] = {{4096, 4096, 14336}, {2688, 14336, 3072}, {2688, 3072, 14336}};
  for (int zero = 0; zero < 2; ++zero)
    for (const auto& sh : shapes) {
      const int M = sh[0], N = sh[1], Kp = sh[2];
      uint8_t *dav, *das, *dbv, *dbs;
      float* dout;
      unsigned long long* dclk;
      CHECK(hipMalloc(&dav, (size_t)M * Kp / 2));
      CHECK(hipMalloc(&das, (size_t)M * Kp / 16));
      CHECK(hipMalloc(&dbv, (size_t)N * Kp / 2));
      CHECK(hipMalloc(&dbs, (size_t)N * Kp / 16));
      CHECK(hipMalloc(&dout, 1 << 20));
      CHECK(hipMalloc(&dclk, 16 * 1024));
      std::vector<uint8_t> h((size_t)(N > M ? N : M) * Kp / 2);
      for (auto& x : h) x = zero ? 0 : (rand() & 0xFF);
      CHECK(hipMemcpy(dbv, h.data(), (size_t)N * Kp / 2, hipMemcpyHostToDevice));
      CHECK(hipMemcpy(dav, h.data(), (size_t)M * Kp / 2, hipMemcpyHostToDevice));
      for (auto& x : h) x = 0x28 + (rand() % 0x30);
      CHECK(hipMemcpy(dbs, h.data(), (size_t)N * Kp / 16, hipMemcpyHostToDevice));
      CHECK(hipMemcpy(das, h.data(), (size_t)M * Kp / 16, hipMemcpyHostToDevice));
      const int tiles = (M / 128) * (N / 512);
      hipEvent_t s, e;
      CHECK(hipEventCreate(&s));
      CHECK(hipEventCreate(&e));
      for (int i = 0; i < 30; ++i) hipLaunchKernelGGL(loop_kernel, dim3(tiles), dim3(256), kSmem, 0, dav, das, dbv, dbs, Kp, M / 128, dout, N, 0, nullptr);
      CHECK(hipEventRecord(s));
      const int reps = 50;
      for (int i = 0; i < reps; ++i) hipLaunchKernelGGL(loop_kernel, dim3(tiles), dim3(256), kSmem, 0, dav, das, dbv, dbs, Kp, M / 128, dout, N, 0, dclk);
      CHECK(hipEventRecord(e));
      CHECK(hipEventSynchronize(e));
      float ms;
      CHECK(hipEventElapsedTime(&ms, s, e));
      unsigned long long hc[2];
      CHECK(hipMemcpy(hc, dclk, 16, hipMemcpyDeviceToHost));  // workgroup 0 of the last launch
      const double us = ms * 1e3 / reps, fl = 2.0 * M * N * Kp;
      printf("%s operands M=%d N=%d K=%d: %d tiles (%.2f per CU of 256), %.1f us per launch, %.0f TFLOP/s = %.3f of 2.5 PFLOP/s; "
             "workgroup 0: %llu shader clocks in %.1f us = %.2f GHz, %.1f clocks per MFMA\n",
             zero ? "all-zero" : "random  ", M, N, Kp, tiles, tiles / 256.0, us, fl / us / 1e6, fl / us / 1e6 / 2500, hc[0], hc[1] / 100.0,
             hc[0] / (hc[1] * 10.0), (double)hc[0] / (128.0 * (Kp / 128)));
      CHECK(hipFree(dav)); CHECK(hipFree(das)); CHECK(hipFree(dbv)); CHECK(hipFree(dbs)); CHECK(hipFree(dout)); CHECK(hipFree(dclk));
    }
  return failures ? 1 : 0;
}
