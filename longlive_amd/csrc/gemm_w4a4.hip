// W4A4 GEMM for gfx950:  D[m, n] = bf16(alpha * sum_k deq(A)[m, k] * deq(B)[n, k]) (+ bias[n])
//
// Operands stay packed (e2m1 nibbles + e4m3 block-16 scales) from HBM through LDS into registers.
// CDNA4's scaled FP4 MFMA only takes power-of-two scales over 32 elements, which cannot express an
// e4m3 scale over 16, so each wave decodes its fragments in registers instead:
//     e2m1 pair --v_cvt_scalef32_pk_f16_fp4--> f16 pair --v_pk_mul_f16 by the f16 block scale--> operand
// The product code x scale has at most 6 significant bits and lies in [2^-10, 2688], so it is exact
// in f16; v_mfma_f32_32x32x16_f16 then accumulates exact products in fp32, which is the arithmetic of
// the reference's dequantize-then-fp32-matmul up to summation order.  The two tensor scales are applied
// once in the epilogue (alpha), as the reference's CUTLASS path does
// (fouroversix/src/fouroversix/matmul/cutlass/backend.py:81-90, csrc/fp4_gemm.cu:143).
//
// Tiling: 256 threads = 4 waves in a 2x2 grid, each wave owns FA x FB MFMA tiles of 32x32
// (workgroup tile = 64*FA rows of A by 64*FB rows of B), K step 128 (64 packed bytes per row),
// two LDS stages filled through registers.  K is consumed in a permuted order (lanes 0-31 and
// 32-63 take alternate 32-element runs), identical for A and B, so the sum is unchanged.
#include "ll_common.h"

namespace ll {

typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef _Float16 half8v __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));

constexpr int kBK = 128;          // K elements per main-loop step
constexpr int kRowBytes = 64;     // packed bytes per row per step
constexpr int kLdsRow = 80;       // padded LDS row pitch (bank-conflict free for 16-byte reads)
constexpr int kGemmThreads = 256;

// Decode 8 e2m1 codes (one dword) and scale them by the f16 pair (s, s).
__device__ __forceinline__ half8v decode8(uint32_t w, half2v s2) {
  const half2v p0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 0) * s2;
  const half2v p1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 1) * s2;
  const half2v p2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 2) * s2;
  const half2v p3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 3) * s2;
  half8v r;
  r[0] = p0[0]; r[1] = p0[1]; r[2] = p1[0]; r[3] = p1[1];
  r[4] = p2[0]; r[5] = p2[1]; r[6] = p3[0]; r[7] = p3[1];
  return r;
}

template <int FA, int FB>
struct GemmSmem {
  static constexpr int BM = 64 * FA;  // rows of A per workgroup
  static constexpr int BN = 64 * FB;  // rows of B per workgroup
  static constexpr int kAVals = BM * kLdsRow;
  static constexpr int kBVals = BN * kLdsRow;
  static constexpr int kAScales = (BM + 127) / 128 * 1024;
  static constexpr int kBScales = (BN + 127) / 128 * 1024;
  static constexpr int kStage = kAVals + kBVals + kAScales + kBScales;
};

template <int FA, int FB>
__global__ __launch_bounds__(kGemmThreads) void gemm_w4a4_kernel(
    const uint8_t* __restrict__ Av, const uint8_t* __restrict__ As, const uint8_t* __restrict__ Bv,
    const uint8_t* __restrict__ Bs, const float* __restrict__ alpha_ptr, const float* __restrict__ amax_a,
    const float* __restrict__ amax_b, float inv_denom_a, float inv_denom_b, int M, int N, int Mp, int Np, int Kp,
    uint16_t* __restrict__ D, int64_t ldd, const uint16_t* __restrict__ bias, int tiles_m, int tiles_n) {
  using S = GemmSmem<FA, FB>;
  constexpr int BM = S::BM, BN = S::BN;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

  // Workgroup -> tile.  Consecutive workgroup ids are dealt round-robin to the 8 XCDs, so ids that
  // share an XCD (and its L2) are mapped to neighbouring tiles: same B panel, consecutive A panels.
  int wg = blockIdx.x;
  {
    const int total = tiles_m * tiles_n;
    const int per_xcd = (total + 7) / 8;
    const int xcd = wg & 7, idx = wg >> 3;
    const int remapped = xcd * per_xcd + idx;
    if (total % 8 == 0) wg = remapped;  // exact split only; otherwise keep the plain order
  }
  const int tile_n = wg / tiles_m, tile_m = wg - tile_n * tiles_m;
  const int row0 = tile_m * BM;  // first row of A (output row)
  const int col0 = tile_n * BN;  // first row of B (output column)

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;
  const int l32 = lane & 31, lh = lane >> 5;

  // ---- global -> register staging plan
  constexpr int kAChunks = BM * 4 / kGemmThreads;  // 16-byte chunks of A values per thread
  constexpr int kBChunks = BN * 4 / kGemmThreads;
  const int64_t row_bytes = Kp >> 1;
  const uint8_t* a_src[kAChunks];
  const uint8_t* b_src[kBChunks];
  int a_dst[kAChunks], b_dst[kBChunks];
#pragma unroll
  for (int i = 0; i < kAChunks; ++i) {
    const int q = tid + i * kGemmThreads, r = q >> 2, ck = q & 3;
    const int gr = min(row0 + r, Mp - 1);
    a_src[i] = Av + (int64_t)gr * row_bytes + ck * 16;
    a_dst[i] = r * kLdsRow + ck * 16;
  }
#pragma unroll
  for (int i = 0; i < kBChunks; ++i) {
    const int q = tid + i * kGemmThreads, r = q >> 2, ck = q & 3;
    const int gr = min(col0 + r, Np - 1);
    b_src[i] = Bv + (int64_t)gr * row_bytes + ck * 16;
    b_dst[i] = S::kAVals + r * kLdsRow + ck * 16;
  }
  // scales: 1024 contiguous bytes per 128-row block per step (two 128x4 tiles) = 64 threads x 16 bytes
  constexpr int kARb = (BM + 127) / 128, kBRb = (BN + 127) / 128;
  const int sgrp = tid >> 6;  // which 1024-byte run this thread copies
  const bool s_active = sgrp < kARb + kBRb;
  const bool s_is_a = sgrp < kARb;
  const uint8_t* s_src = nullptr;
  int s_dst = 0;
  if (s_active) {
    const int rbi = s_is_a ? sgrp : sgrp - kARb;
    const int rb = s_is_a ? min(row0 / 128 + rbi, Mp / 128 - 1) : min(col0 / 128 + rbi, Np / 128 - 1);
    s_src = (s_is_a ? As : Bs) + (int64_t)rb * (Kp >> 6) * 512 + (tid & 63) * 16;
    s_dst = S::kAVals + S::kBVals + (s_is_a ? 0 : S::kAScales) + rbi * 1024 + (tid & 63) * 16;
  }

  uint4 a_reg[kAChunks], b_reg[kBChunks], s_reg;
  const int nk = (Kp + kBK - 1) / kBK;
  auto load_step = [&](int t) {
    const bool second_half_valid = (t * kBK + 64) < Kp;  // Kp is a multiple of 64, maybe not of 128
#pragma unroll
    for (int i = 0; i < kAChunks; ++i) {
      const int ck = (tid + i * kGemmThreads) & 3;
      a_reg[i] = (ck < 2 || second_half_valid) ? *reinterpret_cast<const uint4*>(a_src[i] + (int64_t)t * kRowBytes)
                                               : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < kBChunks; ++i) {
      const int ck = (tid + i * kGemmThreads) & 3;
      b_reg[i] = (ck < 2 || second_half_valid) ? *reinterpret_cast<const uint4*>(b_src[i] + (int64_t)t * kRowBytes)
                                               : make_uint4(0, 0, 0, 0);
    }
    if (s_active) {
      const bool valid = ((tid & 63) < 32) || second_half_valid;
      s_reg = valid ? *reinterpret_cast<const uint4*>(s_src + (int64_t)t * 1024) : make_uint4(0, 0, 0, 0);
    }
  };
  auto store_step = [&](int stage) {
    uint8_t* base = smem + stage * S::kStage;
#pragma unroll
    for (int i = 0; i < kAChunks; ++i) *reinterpret_cast<uint4*>(base + a_dst[i]) = a_reg[i];
#pragma unroll
    for (int i = 0; i < kBChunks; ++i) *reinterpret_cast<uint4*>(base + b_dst[i]) = b_reg[i];
    if (s_active) *reinterpret_cast<uint4*>(base + s_dst) = s_reg;
  };

  // ---- per-lane LDS read offsets
  // fragment f of A: rows wm*32*FA + 32 f + l32 ; chunk (cc, lh) = bytes [32 cc + 16 lh, +16)
  int a_voff[FA], a_soff[FA], b_voff[FB], b_soff[FB];
#pragma unroll
  for (int f = 0; f < FA; ++f) {
    const int r = wm * 32 * FA + 32 * f + l32;
    a_voff[f] = r * kLdsRow + 16 * lh;
    a_soff[f] = S::kAVals + S::kBVals + (r >> 7) * 1024 + (r & 31) * 16 + ((r & 127) >> 5) * 4 + 2 * lh;
  }
#pragma unroll
  for (int f = 0; f < FB; ++f) {
    const int r = wn * 32 * FB + 32 * f + l32;
    b_voff[f] = S::kAVals + r * kLdsRow + 16 * lh;
    b_soff[f] = S::kAVals + S::kBVals + S::kAScales + (r >> 7) * 1024 + (r & 31) * 16 + ((r & 127) >> 5) * 4 + 2 * lh;
  }

  float16v acc[FB][FA];
#pragma unroll
  for (int g = 0; g < FB; ++g)
#pragma unroll
    for (int f = 0; f < FA; ++f)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[g][f][i] = 0.0f;

  load_step(0);
  store_step(0);
  __syncthreads();

  for (int t = 0; t < nk; ++t) {
    if (t + 1 < nk) load_step(t + 1);
    const uint8_t* base = smem + (t & 1) * S::kStage;
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) {
      uint4 araw[FA], braw[FB];
      half2v asc[FA][2], bsc[FB][2];
#pragma unroll
      for (int f = 0; f < FA; ++f) {
        araw[f] = *reinterpret_cast<const uint4*>(base + a_voff[f] + 32 * cc);
        const uint32_t sb = *reinterpret_cast<const uint16_t*>(base + a_soff[f] + 512 * cc);
        const half2v s = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(sb, 1.0f, false);
        asc[f][0] = half2v{s[0], s[0]};
        asc[f][1] = half2v{s[1], s[1]};
      }
#pragma unroll
      for (int g = 0; g < FB; ++g) {
        braw[g] = *reinterpret_cast<const uint4*>(base + b_voff[g] + 32 * cc);
        const uint32_t sb = *reinterpret_cast<const uint16_t*>(base + b_soff[g] + 512 * cc);
        const half2v s = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(sb, 1.0f, false);
        bsc[g][0] = half2v{s[0], s[0]};
        bsc[g][1] = half2v{s[1], s[1]};
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        half8v a16[FA], b16[FB];
#pragma unroll
        for (int f = 0; f < FA; ++f) {
          const uint32_t w = j == 0 ? araw[f].x : j == 1 ? araw[f].y : j == 2 ? araw[f].z : araw[f].w;
          a16[f] = decode8(w, asc[f][j >> 1]);
        }
#pragma unroll
        for (int g = 0; g < FB; ++g) {
          const uint32_t w = j == 0 ? braw[g].x : j == 1 ? braw[g].y : j == 2 ? braw[g].z : braw[g].w;
          b16[g] = decode8(w, bsc[g][j >> 1]);
        }
#pragma unroll
        for (int g = 0; g < FB; ++g)
#pragma unroll
          for (int f = 0; f < FA; ++f)
            acc[g][f] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b16[g], a16[f], acc[g][f], 0, 0, 0);
      }
    }
    if (t + 1 < nk) store_step((t + 1) & 1);
    __syncthreads();
  }

  // ---- epilogue.  acc[g][f][r]: output column n = col0 + wn*32*FB + 32 g + 8 (r/4) + 4 lh + r%4,
  //                               output row    m = row0 + wm*32*FA + 32 f + l32.
  float alpha;
  if (alpha_ptr) {
    alpha = alpha_ptr[0];
  } else {
    alpha = (amax_a[0] * amax_b[0]) * (inv_denom_a * inv_denom_b);
  }
#pragma unroll
  for (int f = 0; f < FA; ++f) {
    const int m = row0 + wm * 32 * FA + 32 * f + l32;
    if (m >= M) continue;
    uint16_t* drow = D + (int64_t)m * ldd;
#pragma unroll
    for (int g = 0; g < FB; ++g) {
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        const int n = col0 + wn * 32 * FB + 32 * g + 8 * rg + 4 * lh;
        if (n >= N) continue;
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = acc[g][f][4 * rg + i] * alpha;
        if (n + 4 <= N && ((ldd & 3) == 0)) {
          uint32_t o[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) o[i] = f32_to_bf16_bits(v[i]);
          if (bias) {
            const uint2 bb = *reinterpret_cast<const uint2*>(bias + n);
            const uint32_t bw[4] = {bb.x & 0xFFFFu, bb.x >> 16, bb.y & 0xFFFFu, bb.y >> 16};
#pragma unroll
            for (int i = 0; i < 4; ++i) o[i] = f32_to_bf16_bits(__uint_as_float(o[i] << 16) + __uint_as_float(bw[i] << 16));
          }
          *reinterpret_cast<uint2*>(drow + n) = make_uint2(o[0] | (o[1] << 16), o[2] | (o[3] << 16));
        } else {
          for (int i = 0; i < 4 && n + i < N; ++i) {
            uint32_t o = f32_to_bf16_bits(v[i]);
            if (bias) o = f32_to_bf16_bits(__uint_as_float(o << 16) + bf16_bits_to_f32(bias[n + i]));
            drow[n + i] = (uint16_t)o;
          }
        }
      }
    }
  }
}

template <int FA, int FB>
int launch_gemm(const uint8_t* Av, const uint8_t* As, const uint8_t* Bv, const uint8_t* Bs, const float* alpha,
                const float* amax_a, const float* amax_b, float denom_a, float denom_b, int M, int N, int Mp, int Np,
                int Kp, void* D, int64_t ldd, const void* bias, hipStream_t stream) {
  using S = GemmSmem<FA, FB>;
  const int tiles_m = (M + S::BM - 1) / S::BM, tiles_n = (N + S::BN - 1) / S::BN;
  const size_t smem = 2 * S::kStage;
  static bool configured = false;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_w4a4_kernel<FA, FB>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) {
      set_error("ll_nvfp4_gemm_tnt: cannot reserve %zu bytes of LDS: %s", smem, hipGetErrorString(e));
      return LL_ELAUNCH;
    }
    configured = true;
  }
  hipLaunchKernelGGL((gemm_w4a4_kernel<FA, FB>), dim3((unsigned)(tiles_m * tiles_n)), dim3(kGemmThreads), smem, stream,
                     Av, As, Bv, Bs, alpha, amax_a, amax_b, 1.0f / denom_a, 1.0f / denom_b, M, N, Mp, Np, Kp,
                     static_cast<uint16_t*>(D), ldd, static_cast<const uint16_t*>(bias), tiles_m, tiles_n);
  LL_CHECK_LAUNCH("gemm_w4a4_kernel");
  return LL_OK;
}

}  // namespace ll

extern "C" int ll_nvfp4_gemm_tnt(const uint8_t* A_values, const uint8_t* A_scales, const uint8_t* B_values,
                                 const uint8_t* B_scales, const float* alpha, const float* amax_a,
                                 const float* amax_b, float denom_a, float denom_b, int64_t M, int64_t N, int64_t Mp,
                                 int64_t Np, int64_t Kp, void* D, int64_t ldd, const void* bias, void* stream) {
  using namespace ll;
  LL_REQUIRE(A_values && A_scales && B_values && B_scales && D, "ll_nvfp4_gemm_tnt: null pointer");
  LL_REQUIRE(alpha || (amax_a && amax_b && denom_a > 0.f && denom_b > 0.f),
             "ll_nvfp4_gemm_tnt: pass alpha, or both amax pointers with positive denominators");
  LL_REQUIRE(M > 0 && N > 0 && Mp % 128 == 0 && Np % 128 == 0 && Kp % 64 == 0 && Kp > 0 && M <= Mp && N <= Np &&
                 ldd >= N,
             "ll_nvfp4_gemm_tnt: bad shape M=%lld N=%lld Mp=%lld Np=%lld Kp=%lld ldd=%lld", (long long)M,
             (long long)N, (long long)Mp, (long long)Np, (long long)Kp, (long long)ldd);
  LL_REQUIRE(Mp < (1 << 30) && Np < (1 << 30) && Kp < (1 << 30), "ll_nvfp4_gemm_tnt: dimension too large");
  LL_REQUIRE(((reinterpret_cast<uintptr_t>(A_values) | reinterpret_cast<uintptr_t>(B_values) |
               reinterpret_cast<uintptr_t>(A_scales) | reinterpret_cast<uintptr_t>(B_scales)) & 15) == 0,
             "ll_nvfp4_gemm_tnt: operands must be 16-byte aligned");
  LL_REQUIRE((reinterpret_cast<uintptr_t>(D) & 7) == 0 && (!bias || (reinterpret_cast<uintptr_t>(bias) & 7) == 0),
             "ll_nvfp4_gemm_tnt: D and bias must be 8-byte aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  // Tile choice: the largest tile that still gives every CU (256) work in about whole rounds.
  auto rounds_eff = [&](int bm, int bn) {
    const double tiles = (double)((M + bm - 1) / bm) * (double)((N + bn - 1) / bn);
    const double rounds = (tiles + 255.0) / 256.0;
    return tiles / (256.0 * (double)(int64_t)rounds);
  };
  struct Cfg { int fa, fb; double bonus; };
  const Cfg cfgs[4] = {{4, 4, 1.00}, {2, 4, 0.93}, {4, 2, 0.93}, {2, 2, 0.80}};
  int best = 0;
  double best_score = -1.0;
  for (int i = 0; i < 4; ++i) {
    const double sc = rounds_eff(64 * cfgs[i].fa, 64 * cfgs[i].fb) * cfgs[i].bonus;
    if (sc > best_score) {
      best_score = sc;
      best = i;
    }
  }
#define LL_GEMM_ARGS A_values, A_scales, B_values, B_scales, alpha, amax_a, amax_b, denom_a, denom_b, (int)M, (int)N, \
                     (int)Mp, (int)Np, (int)Kp, D, ldd, bias, s
  switch (best) {
    case 0: return launch_gemm<4, 4>(LL_GEMM_ARGS);
    case 1: return launch_gemm<2, 4>(LL_GEMM_ARGS);
    case 2: return launch_gemm<4, 2>(LL_GEMM_ARGS);
    default: return launch_gemm<2, 2>(LL_GEMM_ARGS);
  }
#undef LL_GEMM_ARGS
}
