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
// two LDS stages filled straight from global memory (global_load_lds_dwordx4: no staging registers, no LDS
// store instructions).  Such a load writes the 64 lanes' 16-byte pieces to consecutive LDS addresses, so rows are
// unpadded (64 bytes) and the four pieces of a row are stored in the order piece ^ (row / 4 % 4), which spreads
// the fragment reads of 16 consecutive rows over all banks.  The kernel keeps to 256 registers per wave so that
// two workgroups share a CU: while one wave decodes, another wave's MFMAs run.  K is consumed in a
// permuted order (lanes 0-31 and 32-63 take alternate 32-element runs), identical for A and B, so
// the sum is unchanged.
#include "ll_common.h"
#include "gemm_split.h"

namespace ll {

// sixteen zero bytes in global memory: what lanes load in place of K elements beyond the end of a row
__device__ uint4 g_gemm_zero16;

// 16 bytes per lane from global memory straight into LDS at lds_base + 16 * lane (lds_base wave-uniform).
// Written as an asm statement on purpose: for the builtin the compiler's wait-count pass, which cannot tell the
// two LDS stages apart, makes every later LDS read wait for the load, which would expose the whole memory latency
// in every K step.  The kernel waits for these loads itself (vmcnt(0) ahead of the barrier that hands the stage
// over) and issues no other vector-memory loads while they are in flight.
__device__ __forceinline__ void load_to_lds_b128(const void* src, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(lds_base) : "memory");
}
__device__ __forceinline__ uint32_t lds_address(const void* p) {
  return __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)p);
}

typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef _Float16 half8v __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));

constexpr int kBK = 128;          // K elements per main-loop step
constexpr int kRowBytes = 64;     // packed bytes per row per step
constexpr int kLdsRow = 64;       // LDS row pitch: unpadded, pieces swizzled (see above)
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

// 0.5 x (1 + tanh(u)) = x / (1 + exp(-2u)),  u = sqrt(2/pi) (x + 0.044715 x^3)  (nn.GELU(approximate="tanh"))
__device__ __forceinline__ float gelu_tanh_f32(float x) {
  const float u2 = x * (1.5957691216057308f + 0.07135481627260025f * (x * x));  // 2u
  return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * u2));
}

// What the epilogue does to y = bf16(alpha * acc), in this order (each step optional):
//   y = bf16(y + bias[n]);  y = bf16(act(y));  y = bf16(y * gate[m / gate_rows, n]) (only with residual);
//   y = bf16(residual[m, n] + y);  max |y| goes to the amax sink.
struct GemmEpilogue {
  const uint16_t* bias;
  int act;
  const uint16_t* gate;
  int gate_rows;
  int64_t gate_stride;
  const uint16_t* residual;
  int64_t ldr;
  AmaxSink sink;
};

// Several products with the same A operand and the same N and K in one launch (the q / k / v projections of one
// activation): the weight, its scales and tensor scale, the bias, the output and the amax sink of the products
// behind the first one.  The column tiles of all products form one row of tiles_n tiles, tiles_n_each per product.
constexpr int kMaxGemmGroups = 4;
struct GemmGroup {
  const uint8_t* Bv;
  const uint8_t* Bs;
  const float* alpha;
  const float* amax_b;
  float inv_denom_b;
  uint16_t* D;
  int64_t ldd;
  const uint16_t* bias;
  AmaxSink sink;
};
struct GemmGroups {
  int n;             // number of products (1: the plain call, `more` unused)
  int tiles_n_each;  // column tiles per product
  GemmGroup more[kMaxGemmGroups - 1];
};

// Epilogue of one wave: acc[g][f][r] holds output row m = row_base + 32 f + lane % 32 and output column
// n = col_base + 32 g + 8 (r / 4) + 4 (lane / 32) + r % 4.  The wave transposes one 32-row slab at a time through its
// own LDS patch (the stages of the main loop are free by now) and writes rows with coalesced 16-byte stores.
template <int FA, int FB>
__device__ __forceinline__ void gemm_epilogue(float16v (&acc)[FB][FA], float alpha, uint8_t* smem, int wave, int lane, int row_base,
                                              int col_base, int M, int N, uint16_t* __restrict__ D, int64_t ldd,
                                              const uint16_t* __restrict__ bias, int act, const GemmEpilogue& epi,
                                              uint32_t sink_slot) {
  const int l32 = lane & 31, lh = lane >> 5;
  constexpr int kEpiPitch = 64 * FB + 16;  // bytes per slab row: 32*FB bf16 + pad
  uint8_t* ebuf = smem + wave * (32 * kEpiPitch);
  constexpr int kChunksPerRow = 4 * FB;     // 16-byte chunks (8 columns) per slab row
  const int ch = lane % kChunksPerRow;      // this lane's chunk column, the same in every pass
  const int n_lane = col_base + 8 * ch;
  const bool vec_ok = ((ldd & 7) == 0) && ((reinterpret_cast<uintptr_t>(D) & 15) == 0);
  float out_max = 0.0f;
  float bias_f[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) bias_f[i] = (bias && n_lane + i < N) ? bf16_bits_to_f32(bias[n_lane + i]) : 0.0f;
#pragma unroll
  for (int f = 0; f < FA; ++f) {
#pragma unroll
    for (int g = 0; g < FB; ++g)
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        *reinterpret_cast<uint2*>(ebuf + l32 * kEpiPitch + (32 * g + 8 * rg + 4 * lh) * 2) =
            make_uint2(pack_bf16x2(acc[g][f][4 * rg] * alpha, acc[g][f][4 * rg + 1] * alpha),
                       pack_bf16x2(acc[g][f][4 * rg + 2] * alpha, acc[g][f][4 * rg + 3] * alpha));
      }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int it = 0; it < (32 * kChunksPerRow) / 64; ++it) {
      const int row = (it * 64 + lane) / kChunksPerRow;
      const int m = row_base + 32 * f + row;
      uint4 v = *reinterpret_cast<const uint4*>(ebuf + row * kEpiPitch + ch * 16);
      if (m < M && n_lane < N) {
        uint32_t w[4] = {v.x, v.y, v.z, v.w};
        if (bias) {  // bf16 result + bf16 bias, rounded to bf16 (the separate add of the reference)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            w[i] = pack_bf16x2(__uint_as_float(w[i] << 16) + bias_f[2 * i],
                               __uint_as_float(w[i] & 0xFFFF0000u) + bias_f[2 * i + 1]);
          }
        }
        if (act == LL_ACT_GELU_TANH) {  // GELU (tanh form) of the bf16 value, computed in fp32, rounded to bf16
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            w[i] = pack_bf16x2(gelu_tanh_f32(__uint_as_float(w[i] << 16)),
                               gelu_tanh_f32(__uint_as_float(w[i] & 0xFFFF0000u)));
          }
        }
        if (epi.residual) {  // host side guarantees 16-byte aligned rows and N % 8 == 0 for this path
          const uint4 rv = *reinterpret_cast<const uint4*>(epi.residual + (int64_t)m * epi.ldr + n_lane);
          const uint32_t r[4] = {rv.x, rv.y, rv.z, rv.w};
          if (epi.gate) {
            const uint4 gv = *reinterpret_cast<const uint4*>(epi.gate + (int64_t)(m / epi.gate_rows) * epi.gate_stride + n_lane);
            const uint32_t g[4] = {gv.x, gv.y, gv.z, gv.w};
#pragma unroll
            for (int i = 0; i < 4; ++i)
              w[i] = pack_bf16x2(__uint_as_float(w[i] << 16) * __uint_as_float(g[i] << 16),
                                 __uint_as_float(w[i] & 0xFFFF0000u) * __uint_as_float(g[i] & 0xFFFF0000u));
          }
#pragma unroll
          for (int i = 0; i < 4; ++i)
            w[i] = pack_bf16x2(__uint_as_float(r[i] << 16) + __uint_as_float(w[i] << 16),
                               __uint_as_float(r[i] & 0xFFFF0000u) + __uint_as_float(w[i] & 0xFFFF0000u));
        }
        if (epi.sink.parts) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const bool lo_ok = n_lane + 2 * i < N, hi_ok = n_lane + 2 * i + 1 < N;
            if (lo_ok) out_max = fmaxf(out_max, fabsf(__uint_as_float(w[i] << 16)));
            if (hi_ok) out_max = fmaxf(out_max, fabsf(__uint_as_float(w[i] & 0xFFFF0000u)));
          }
        }
        uint16_t* dst = D + (int64_t)m * ldd + n_lane;
        if (vec_ok && n_lane + 8 <= N) {
          *reinterpret_cast<uint4*>(dst) = make_uint4(w[0], w[1], w[2], w[3]);
        } else {
          for (int i = 0; i < 8 && n_lane + i < N; ++i) dst[i] = (uint16_t)(w[i >> 1] >> (16 * (i & 1)));
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  if (epi.sink.parts) {  // one atomic per wave
    out_max = wave_max(out_max);
    if (lane == 0) amax_sink_update(epi.sink, sink_slot, out_max);
  }
}

template <int FA, int FB>
__global__ __launch_bounds__(kGemmThreads, 2) void gemm_w4a4_kernel(
    const uint8_t* __restrict__ Av, const uint8_t* __restrict__ As, const uint8_t* __restrict__ Bv0,
    const uint8_t* __restrict__ Bs0, const float* __restrict__ alpha_ptr0, const float* __restrict__ amax_a,
    const float* __restrict__ amax_b0, float inv_denom_a, float inv_denom_b0, int M, int N, int Mp, int Np, int Kp,
    uint16_t* __restrict__ D0, int64_t ldd0, int tiles_m, int tiles_n, GemmEpilogue epi, GemmGroups groups) {
  using S = GemmSmem<FA, FB>;
  const uint8_t* __restrict__ Bv = Bv0;
  const uint8_t* __restrict__ Bs = Bs0;
  const float* __restrict__ alpha_ptr = alpha_ptr0;
  const float* __restrict__ amax_b = amax_b0;
  float inv_denom_b = inv_denom_b0;
  uint16_t* __restrict__ D = D0;
  int64_t ldd = ldd0;
  const uint16_t* __restrict__ bias = epi.bias;
  const int act = epi.act;
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
  int tile_n = wg / tiles_m, tile_m = wg - tile_n * tiles_m;
  {
    // Inside an XCD's block of column panels, walk bands of kBandRows row tiles (row tile fastest, then column
    // panel, then the next band) instead of whole columns: the A rows of a band and the B panels then being
    // streamed fit the XCD's 4 MB L2 together, which cuts the L2 fetch of the FFN shapes by 18-23 %.
    constexpr int kBandRows = 8;
    const int total = tiles_m * tiles_n, per_xcd = total / 8;
    const int panels = per_xcd / tiles_m;                      // column panels per XCD
    if (total % 8 == 0 && panels * tiles_m == per_xcd) {
      const int xcd = wg / per_xcd, idx = wg - xcd * per_xcd;  // wg is already the XCD-remapped id
      const int band = min(idx / (kBandRows * panels), tiles_m / kBandRows);
      const int rows_in_band = min(kBandRows, tiles_m - band * kBandRows);
      const int in_band = idx - band * kBandRows * panels;
      const int c = in_band / rows_in_band;
      tile_m = band * kBandRows + (in_band - c * rows_in_band);
      tile_n = xcd * panels + c;
    }
  }
  if (groups.n > 1) {  // which product this column tile belongs to (uniform over the workgroup)
    const int g = tile_n / groups.tiles_n_each;
    tile_n -= g * groups.tiles_n_each;
    if (g > 0) {
      const GemmGroup& gg = groups.more[g - 1];
      Bv = gg.Bv;
      Bs = gg.Bs;
      alpha_ptr = gg.alpha;
      amax_b = gg.amax_b;
      inv_denom_b = gg.inv_denom_b;
      D = gg.D;
      ldd = gg.ldd;
      bias = gg.bias;
      epi.sink = gg.sink;
    }
  }
  const int row0 = tile_m * BM;  // first row of A (output row)
  const int col0 = tile_n * BN;  // first row of B (output column)

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;
  const int l32 = lane & 31, lh = lane >> 5;

  // ---- global -> LDS plan.  Load instruction i of a wave covers the 1024 bytes (16 rows) at piece index
  // i * 256 + wave * 64 of the A (or B) region; lane -> (row, stored position), and the piece of the row that
  // belongs there is position ^ (row / 4 % 4).
  constexpr int kAChunks = BM * 4 / kGemmThreads;  // 16-byte pieces of A values per thread
  constexpr int kBChunks = BN * 4 / kGemmThreads;
  const int64_t row_bytes = Kp >> 1;
  const uint8_t* a_src[kAChunks];
  const uint8_t* b_src[kBChunks];
  bool tail_piece;  // the thread's pieces lie in the second 64 K elements of a step (the same for all its pieces)
  {
    const int q = tid, r = q >> 2;
    tail_piece = (((q & 3) ^ ((r >> 2) & 3)) & 2) != 0;
  }
#pragma unroll
  for (int i = 0; i < kAChunks; ++i) {
    const int q = tid + i * kGemmThreads, r = q >> 2, ck = (q & 3) ^ ((r >> 2) & 3);
    const int gr = min(row0 + r, Mp - 1);
    a_src[i] = Av + (int64_t)gr * row_bytes + ck * 16;
  }
#pragma unroll
  for (int i = 0; i < kBChunks; ++i) {
    const int q = tid + i * kGemmThreads, r = q >> 2, ck = (q & 3) ^ ((r >> 2) & 3);
    const int gr = min(col0 + r, Np - 1);
    b_src[i] = Bv + (int64_t)gr * row_bytes + ck * 16;
  }
  // scales: 1024 contiguous bytes per 128-row block per step (two 128x4 tiles) = one load instruction of one wave
  constexpr int kARb = (BM + 127) / 128, kBRb = (BN + 127) / 128;
  const bool s_wave = wave < kARb + kBRb;
  const bool s_is_a = wave < kARb;
  const uint8_t* s_src;
  int s_dst;  // wave-uniform
  {
    const int rbi = s_is_a ? wave : wave - kARb;
    const int rb = s_is_a ? min(row0 / 128 + rbi, Mp / 128 - 1) : min(col0 / 128 + rbi, Np / 128 - 1);
    s_src = (s_is_a ? As : Bs) + (int64_t)rb * (Kp >> 6) * 512 + lane * 16;
    s_dst = S::kAVals + S::kBVals + (s_is_a ? 0 : S::kAScales) + rbi * 1024;
  }
  static_assert(kARb + kBRb <= 4, "one wave per 128-row block of scales");

  const int nk = (Kp + kBK - 1) / kBK;
  const uint8_t* zero16 = reinterpret_cast<const uint8_t*>(&g_gemm_zero16);
  // Kp is a multiple of 64 but maybe not of 128: in the last step the second 64 elements may not exist; the
  // lanes that would fetch them fetch zeros instead.
  auto load_step = [&](int t, int stage) {
    const uint32_t base = lds_address(smem + stage * S::kStage + wave * 1024);
    const uint32_t sbase = lds_address(smem + stage * S::kStage + s_dst);
    const bool second_half_valid = (t * kBK + 64) < Kp;
    if (second_half_valid) {
#pragma unroll
      for (int i = 0; i < kAChunks; ++i) load_to_lds_b128(a_src[i] + (int64_t)t * kRowBytes, base + i * 4096);
#pragma unroll
      for (int i = 0; i < kBChunks; ++i) load_to_lds_b128(b_src[i] + (int64_t)t * kRowBytes, base + S::kAVals + i * 4096);
      if (s_wave) load_to_lds_b128(s_src + (int64_t)t * 1024, sbase);
    } else {
#pragma unroll
      for (int i = 0; i < kAChunks; ++i)
        load_to_lds_b128(tail_piece ? zero16 : a_src[i] + (int64_t)t * kRowBytes, base + i * 4096);
#pragma unroll
      for (int i = 0; i < kBChunks; ++i)
        load_to_lds_b128(tail_piece ? zero16 : b_src[i] + (int64_t)t * kRowBytes, base + S::kAVals + i * 4096);
      if (s_wave) load_to_lds_b128(lane >= 32 ? zero16 : s_src + (int64_t)t * 1024, sbase);
    }
  };

  // ---- per-lane LDS read offsets
  // fragment f of A: rows wm*32*FA + 32 f + l32 ; piece 2 cc + lh of the row, stored at position piece ^ (row / 4 % 4):
  // the offsets below are those of cc = 0, cc = 1 flips the 32-byte bit
  int a_voff[FA], a_soff[FA], b_voff[FB], b_soff[FB];
#pragma unroll
  for (int f = 0; f < FA; ++f) {
    const int r = wm * 32 * FA + 32 * f + l32;
    const int rs = r + (row0 & 127);  // row inside the staged 128-row scale blocks (64-row tiles start mid-block)
    a_voff[f] = r * kLdsRow + 16 * (lh ^ ((r >> 2) & 3));
    a_soff[f] = S::kAVals + S::kBVals + (rs >> 7) * 1024 + (rs & 31) * 16 + ((rs & 127) >> 5) * 4 + 2 * lh;
  }
#pragma unroll
  for (int f = 0; f < FB; ++f) {
    const int r = wn * 32 * FB + 32 * f + l32;
    const int rs = r + (col0 & 127);
    b_voff[f] = S::kAVals + r * kLdsRow + 16 * (lh ^ ((r >> 2) & 3));
    b_soff[f] = S::kAVals + S::kBVals + S::kAScales + (rs >> 7) * 1024 + (rs & 31) * 16 + ((rs & 127) >> 5) * 4 + 2 * lh;
  }

  float16v acc[FB][FA];
#pragma unroll
  for (int g = 0; g < FB; ++g)
#pragma unroll
    for (int f = 0; f < FA; ++f)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[g][f][i] = 0.0f;

  // Register staging of one half step (64 K elements): raw packed dwords and the two f16 block scales.
  struct Half {
    uint4 a[FA], b[FB];
    half2v as[FA][2], bs[FB][2];
  };
  auto read_half = [&](Half& h, int stage, int cc) {
    const uint8_t* base = smem + stage * S::kStage;
#pragma unroll
    for (int f = 0; f < FA; ++f) {
      h.a[f] = *reinterpret_cast<const uint4*>(base + (a_voff[f] ^ (32 * cc)));
      const uint32_t sb = *reinterpret_cast<const uint16_t*>(base + a_soff[f] + 512 * cc);
      const half2v sc = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(sb, 1.0f, false);
      h.as[f][0] = half2v{sc[0], sc[0]};
      h.as[f][1] = half2v{sc[1], sc[1]};
    }
#pragma unroll
    for (int g = 0; g < FB; ++g) {
      h.b[g] = *reinterpret_cast<const uint4*>(base + (b_voff[g] ^ (32 * cc)));
      const uint32_t sb = *reinterpret_cast<const uint16_t*>(base + b_soff[g] + 512 * cc);
      const half2v sc = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(sb, 1.0f, false);
      h.bs[g][0] = half2v{sc[0], sc[0]};
      h.bs[g][1] = half2v{sc[1], sc[1]};
    }
  };
  struct Operands {
    half8v a[FA], b[FB];
  };
  auto decode = [&](Operands& o, const Half& h, int j) {
#pragma unroll
    for (int f = 0; f < FA; ++f) {
      const uint32_t w = j == 0 ? h.a[f].x : j == 1 ? h.a[f].y : j == 2 ? h.a[f].z : h.a[f].w;
      o.a[f] = decode8(w, h.as[f][j >> 1]);
    }
#pragma unroll
    for (int g = 0; g < FB; ++g) {
      const uint32_t w = j == 0 ? h.b[g].x : j == 1 ? h.b[g].y : j == 2 ? h.b[g].z : h.b[g].w;
      o.b[g] = decode8(w, h.bs[g][j >> 1]);
    }
  };
  auto mma = [&](const Operands& o) {
#pragma unroll
    for (int g = 0; g < FB; ++g)
#pragma unroll
      for (int f = 0; f < FA; ++f) acc[g][f] = __builtin_amdgcn_mfma_f32_32x32x16_f16(o.b[g], o.a[f], acc[g][f], 0, 0, 0);
  };
  // ---- main loop: two LDS stages, the loads of step t+1 in flight into the other stage while step t is
  // computed.
  {
    load_step(0, 0);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's pieces are in LDS
    __syncthreads();
    // A wave whose rows (or columns) all lie beyond M (N) only helps with the staging: in the last row of
    // tiles of M = 2640 with 256-row tiles that is half of the waves.
    const bool wave_has_output = row0 + wm * 32 * FA < M && col0 + wn * 32 * FB < N;
    if constexpr (FA * FB <= 4) {
      // Software pipeline inside the wave (the tiles with up to 2x2 fragments have the registers for it): the
      // operands of sub-step j + 1 are decoded between the MFMAs of sub-step j, one MFMA per group of VALU
      // instructions, so that the wave never issues MFMAs back to back (the second one would block the wave's
      // issue until the matrix pipe is free again).  The MFMAs of the last sub-step of a K step are issued after
      // the barrier, behind the LDS reads of the next step, whose latency they cover.
      Operands o[2];
      for (int t = 0; t < nk; ++t) {
        if (t + 1 < nk) load_step(t + 1, (t + 1) & 1);
        if (wave_has_output) {
          Half h[2];
          read_half(h[0], t & 1, 0);
          read_half(h[1], t & 1, 1);
          if (t > 0) mma(o[1]);
          decode(o[0], h[0], 0);
#pragma unroll
          for (int j = 0; j < 7; ++j) {
            decode(o[(j + 1) & 1], h[(j + 1) >> 2], (j + 1) & 3);
            mma(o[j & 1]);
#pragma unroll
            for (int g = 0; g < FA * FB; ++g) {
              __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                          // one MFMA
              __builtin_amdgcn_sched_group_barrier(0x002, (9 * (FA + FB) + FA * FB - 1) / (FA * FB), 0);  // its share of the decode
            }
          }
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
      }
      if (wave_has_output) mma(o[1]);
    } else {
      // Large tiles (8 fragments pairs per wave): the same software pipeline, with the packed dwords read from LDS
      // one sub-step ahead instead of a whole K step at a time, which is what lets it fit 256 registers.
      struct Raw {
        uint32_t a[FA], b[FB];
      };
      struct Scales {
        half2v a[FA][2], b[FB][2];
      };
      auto read_scales = [&](Scales& sc, int stage, int cc) {
        const uint8_t* base = smem + stage * S::kStage;
#pragma unroll
        for (int f = 0; f < FA; ++f) {
          const uint32_t sb = *reinterpret_cast<const uint16_t*>(base + a_soff[f] + 512 * cc);
          const half2v v = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(sb, 1.0f, false);
          sc.a[f][0] = half2v{v[0], v[0]};
          sc.a[f][1] = half2v{v[1], v[1]};
        }
#pragma unroll
        for (int g = 0; g < FB; ++g) {
          const uint32_t sb = *reinterpret_cast<const uint16_t*>(base + b_soff[g] + 512 * cc);
          const half2v v = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(sb, 1.0f, false);
          sc.b[g][0] = half2v{v[0], v[0]};
          sc.b[g][1] = half2v{v[1], v[1]};
        }
      };
      auto read_raw = [&](Raw& r, int stage, int j) {  // j = 0..7: half j / 4, dword j % 4 of the lane's 16-byte piece
        const uint8_t* base = smem + stage * S::kStage + 4 * (j & 3);
        const int flip = 32 * (j >> 2);
#pragma unroll
        for (int f = 0; f < FA; ++f) r.a[f] = *reinterpret_cast<const uint32_t*>(base + (a_voff[f] ^ flip));
#pragma unroll
        for (int g = 0; g < FB; ++g) r.b[g] = *reinterpret_cast<const uint32_t*>(base + (b_voff[g] ^ flip));
      };
      auto decode_raw = [&](Operands& o, const Raw& r, const Scales& sc, int jj) {
#pragma unroll
        for (int f = 0; f < FA; ++f) o.a[f] = decode8(r.a[f], sc.a[f][jj >> 1]);
#pragma unroll
        for (int g = 0; g < FB; ++g) o.b[g] = decode8(r.b[g], sc.b[g][jj >> 1]);
      };
      Operands o[2];
      for (int t = 0; t < nk; ++t) {
        if (t + 1 < nk) load_step(t + 1, (t + 1) & 1);
        if (wave_has_output) {
          Scales sc[2];
          Raw raw[2];
          read_raw(raw[0], t & 1, 0);
          read_scales(sc[0], t & 1, 0);
          read_raw(raw[1], t & 1, 1);
          read_scales(sc[1], t & 1, 1);
          if (t > 0) mma(o[1]);
          decode_raw(o[0], raw[0], sc[0], 0);
#pragma unroll
          for (int j = 0; j < 7; ++j) {
            if (j + 2 < 8) read_raw(raw[j & 1], t & 1, j + 2);
            decode_raw(o[(j + 1) & 1], raw[(j + 1) & 1], sc[(j + 1) >> 2], (j + 1) & 3);
            mma(o[j & 1]);
#pragma unroll
            for (int g = 0; g < FA * FB; ++g) {
              __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
              __builtin_amdgcn_sched_group_barrier(0x002, (8 * (FA + FB) + FA * FB - 1) / (FA * FB), 0);  // its share of the decode
            }
          }
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
      }
      if (wave_has_output) mma(o[1]);
    }
  }

  // ---- epilogue
  float alpha;
  if (alpha_ptr) {
    alpha = alpha_ptr[0];
  } else {
    alpha = (amax_a[0] * amax_b[0]) * (inv_denom_a * inv_denom_b);
  }
  gemm_epilogue<FA, FB>(acc, alpha, smem, wave, lane, row0 + wm * 32 * FA, col0 + wn * 32 * FB, M, N, D, ldd, bias, act, epi,
                        (uint32_t)blockIdx.x * 4 + wave);
}

// ============================================================================ persistent kernel
// One workgroup per compute unit, four waves, one per SIMD; each wave owns 128 rows x 128 columns of a 128 x 512
// output tile (4 x 4 MFMA tiles: all 256 accumulator registers, and four decode instructions per MFMA instead of the
// six to nine of the kernel above - on this chip a SIMD issues one vector instruction at a time, and under load its
// clock follows the power drawn, so instructions per MFMA are what the speed of the loop comes down to).  The A tile
// (128 rows) is shared by the four waves, the B rows are the wave's own.  The (tile, K step) pairs of the launch are
// cut into one equal share per workgroup (gemm_split.h); a tile whose K range several workgroups share is summed
// from their fp32 partial tiles by whoever arrives last, always in the same order.
// The main loop is a generated instruction sequence (gemm_loop_gen.py), included below as one asm statement.
constexpr int kPStage = 46080;                    // bytes per LDS stage, as in gemm_loop_gen.py
constexpr int kPSmem = 2 * kPStage + 16;          // two stages and a flag
constexpr int kPRecordFloats = 4 * 256 * 64;      // a workgroup's fp32 partial tile: per wave 256 registers of 64 lanes

struct PersistentParams {
  const uint8_t* Av;
  const uint8_t* As;
  const float* amax_a;
  float inv_denom_a;
  GemmGroup prod[kMaxGemmGroups];  // every product, the first one included
  int tiles_n_each;                // column tiles per product
  int M, N, Np, Kp, tiles_m;
  GemmDivision d;
  GemmEpilogue epi;                // bias and sink come from the product
  float* records;                  // [2 G] partial tiles of kPRecordFloats floats
  int* arrivals;                   // [split tiles], zero between launches
};

// Partial tiles travel between workgroups on different XCDs, whose L2 caches do not see each other's lines.
// Device-scope accesses (sc1) go past the L2: the stores write through, the loads fetch from memory.  They are
// written as instructions here because sixteen bytes at a time and many loads in flight are what makes the exchange
// cheap (as atomic operations of the language they come out one dword at a time, each load waited for).
typedef float float4v __attribute__((ext_vector_type(4)));
template <int OFFSET>
__device__ __forceinline__ void store_shared_f32x4(float* ptr, float4v v) {
  asm volatile("global_store_dwordx4 %0, %1, off offset:%2 sc1" ::"v"(ptr), "v"(v), "n"(OFFSET) : "memory");
}
template <int OFFSET>
__device__ __forceinline__ void load_shared_f32x4(const float* ptr, float4v& v) {
  asm volatile("global_load_dwordx4 %0, %1, off offset:%2 sc1" : "=v"(v) : "v"(ptr), "n"(OFFSET) : "memory");
}
// Waits for the loads above; the values pass through the statement so that nothing uses them before the wait.
__device__ __forceinline__ void wait_shared_loads(float4v (&v)[32]) {
  asm volatile("s_waitcnt vmcnt(0)"
               : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]), "+v"(v[8]),
                 "+v"(v[9]), "+v"(v[10]), "+v"(v[11]), "+v"(v[12]), "+v"(v[13]), "+v"(v[14]), "+v"(v[15]), "+v"(v[16]),
                 "+v"(v[17]), "+v"(v[18]), "+v"(v[19]), "+v"(v[20]), "+v"(v[21]), "+v"(v[22]), "+v"(v[23]), "+v"(v[24]),
                 "+v"(v[25]), "+v"(v[26]), "+v"(v[27]), "+v"(v[28]), "+v"(v[29])
               :
               : "memory");
  asm volatile("" : "+v"(v[30]), "+v"(v[31])::"memory");
}
// A wave's part of a record: 64 groups of four accumulator registers, group q at floats [q * 256 + lane * 4, + 4).
// Group q = 16 gi + 4 f + rg holds acc[gi][f][4 rg .. 4 rg + 3].
__device__ __forceinline__ void store_partial_tile(float* rec, float16v (&acc)[4][4]) {
#pragma unroll
  for (int q0 = 0; q0 < 64; q0 += 4) {
    float* base = rec + q0 * 256;
    const int gi = q0 >> 4, f = (q0 >> 2) & 3;
    const float16v& a = acc[gi][f];
    store_shared_f32x4<0>(base, float4v{a[0], a[1], a[2], a[3]});
    store_shared_f32x4<1024>(base, float4v{a[4], a[5], a[6], a[7]});
    store_shared_f32x4<2048>(base, float4v{a[8], a[9], a[10], a[11]});
    store_shared_f32x4<3072>(base, float4v{a[12], a[13], a[14], a[15]});
  }
}
// acc = record (ADD false) or acc += record, thirty-two loads of sixteen bytes in flight at a time.
template <bool ADD>
__device__ __forceinline__ void load_partial_tile(const float* rec, float16v (&acc)[4][4]) {
#pragma unroll
  for (int g2 = 0; g2 < 4; g2 += 2) {
    float4v t[32];
#pragma unroll
    for (int x = 0; x < 8; ++x) {  // x = 4 (gi - g2) + f
      const float* base = rec + (g2 * 16 + x * 4) * 256;
      load_shared_f32x4<0>(base, t[4 * x]);
      load_shared_f32x4<1024>(base, t[4 * x + 1]);
      load_shared_f32x4<2048>(base, t[4 * x + 2]);
      load_shared_f32x4<3072>(base, t[4 * x + 3]);
    }
    wait_shared_loads(t);
#pragma unroll
    for (int x = 0; x < 8; ++x)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        if (ADD) acc[g2 + (x >> 2)][x & 3][i] += t[4 * x + (i >> 2)][i & 3];
        else acc[g2 + (x >> 2)][x & 3][i] = t[4 * x + (i >> 2)][i & 3];
      }
  }
}

#define LL_V10(a) "v" #a "0", "v" #a "1", "v" #a "2", "v" #a "3", "v" #a "4", "v" #a "5", "v" #a "6", "v" #a "7", "v" #a "8", "v" #a "9"

__global__ __launch_bounds__(256) void gemm_w4a4_persistent_kernel(PersistentParams p) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // Consecutive hardware workgroup numbers go to different XCDs; every XCD gets a contiguous range of the shares
  // instead, so that workgroups that share an L2 work on neighbouring tiles (the same B rows, adjacent A rows).
  const uint32_t g = p.d.G % 8 == 0 ? (blockIdx.x & 7) * (p.d.G / 8) + (blockIdx.x >> 3) : blockIdx.x;
  GemmCursor at = gemm_start_of_work(g, p.d);
  const uint32_t row_bytes = (uint32_t)p.Kp >> 1;
  const uint32_t rb16 = 16u * row_bytes;
  const uint32_t swz = (l32 >> 2) & 3;
  // What a lane contributes to the addresses of the loop (gemm_loop_gen.py): its row and 16-byte piece in a load of
  // 16 rows; its row, piece and scale group in the LDS reads; the shift that picks its pair of scale bytes.
  const uint32_t lane_voff = (uint32_t)(lane >> 2) * row_bytes + 16u * ((lane & 3) ^ ((lane >> 4) & 3));
  const uint32_t lane_soff = (uint32_t)lane * 16u;
  const uint32_t ard = (uint32_t)l32 * 64u + 16u * ((lh ^ (swz & 1)) | (swz & 2));
  const uint32_t sard = 40960u + (uint32_t)l32 * 16u;
  const uint32_t sh = 16u * lh;
  int* flag = reinterpret_cast<int*>(smem + 2 * kPStage);

  GemmSegment seg;
  while (gemm_next_segment(at, g, p.d, seg)) {
    const int tile_m = (int)(seg.tile % (uint32_t)p.tiles_m), tile_n_all = (int)(seg.tile / (uint32_t)p.tiles_m);
    const int pi = tile_n_all / p.tiles_n_each, tile_n = tile_n_all - pi * p.tiles_n_each;
    const GemmGroup& pr = p.prod[pi];
    const int row0 = tile_m * kPTileM, col0 = tile_n * kPTileN;
    // The wave's 128 rows of B; a wave whose columns lie beyond the padded matrix recomputes the last block (its
    // output is masked).
    const int bcol = min(col0 + 128 * wave, p.Np - 128);
    const uint32_t nsteps = seg.end - seg.begin;
    const uint32_t voff = lane_voff + seg.begin * 64u, soff = lane_soff + seg.begin * 1024u;
    const uint8_t* sA = p.Av + (size_t)(row0 + 32 * wave) * row_bytes;
    const uint8_t* sB = pr.Bv + (size_t)bcol * row_bytes;
    const uint8_t* sAs = p.As + (size_t)(row0 >> 7) * (size_t)(p.Kp >> 6) * 512;
    const uint8_t* sBs = pr.Bs + (size_t)(bcol >> 7) * (size_t)(p.Kp >> 6) * 512;
    float16v acc[4][4];
#pragma unroll
    for (int gi = 0; gi < 4; ++gi)
#pragma unroll
      for (int f = 0; f < 4; ++f)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[gi][f][i] = 0.0f;
    __syncthreads();  // LDS is free: the previous segment's epilogue is over in every wave
    asm volatile(
#include "gemm_loop_gfx950.inc"
        : "+a"(acc[0][0]), "+a"(acc[0][1]), "+a"(acc[0][2]), "+a"(acc[0][3]), "+a"(acc[1][0]), "+a"(acc[1][1]), "+a"(acc[1][2]),
          "+a"(acc[1][3]), "+a"(acc[2][0]), "+a"(acc[2][1]), "+a"(acc[2][2]), "+a"(acc[2][3]), "+a"(acc[3][0]), "+a"(acc[3][1]),
          "+a"(acc[3][2]), "+a"(acc[3][3])
        : "s"(nsteps), "v"(voff), "v"(soff), "v"(ard), "v"(sard), "v"(sh), "s"(sA), "s"(sB), "s"(rb16), "s"(sAs), "s"(sBs), "s"(wave)
        : "memory", "scc", "vcc", "v0", "v1", "v2", "v3", "v4", "v5", "v6", "v7", "v8", "v9", LL_V10(1), LL_V10(2), LL_V10(3), LL_V10(4),
          LL_V10(5), LL_V10(6), LL_V10(7), LL_V10(8), LL_V10(9), LL_V10(10), LL_V10(11), LL_V10(12), LL_V10(13), LL_V10(14), LL_V10(15),
          LL_V10(16), "s56", "s57", "s58", "s59", "s60", "s61", "s62", "s63", "s64", "s65", "s66", "s67", "s68", "s69", "s70", "s71",
          "s72", "s73", "s74", "s75", "s76", "s77", "s78", "s79", "s80", "s81", "s82", "s83", "s84", "s85", "s86", "s87");

    bool write_out = true;
    if (seg.begin != 0 || seg.end != p.d.nk) {
      // Part of a tile.  Whoever arrives last at a tile adds the parts up, from the part with the last K steps
      // backwards whoever does it, so the result does not depend on the order of arrival; the others leave their
      // accumulators in a record and count their arrival.  The workgroup that holds the last part is normally the
      // last to arrive (shares are walked backwards): if a look at the counter shows that, it goes on from its
      // registers without writing a record.
      const uint32_t split_tile = seg.tile - p.d.whole_rounds * p.d.G;  // the tile's number among the split ones
      uint32_t g_first, g_last;
      gemm_parts_of_tile(split_tile, p.d, g_first, g_last);
      const int others = (int)(g_last - g_first);
      if (tid == 0)
        *flag = g == g_last && __hip_atomic_load(p.arrivals + split_tile, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == others;
      __syncthreads();
      const bool from_registers = *flag != 0;
      write_out = from_registers;
      if (!from_registers) {
        store_partial_tile(p.records + (size_t)gemm_record_of_part(g, split_tile, p.d) * kPRecordFloats + wave * (256 * 64) + lane * 4, acc);
        // Every wave waits until its own record stores are complete (a write-through store is acknowledged once it
        // is visible device-wide) before the barrier behind which thread 0 counts the arrival.
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
        if (tid == 0)
          *flag = __hip_atomic_fetch_add(p.arrivals + split_tile, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == others;
        __syncthreads();
        write_out = *flag != 0;
      }
      if (write_out) {
        if (tid == 0) __hip_atomic_store(p.arrivals + split_tile, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
        // The part with the last K steps comes first (from the registers, or read back like the others), then the
        // parts before it one by one: the same sequence of additions whoever does it.
        for (int gg = (int)g_last - (from_registers ? 1 : 0); gg >= (int)g_first; --gg) {
          const float* theirs = p.records + (size_t)gemm_record_of_part((uint32_t)gg, split_tile, p.d) * kPRecordFloats + wave * (256 * 64) + lane * 4;
          if (!from_registers && gg == (int)g_last) load_partial_tile<false>(theirs, acc);
          else load_partial_tile<true>(theirs, acc);
        }
      }
    }
    if (write_out) {
      const float alpha = pr.alpha ? pr.alpha[0] : (p.amax_a[0] * pr.amax_b[0]) * (p.inv_denom_a * pr.inv_denom_b);
      GemmEpilogue epi = p.epi;
      epi.sink = pr.sink;
      gemm_epilogue<4, 4>(acc, alpha, smem, wave, lane, row0, col0 + 128 * wave, p.M, p.N, pr.D, pr.ldd, pr.bias, epi.act, epi,
                          seg.tile * 4 + wave);
    }
  }
}
#undef LL_V10


// ============================================================================ tile kernel, hand-scheduled loop
// gemm_w4a4_kernel<FA, FB> with its main loop replaced by a generated instruction sequence
// (gemm_tile_loop_gen.py): the same workgroup -> tile map, the same arithmetic in the same order (the accumulators
// receive the same MFMAs in the same sequence, so the results are bit-identical), the same epilogue.  Needs Kp to be a
// multiple of 128.  Tiles 256 x 128 and 128 x 256: the 128 x 128 tile, with 8 decode instructions per MFMA against 6, is
// bound by the issue of those whatever their order (measured: 53.5 us against the compiler's 52.6 on 2640 x 3072 x 3072).
template <int FA, int FB>
struct AsmTile {
  static constexpr int BM = 64 * FA, BN = 64 * FB;
  static constexpr int kAScales = (BM + BN) * 64;                      // LDS offsets inside a stage, as in the generator
  static constexpr int kBScales = kAScales + 1024 * (BM / 128);
  static constexpr int kStage = kBScales + 1024 * (BN / 128);
  static constexpr int kScaleBlocks = BM / 128 + BN / 128;
};

#define LL_V10(a) "v" #a "0", "v" #a "1", "v" #a "2", "v" #a "3", "v" #a "4", "v" #a "5", "v" #a "6", "v" #a "7", "v" #a "8", "v" #a "9"
#define LL_ASM_TILE_INPUTS                                                                                              \
  "s"(nsteps), "v"(lane_voff), "v"(lane_soff), "v"(ard), "v"(brd), "v"(sard), "v"(sbrd), "v"(sh), "s"(sA), "s"(sB), "s"(sS),    \
      "s"(rb16), "s"(adst), "s"(bdst), "s"(sdst), "s"(idle)
#define LL_ASM_TILE_SGPRS                                                                                               \
  "s56", "s57", "s58", "s59", "s60", "s61", "s62", "s63", "s64", "s65", "s66", "s67", "s68", "s69", "s70", "s71", "s72", "s73",  \
      "s74", "s75", "s76", "s77", "s78", "s79", "s80", "s81", "s82", "s83", "s84", "s85", "s86", "s87"

template <int FA, int FB>
__global__ __launch_bounds__(kGemmThreads, 2) void gemm_w4a4_asm_kernel(
    const uint8_t* __restrict__ Av, const uint8_t* __restrict__ As, const uint8_t* __restrict__ Bv0,
    const uint8_t* __restrict__ Bs0, const float* __restrict__ alpha_ptr0, const float* __restrict__ amax_a,
    const float* __restrict__ amax_b0, float inv_denom_a, float inv_denom_b0, int M, int N, int Mp, int Np, int Kp,
    uint16_t* __restrict__ D0, int64_t ldd0, int tiles_m, int tiles_n, GemmEpilogue epi, GemmGroups groups) {
  using T = AsmTile<FA, FB>;
  constexpr int BM = T::BM, BN = T::BN;
  const uint8_t* __restrict__ Bv = Bv0;
  const uint8_t* __restrict__ Bs = Bs0;
  const float* __restrict__ alpha_ptr = alpha_ptr0;
  const float* __restrict__ amax_b = amax_b0;
  float inv_denom_b = inv_denom_b0;
  uint16_t* __restrict__ D = D0;
  int64_t ldd = ldd0;
  const uint16_t* __restrict__ bias = epi.bias;
  const int act = epi.act;
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];  // the loop forms addresses by xor: whole pieces of 64 bytes

  // Workgroup -> tile, as in gemm_w4a4_kernel.
  int wg = blockIdx.x;
  {
    const int total = tiles_m * tiles_n;
    const int per_xcd = (total + 7) / 8;
    const int xcd = wg & 7, idx = wg >> 3;
    const int remapped = xcd * per_xcd + idx;
    if (total % 8 == 0) wg = remapped;
  }
  int tile_n = wg / tiles_m, tile_m = wg - tile_n * tiles_m;
  {
    constexpr int kBandRows = 8;
    const int total = tiles_m * tiles_n, per_xcd = total / 8;
    const int panels = per_xcd / tiles_m;
    if (total % 8 == 0 && panels * tiles_m == per_xcd) {
      const int xcd = wg / per_xcd, idx = wg - xcd * per_xcd;
      const int band = min(idx / (kBandRows * panels), tiles_m / kBandRows);
      const int rows_in_band = min(kBandRows, tiles_m - band * kBandRows);
      const int in_band = idx - band * kBandRows * panels;
      const int c = in_band / rows_in_band;
      tile_m = band * kBandRows + (in_band - c * rows_in_band);
      tile_n = xcd * panels + c;
    }
  }
  if (groups.n > 1) {
    const int g = tile_n / groups.tiles_n_each;
    tile_n -= g * groups.tiles_n_each;
    if (g > 0) {
      const GemmGroup& gg = groups.more[g - 1];
      Bv = gg.Bv;
      Bs = gg.Bs;
      alpha_ptr = gg.alpha;
      amax_b = gg.amax_b;
      inv_denom_b = gg.inv_denom_b;
      D = gg.D;
      ldd = gg.ldd;
      bias = gg.bias;
      epi.sink = gg.sink;
    }
  }
  const int row0 = tile_m * BM, col0 = tile_n * BN;
  const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave & 1, wn = wave >> 1;

  // What the loop needs from here (gemm_tile_loop_gen.py): the wave's quarter of the A and B rows of the tile to load
  // (rows beyond the padded matrix are replaced by the last rows: their outputs are masked), its scale block, the
  // lane's offsets in a load of 16 rows, its read addresses in LDS, the shift that picks its pair of scale bytes.
  const uint32_t row_bytes = (uint32_t)Kp >> 1;
  const uint32_t swz = (l32 >> 2) & 3;
  const uint32_t lane_voff = (uint32_t)(lane >> 2) * row_bytes + 16u * ((lane & 3) ^ ((lane >> 4) & 3));
  const uint32_t lane_soff = (uint32_t)lane * 16u;
  const uint32_t lds0 = lds_address(smem);  // the loop addresses LDS with plain offsets: they start where smem does
  const uint32_t lane_rd = lds0 + (uint32_t)l32 * 64u + 16u * ((lh ^ (swz & 1)) | (swz & 2));
  const uint32_t ard = (uint32_t)(32 * FA * wm) * 64u + lane_rd;
  const uint32_t brd = (uint32_t)(BM * 64) + (uint32_t)(32 * FB * wn) * 64u + lane_rd;
  // a wave with four fragments of an operand owns a whole 128-row group of its scales, one with two owns half of one
  const uint32_t sard = lds0 + T::kAScales + (uint32_t)l32 * 16u + (FA == 4 ? 1024u : 8u) * wm;
  const uint32_t sbrd = lds0 + T::kBScales + (uint32_t)l32 * 16u + (FB == 4 ? 1024u : 8u) * wn;
  const uint32_t sh = 16u * lh;
  const int a_rows = min(row0 + (BM / 4) * wave, Mp - BM / 4), b_rows = min(col0 + (BN / 4) * wave, Np - BN / 4);
  const uint8_t* sA = Av + (size_t)a_rows * row_bytes;
  const uint8_t* sB = Bv + (size_t)b_rows * row_bytes;
  // scale blocks of a K step (1 KB per 128 rows): those of A, then those of B; wave w loads block w (the last waves
  // the last block again)
  const int block = min(wave, T::kScaleBlocks - 1);
  const uint8_t* sS = block < BM / 128 ? As + (size_t)min((row0 >> 7) + block, (Mp >> 7) - 1) * (size_t)(Kp >> 6) * 512
                                       : Bs + (size_t)min((col0 >> 7) + block - BM / 128, (Np >> 7) - 1) * (size_t)(Kp >> 6) * 512;
  const uint32_t adst = lds0 + (uint32_t)wave * (BM / 4) * 64u, bdst = lds0 + (uint32_t)(BM * 64) + (uint32_t)wave * (BN / 4) * 64u;
  const uint32_t sdst = lds0 + T::kAScales + 1024u * (uint32_t)block;
  const uint32_t nsteps = (uint32_t)Kp >> 7, rb16 = 16u * row_bytes;
  // A wave whose rows (or columns) all lie beyond M (N) only helps with the staging.
  const uint32_t idle = __builtin_amdgcn_readfirstlane(row0 + wm * 32 * FA < M && col0 + wn * 32 * FB < N ? 0 : 1);

  float16v acc[FB][FA];
#pragma unroll
  for (int g = 0; g < FB; ++g)
#pragma unroll
    for (int f = 0; f < FA; ++f)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[g][f][i] = 0.0f;
  if constexpr (FA == 4 && FB == 2) {
    asm volatile(
#include "gemm_tile_loop_42_gfx950.inc"
        : "+a"(acc[0][0]), "+a"(acc[0][1]), "+a"(acc[0][2]), "+a"(acc[0][3]), "+a"(acc[1][0]), "+a"(acc[1][1]), "+a"(acc[1][2]),
          "+a"(acc[1][3])
        : LL_ASM_TILE_INPUTS
        : "memory", "scc", "vcc", "v0", "v1", "v2", "v3", "v4", "v5", "v6", "v7", "v8", "v9", LL_V10(1), LL_V10(2), LL_V10(3),
          LL_V10(4), LL_V10(5), LL_V10(6), LL_V10(7), LL_V10(8), LL_V10(9), "v100", "v101", LL_ASM_TILE_SGPRS);
  } else {
    static_assert(FA == 2 && FB == 4, "generated loops exist for the 256 x 128 and the 128 x 256 tile");
    asm volatile(
#include "gemm_tile_loop_24_gfx950.inc"
        : "+a"(acc[0][0]), "+a"(acc[0][1]), "+a"(acc[1][0]), "+a"(acc[1][1]), "+a"(acc[2][0]), "+a"(acc[2][1]), "+a"(acc[3][0]),
          "+a"(acc[3][1])
        : LL_ASM_TILE_INPUTS
        : "memory", "scc", "vcc", "v0", "v1", "v2", "v3", "v4", "v5", "v6", "v7", "v8", "v9", LL_V10(1), LL_V10(2), LL_V10(3),
          LL_V10(4), LL_V10(5), LL_V10(6), LL_V10(7), LL_V10(8), LL_V10(9), "v100", "v101", LL_ASM_TILE_SGPRS);
  }
  __syncthreads();  // every wave has left the stages: the epilogue reuses them

  float alpha;
  if (alpha_ptr) {
    alpha = alpha_ptr[0];
  } else {
    alpha = (amax_a[0] * amax_b[0]) * (inv_denom_a * inv_denom_b);
  }
  gemm_epilogue<FA, FB>(acc, alpha, smem, wave, lane, row0 + wm * 32 * FA, col0 + wn * 32 * FB, M, N, D, ldd, bias, act, epi,
                        (uint32_t)blockIdx.x * 4 + wave);
}
// ============================================================================ one workgroup per compute unit, K split inside it
// A 128 x 256 tile by eight waves: waves 0-3 and 4-7 hold the same 2 x 2 arrangement of 64 x 128 wave tiles; of every K
// step of 128 the first group multiplies the first 64 elements, the second group the other 64 (generated loop,
// gemm_tile_loop_gen.py --waves 8: three LDS stages in a ring, the loads of a step shared by all eight waves).  Behind
// the loop the partners exchange half of their partial tiles through LDS - wave w keeps its first 32 rows and
// receives the partner's, wave w + 4 the other 32 - and every wave runs the epilogue on the 32 x 128 sums it holds.
// fp32 addition is commutative, so the result does not depend on which side adds; it differs from the kernels above
// by the order of the fp32 additions only (two halves of K summed separately).  For shapes that give at most one
// 128 x 256 tile per compute unit: two waves per SIMD with 6 decode instructions per MFMA, where 128 x 128 tiles in
// pairs need 8.  Kp is a multiple of 128.
constexpr int kSplitThreads = 512;
constexpr int kSplitStages = 3;
constexpr int kSplitSmem = 8 * 64 * 64 * 4;  // the exchange: 64 accumulator registers of 8 waves; the ring needs less

__global__ __launch_bounds__(kSplitThreads) void gemm_w4a4_asm8_kernel(
    const uint8_t* __restrict__ Av, const uint8_t* __restrict__ As, const uint8_t* __restrict__ Bv0,
    const uint8_t* __restrict__ Bs0, const float* __restrict__ alpha_ptr0, const float* __restrict__ amax_a,
    const float* __restrict__ amax_b0, float inv_denom_a, float inv_denom_b0, int M, int N, int Mp, int Np, int Kp,
    uint16_t* __restrict__ D0, int64_t ldd0, int tiles_m, int tiles_n, GemmEpilogue epi, GemmGroups groups) {
  constexpr int FA = 2, FB = 4;
  using T = AsmTile<FA, FB>;
  constexpr int BM = T::BM, BN = T::BN;
  static_assert(kSplitStages * T::kStage <= kSplitSmem && 8 * 32 * (64 * FB + 16) <= kSplitSmem, "ring and epilogue patches fit");
  const uint8_t* __restrict__ Bv = Bv0;
  const uint8_t* __restrict__ Bs = Bs0;
  const float* __restrict__ alpha_ptr = alpha_ptr0;
  const float* __restrict__ amax_b = amax_b0;
  float inv_denom_b = inv_denom_b0;
  uint16_t* __restrict__ D = D0;
  int64_t ldd = ldd0;
  const uint16_t* __restrict__ bias = epi.bias;
  const int act = epi.act;
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];  // the loop forms addresses by xor: whole pieces of 64 bytes

  // Workgroup -> tile.  The grid is the number of tiles rounded up to a multiple of 8; workgroup b runs on XCD b % 8,
  // and every XCD takes a run of consecutive tiles (whole column panels first), so that its L2 holds the A rows once
  // and few B panels.
  const int total = tiles_m * tiles_n;
  const int per_xcd = (int)gridDim.x >> 3;
  const int tile = ((int)blockIdx.x & 7) * per_xcd + ((int)blockIdx.x >> 3);
  if (tile >= total) return;
  int tile_n = tile / tiles_m;
  const int tile_m = tile - tile_n * tiles_m;
  if (groups.n > 1) {
    const int g = tile_n / groups.tiles_n_each;
    tile_n -= g * groups.tiles_n_each;
    if (g > 0) {
      const GemmGroup& gg = groups.more[g - 1];
      Bv = gg.Bv;
      Bs = gg.Bs;
      alpha_ptr = gg.alpha;
      amax_b = gg.amax_b;
      inv_denom_b = gg.inv_denom_b;
      D = gg.D;
      ldd = gg.ldd;
      bias = gg.bias;
      epi.sink = gg.sink;
    }
  }
  const int row0 = tile_m * BM, col0 = tile_n * BN;
  const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = wave >> 2, wm = wave & 1, wn = (wave >> 1) & 1;

  const uint32_t row_bytes = (uint32_t)Kp >> 1;
  const uint32_t swz = (l32 >> 2) & 3;
  const uint32_t lane_voff = (uint32_t)(lane >> 2) * row_bytes + 16u * ((lane & 3) ^ ((lane >> 4) & 3));
  const uint32_t lane_soff = (uint32_t)lane * 16u;
  // the lane's 16-byte piece of this wave's half of a K step: piece 2 half + lane / 32, stored at piece ^ swz
  const uint32_t lds0 = lds_address(smem);  // the loop addresses LDS with plain offsets: they start where smem does
  const uint32_t lane_rd = lds0 + (((uint32_t)l32 * 64u + 16u * ((lh ^ (swz & 1)) | (swz & 2))) ^ (32u * half));
  const uint32_t ard = (uint32_t)(32 * FA * wm) * 64u + lane_rd;
  const uint32_t brd = (uint32_t)(BM * 64) + (uint32_t)(32 * FB * wn) * 64u + lane_rd;
  // scales of a K step and a 128-row group: two halves of 512 bytes, 16 bytes per row of 32 and half
  const uint32_t sard = lds0 + T::kAScales + 512u * half + (uint32_t)l32 * 16u + 8u * wm;
  const uint32_t sbrd = lds0 + T::kBScales + 512u * half + 1024u * wn + (uint32_t)l32 * 16u;
  const uint32_t sh = 16u * lh;
  // loads of a K step: wave w brings 16 rows of A, 32 rows of B, and (waves 0-2) one 1 KB block of scales
  const int a_rows = min(row0 + 16 * wave, Mp - 16), b_rows = min(col0 + 32 * wave, Np - 32);
  const uint8_t* sA = Av + (size_t)a_rows * row_bytes;
  const uint8_t* sB = Bv + (size_t)b_rows * row_bytes;
  const int block = min(wave, T::kScaleBlocks - 1);
  const uint8_t* sS = block < BM / 128 ? As + (size_t)min((row0 >> 7) + block, (Mp >> 7) - 1) * (size_t)(Kp >> 6) * 512
                                       : Bs + (size_t)min((col0 >> 7) + block - BM / 128, (Np >> 7) - 1) * (size_t)(Kp >> 6) * 512;
  const uint32_t adst = lds0 + (uint32_t)wave * 1024u, bdst = lds0 + (uint32_t)(BM * 64) + (uint32_t)wave * 2048u;
  const uint32_t sdst = lds0 + T::kAScales + 1024u * (uint32_t)block;
  const uint32_t hassc = __builtin_amdgcn_readfirstlane(wave < T::kScaleBlocks ? 1 : 0);
  const uint32_t nsteps = (uint32_t)Kp >> 7, rb16 = 16u * row_bytes;
  const uint32_t idle = __builtin_amdgcn_readfirstlane(row0 + wm * 32 * FA < M && col0 + wn * 32 * FB < N ? 0 : 1);

  float16v acc[FB][FA];
#pragma unroll
  for (int g = 0; g < FB; ++g)
#pragma unroll
    for (int f = 0; f < FA; ++f)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[g][f][i] = 0.0f;
  asm volatile(
#include "gemm_tile_loop_24w8_gfx950.inc"
      : "+a"(acc[0][0]), "+a"(acc[0][1]), "+a"(acc[1][0]), "+a"(acc[1][1]), "+a"(acc[2][0]), "+a"(acc[2][1]), "+a"(acc[3][0]),
        "+a"(acc[3][1])
      : LL_ASM_TILE_INPUTS, "s"(hassc)
      : "memory", "scc", "vcc", "v0", "v1", "v2", "v3", "v4", "v5", "v6", "v7", "v8", "v9", LL_V10(1), LL_V10(2), LL_V10(3),
        LL_V10(4), LL_V10(5), LL_V10(6), LL_V10(7), LL_V10(8), LL_V10(9), "v100", "v101", LL_ASM_TILE_SGPRS);
  __syncthreads();  // every wave has left the ring

  // Everything behind the loop is computed from this copy of the lane number: the loop leaves the compiler 26
  // registers, and what it would otherwise prepare for the epilogue ahead of the loop does not fit them.
  int lane_after = lane;
  asm volatile("" : "+v"(lane_after));
  // Exchange: 16 KB per receiving wave, [register / 4][lane][4 floats].  Waves 0-3 keep their first 32 rows, waves 4-7
  // their second 32 (selects instead of two code paths: the choice is uniform and made once per tile).
  float* out = reinterpret_cast<float*>(smem) + (size_t)(wave ^ 4) * 4096 + lane_after * 4;
  const float* in = reinterpret_cast<const float*>(smem) + (size_t)wave * 4096 + lane_after * 4;
  float16v kept[FB][1];
#pragma unroll
  for (int g = 0; g < FB; ++g)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      float send[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float first = acc[g][0][4 * q + i], second = acc[g][1][4 * q + i];
        send[i] = half ? first : second;
        kept[g][0][4 * q + i] = half ? second : first;
      }
      *reinterpret_cast<float4*>(out + (4 * g + q) * 256) = make_float4(send[0], send[1], send[2], send[3]);
    }
  __syncthreads();
#pragma unroll
  for (int g = 0; g < FB; ++g)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float4 v = *reinterpret_cast<const float4*>(in + (4 * g + q) * 256);
      kept[g][0][4 * q] += v.x;
      kept[g][0][4 * q + 1] += v.y;
      kept[g][0][4 * q + 2] += v.z;
      kept[g][0][4 * q + 3] += v.w;
    }
  __syncthreads();  // the patches of the epilogue overlap the exchange
  float alpha;
  if (alpha_ptr) {
    alpha = alpha_ptr[0];
  } else {
    alpha = (amax_a[0] * amax_b[0]) * (inv_denom_a * inv_denom_b);
  }
  gemm_epilogue<1, FB>(kept, alpha, smem, wave, lane_after, row0 + wm * 32 * FA + 32 * half, col0 + wn * 32 * FB, M, N, D, ldd, bias, act,
                       epi, (uint32_t)blockIdx.x * 8 + wave);
}
#undef LL_ASM_TILE_SGPRS
#undef LL_ASM_TILE_INPUTS
#undef LL_V10

static std::atomic<int> g_gemm_schedule{LL_GEMM_AUTO};

template <int FA, int FB>
int launch_gemm(const uint8_t* Av, const uint8_t* As, const uint8_t* Bv, const uint8_t* Bs, const float* alpha,
                const float* amax_a, const float* amax_b, float denom_a, float denom_b, int M, int N, int Mp, int Np,
                int Kp, void* D, int64_t ldd, const GemmEpilogue& epi, GemmGroups groups, hipStream_t stream,
                bool hand_scheduled) {
  using S = GemmSmem<FA, FB>;
  groups.tiles_n_each = (N + S::BN - 1) / S::BN;
  const int tiles_m = (M + S::BM - 1) / S::BM, tiles_n = groups.tiles_n_each * groups.n;
  if constexpr (FA + FB == 6) {
    if (hand_scheduled) {
      // the same kernel with its main loop as a hand-scheduled instruction sequence
      using T = AsmTile<FA, FB>;
      static_assert(2 * T::kStage >= 4 * 32 * (64 * FB + 16), "the epilogue's patches fit the stages");
      const size_t smem = 2 * T::kStage;
      static std::atomic<uint64_t> lds_allowed{0};
      if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(&gemm_w4a4_asm_kernel<FA, FB>), smem, lds_allowed, "ll_nvfp4_gemm_tnt")) return rc;
      hipLaunchKernelGGL((gemm_w4a4_asm_kernel<FA, FB>), dim3((unsigned)(tiles_m * tiles_n)), dim3(kGemmThreads), smem, stream, Av,
                         As, Bv, Bs, alpha, amax_a, amax_b, 1.0f / denom_a, 1.0f / denom_b, M, N, Mp, Np, Kp,
                         static_cast<uint16_t*>(D), ldd, tiles_m, tiles_n, epi, groups);
      LL_CHECK_LAUNCH("gemm_w4a4_asm_kernel");
      return LL_OK;
    }
  }
  const size_t smem = 2 * S::kStage;
  static std::atomic<uint64_t> lds_allowed{0};  // one per tile configuration
  if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(&gemm_w4a4_kernel<FA, FB>), smem, lds_allowed, "ll_nvfp4_gemm_tnt")) return rc;
  hipLaunchKernelGGL((gemm_w4a4_kernel<FA, FB>), dim3((unsigned)(tiles_m * tiles_n)), dim3(kGemmThreads), smem, stream,
                     Av, As, Bv, Bs, alpha, amax_a, amax_b, 1.0f / denom_a, 1.0f / denom_b, M, N, Mp, Np, Kp,
                     static_cast<uint16_t*>(D), ldd, tiles_m, tiles_n, epi, groups);
  LL_CHECK_LAUNCH("gemm_w4a4_kernel");
  return LL_OK;
}

int dispatch_gemm(const uint8_t* A_values, const uint8_t* A_scales, const uint8_t* B_values, const uint8_t* B_scales,
                  const float* alpha, const float* amax_a, const float* amax_b, float denom_a, float denom_b, int64_t M,
                  int64_t N, int64_t Mp, int64_t Np, int64_t Kp, void* D, int64_t ldd, const GemmEpilogue& epi,
                  const GemmGroups& groups, hipStream_t s);

}  // namespace ll

extern "C" int ll_nvfp4_gemm_tnt(const uint8_t* A_values, const uint8_t* A_scales, const uint8_t* B_values,
                                 const uint8_t* B_scales, const float* alpha, const float* amax_a,
                                 const float* amax_b, float denom_a, float denom_b, int64_t M, int64_t N, int64_t Mp,
                                 int64_t Np, int64_t Kp, void* D, int64_t ldd, const void* bias, void* stream) {
  return ll_nvfp4_gemm_tnt_act(A_values, A_scales, B_values, B_scales, alpha, amax_a, amax_b, denom_a, denom_b, M, N,
                               Mp, Np, Kp, D, ldd, bias, LL_ACT_NONE, stream);
}

extern "C" int ll_nvfp4_gemm_tnt_act(const uint8_t* A_values, const uint8_t* A_scales, const uint8_t* B_values,
                                     const uint8_t* B_scales, const float* alpha, const float* amax_a,
                                     const float* amax_b, float denom_a, float denom_b, int64_t M, int64_t N,
                                     int64_t Mp, int64_t Np, int64_t Kp, void* D, int64_t ldd, const void* bias,
                                     int activation, void* stream) {
  ll_gemm_epilogue e = {};
  e.bias = bias;
  e.activation = activation;
  return ll_nvfp4_gemm_tnt_fused(A_values, A_scales, B_values, B_scales, alpha, amax_a, amax_b, denom_a, denom_b, M,
                                 N, Mp, Np, Kp, D, ldd, &e, stream);
}

extern "C" int ll_nvfp4_gemm_tnt_fused(const uint8_t* A_values, const uint8_t* A_scales, const uint8_t* B_values,
                                       const uint8_t* B_scales, const float* alpha, const float* amax_a,
                                       const float* amax_b, float denom_a, float denom_b, int64_t M, int64_t N,
                                       int64_t Mp, int64_t Np, int64_t Kp, void* D, int64_t ldd,
                                       const ll_gemm_epilogue* epilogue, void* stream) {
  using namespace ll;
  LL_REQUIRE(epilogue, "ll_nvfp4_gemm_tnt_fused: null epilogue");
  const int activation = epilogue->activation;
  const void* bias = epilogue->bias;
  LL_REQUIRE(activation == LL_ACT_NONE || activation == LL_ACT_GELU_TANH, "ll_nvfp4_gemm_tnt: unknown activation %d",
             activation);
  GemmEpilogue epi{};
  epi.bias = static_cast<const uint16_t*>(bias);
  epi.act = activation;
  LL_REQUIRE(sink_is_valid(&epilogue->amax_sink), "ll_nvfp4_gemm_tnt_fused: amax sink needs 8-byte alignment and a non-zero epoch");
  epi.sink = make_sink(&epilogue->amax_sink);
  if (epilogue->residual) {
    LL_REQUIRE(N % 8 == 0 && epilogue->ldr % 8 == 0 && epilogue->ldr >= N &&
                   (reinterpret_cast<uintptr_t>(epilogue->residual) & 15) == 0,
               "ll_nvfp4_gemm_tnt_fused: residual needs N %% 8 == 0, ldr %% 8 == 0 and 16-byte alignment");
    epi.residual = static_cast<const uint16_t*>(epilogue->residual);
    epi.ldr = epilogue->ldr;
    if (epilogue->gate) {
      LL_REQUIRE(epilogue->gate_rows > 0 && epilogue->gate_rows < (1ll << 31) && epilogue->gate_stride % 8 == 0 &&
                     (reinterpret_cast<uintptr_t>(epilogue->gate) & 15) == 0,
                 "ll_nvfp4_gemm_tnt_fused: gate needs gate_rows > 0, gate_stride %% 8 == 0 and 16-byte alignment");
      epi.gate = static_cast<const uint16_t*>(epilogue->gate);
      epi.gate_rows = (int)epilogue->gate_rows;
      epi.gate_stride = epilogue->gate_stride;
    }
  } else {
    LL_REQUIRE(!epilogue->gate, "ll_nvfp4_gemm_tnt_fused: a gate needs a residual");
  }
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
  LL_REQUIRE((reinterpret_cast<uintptr_t>(D) & 1) == 0 && (!bias || (reinterpret_cast<uintptr_t>(bias) & 1) == 0),
             "ll_nvfp4_gemm_tnt: D and bias must be 2-byte aligned");
  GemmGroups groups{};
  groups.n = 1;
  return dispatch_gemm(A_values, A_scales, B_values, B_scales, alpha, amax_a, amax_b, denom_a, denom_b, M, N, Mp, Np, Kp,
                       D, ldd, epi, groups, static_cast<hipStream_t>(stream));
}

namespace ll {

inline size_t persistent_record_bytes(const GemmDivision& d) { return (size_t)2 * d.G * kPRecordFloats * sizeof(float); }

// Launches the persistent kernel if the plan says so and its memory is at hand; *launched tells.
static int try_persistent(const uint8_t* A_values, const uint8_t* A_scales, const uint8_t* B_values, const uint8_t* B_scales,
                          const float* alpha, const float* amax_a, const float* amax_b, float denom_a, float denom_b, int64_t M,
                          int64_t N, int64_t Np, int64_t Kp, void* D, int64_t ldd, const GemmEpilogue& epi,
                          const GemmGroups& groups, hipStream_t stream, bool* launched) {
  *launched = false;
  const int schedule = g_gemm_schedule.load(std::memory_order_relaxed);
  if (schedule == LL_GEMM_TILES || schedule == LL_GEMM_TILES_COMPILED || Kp % 128 != 0) return LL_OK;
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    set_error("ll_nvfp4_gemm_tnt: hipGetDevice failed");
    return LL_ELAUNCH;
  }
  if (int rc = compute_units_of(dev, cus, "ll_nvfp4_gemm_tnt")) return rc;
  const PersistentPlan plan = plan_persistent(M, N, Kp, groups.n, cus, schedule);
  if (!plan.use) return LL_OK;
  StreamScratch w;
  bool missing = false;
  if (int rc = stream_scratch(dev, stream, persistent_record_bytes(plan.d), gemm_split_tiles(plan.d), !stream_is_capturing(stream), w, &missing,
                              "ll_nvfp4_gemm_tnt")) return rc;
  if (missing) return LL_OK;  // a capturing stream without the memory: one workgroup per tile, which needs none
  PersistentParams p{};
  p.Av = A_values;
  p.As = A_scales;
  p.amax_a = amax_a;
  p.inv_denom_a = denom_a > 0.f ? 1.0f / denom_a : 0.f;
  p.prod[0] = GemmGroup{B_values, B_scales, alpha, amax_b, denom_b > 0.f ? 1.0f / denom_b : 0.f, static_cast<uint16_t*>(D), ldd,
                        epi.bias, epi.sink};
  for (int i = 1; i < groups.n; ++i) p.prod[i] = groups.more[i - 1];
  p.tiles_n_each = plan.tiles_n_each;
  p.M = (int)M;
  p.N = (int)N;
  p.Np = (int)Np;
  p.Kp = (int)Kp;
  p.tiles_m = plan.tiles_m;
  p.d = plan.d;
  p.epi = epi;
  p.records = reinterpret_cast<float*>(w.records);
  p.arrivals = w.counters;
  static std::atomic<uint64_t> lds_allowed{0};
  if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(&gemm_w4a4_persistent_kernel), kPSmem, lds_allowed, "ll_nvfp4_gemm_tnt")) return rc;
  hipLaunchKernelGGL(gemm_w4a4_persistent_kernel, dim3(plan.d.G), dim3(256), kPSmem, stream, p);
  LL_CHECK_LAUNCH("gemm_w4a4_persistent_kernel");
  *launched = true;
  return LL_OK;
}

// Tile choice and launch; `groups.n` products side by side count as one product of groups.n * N columns.
int dispatch_gemm(const uint8_t* A_values, const uint8_t* A_scales, const uint8_t* B_values, const uint8_t* B_scales,
                  const float* alpha, const float* amax_a, const float* amax_b, float denom_a, float denom_b, int64_t M,
                  int64_t N, int64_t Mp, int64_t Np, int64_t Kp, void* D, int64_t ldd, const GemmEpilogue& epi,
                  const GemmGroups& groups, hipStream_t s) {
  {
    bool launched = false;
    if (int rc = try_persistent(A_values, A_scales, B_values, B_scales, alpha, amax_a, amax_b, denom_a, denom_b, M, N, Np, Kp, D, ldd,
                                epi, groups, s, &launched)) return rc;
    if (launched) return LL_OK;
  }
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    set_error("ll_nvfp4_gemm_tnt: hipGetDevice failed");
    return LL_ELAUNCH;
  }
  if (int rc = compute_units_of(dev, cus, "ll_nvfp4_gemm_tnt")) return rc;
  const TileKernelChoice choice = choose_tile_kernel(M, N, Kp, groups.n, cus, g_gemm_schedule.load(std::memory_order_relaxed));
  if (choice.kernel == LL_GEMM_KERNEL_EIGHT_WAVES) {
    GemmGroups gr = groups;
    gr.tiles_n_each = (int)((N + 255) / 256);
    const int tiles_m = (int)((M + 127) / 128), tiles_n = gr.tiles_n_each * gr.n;
    const int64_t tiles = (int64_t)tiles_m * tiles_n;
    static std::atomic<uint64_t> lds_allowed{0};
    if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(&gemm_w4a4_asm8_kernel), kSplitSmem, lds_allowed, "ll_nvfp4_gemm_tnt")) return rc;
    hipLaunchKernelGGL(gemm_w4a4_asm8_kernel, dim3((unsigned)((tiles + 7) / 8 * 8)), dim3(kSplitThreads), kSplitSmem, s, A_values,
                       A_scales, B_values, B_scales, alpha, amax_a, amax_b, 1.0f / denom_a, 1.0f / denom_b, (int)M, (int)N, (int)Mp,
                       (int)Np, (int)Kp, static_cast<uint16_t*>(D), ldd, tiles_m, tiles_n, epi, gr);
    LL_CHECK_LAUNCH("gemm_w4a4_asm8_kernel");
    return LL_OK;
  }
#define LL_GEMM_ARGS A_values, A_scales, B_values, B_scales, alpha, amax_a, amax_b, denom_a, denom_b, (int)M, (int)N, \
                     (int)Mp, (int)Np, (int)Kp, D, ldd, epi, groups, s, choice.hand_scheduled
  switch (choice.kernel) {
    case LL_GEMM_KERNEL_256X128: return launch_gemm<4, 2>(LL_GEMM_ARGS);
    case LL_GEMM_KERNEL_128X256: return launch_gemm<2, 4>(LL_GEMM_ARGS);
    case LL_GEMM_KERNEL_128X128: return launch_gemm<2, 2>(LL_GEMM_ARGS);
    default: return launch_gemm<1, 1>(LL_GEMM_ARGS);
  }
#undef LL_GEMM_ARGS
}
}  // namespace ll

extern "C" int ll_nvfp4_gemm_tnt_grouped(const uint8_t* A_values, const uint8_t* A_scales, const float* amax_a,
                                         float denom_a, int64_t M, int64_t N, int64_t Mp, int64_t Np, int64_t Kp,
                                         int n_products, const ll_gemm_product* products, void* stream) {
  using namespace ll;
  LL_REQUIRE(products && n_products >= 1 && n_products <= kMaxGemmGroups,
             "ll_nvfp4_gemm_tnt_grouped: 1 to %d products, got %d", kMaxGemmGroups, n_products);
  LL_REQUIRE(A_values && A_scales, "ll_nvfp4_gemm_tnt_grouped: null pointer");
  LL_REQUIRE(M > 0 && N > 0 && Mp % 128 == 0 && Np % 128 == 0 && Kp % 64 == 0 && Kp > 0 && M <= Mp && N <= Np,
             "ll_nvfp4_gemm_tnt_grouped: bad shape M=%lld N=%lld Mp=%lld Np=%lld Kp=%lld", (long long)M, (long long)N,
             (long long)Mp, (long long)Np, (long long)Kp);
  LL_REQUIRE(Mp < (1 << 30) && Np * n_products < (1 << 30) && Kp < (1 << 30), "ll_nvfp4_gemm_tnt_grouped: dimension too large");
  LL_REQUIRE(((reinterpret_cast<uintptr_t>(A_values) | reinterpret_cast<uintptr_t>(A_scales)) & 15) == 0,
             "ll_nvfp4_gemm_tnt_grouped: operands must be 16-byte aligned");
  GemmGroups groups{};
  groups.n = n_products;
  GemmEpilogue epi{};
  for (int i = 0; i < n_products; ++i) {
    const ll_gemm_product& pr = products[i];
    LL_REQUIRE(pr.B_values && pr.B_scales && pr.D && pr.ldd >= N, "ll_nvfp4_gemm_tnt_grouped: product %d: null pointer or ldd < N", i);
    LL_REQUIRE(pr.alpha || (amax_a && pr.amax_b && denom_a > 0.f && pr.denom_b > 0.f),
               "ll_nvfp4_gemm_tnt_grouped: product %d: pass alpha, or both amax pointers with positive denominators", i);
    LL_REQUIRE(((reinterpret_cast<uintptr_t>(pr.B_values) | reinterpret_cast<uintptr_t>(pr.B_scales)) & 15) == 0,
               "ll_nvfp4_gemm_tnt_grouped: product %d: operands must be 16-byte aligned", i);
    LL_REQUIRE((reinterpret_cast<uintptr_t>(pr.D) & 1) == 0 && (!pr.bias || (reinterpret_cast<uintptr_t>(pr.bias) & 1) == 0),
               "ll_nvfp4_gemm_tnt_grouped: product %d: D and bias must be 2-byte aligned", i);
    LL_REQUIRE(sink_is_valid(&pr.amax_sink), "ll_nvfp4_gemm_tnt_grouped: product %d: amax sink needs 8-byte alignment and a non-zero epoch", i);
    if (i == 0) {
      epi.bias = static_cast<const uint16_t*>(pr.bias);
      epi.sink = make_sink(&pr.amax_sink);
    } else {
      GemmGroup& g = groups.more[i - 1];
      g.Bv = pr.B_values;
      g.Bs = pr.B_scales;
      g.alpha = pr.alpha;
      g.amax_b = pr.amax_b;
      g.inv_denom_b = pr.denom_b > 0.f ? 1.0f / pr.denom_b : 0.f;
      g.D = static_cast<uint16_t*>(pr.D);
      g.ldd = pr.ldd;
      g.bias = static_cast<const uint16_t*>(pr.bias);
      g.sink = make_sink(&pr.amax_sink);
    }
  }
  const ll_gemm_product& p0 = products[0];
  return dispatch_gemm(A_values, A_scales, p0.B_values, p0.B_scales, p0.alpha, amax_a, p0.amax_b, denom_a,
                       p0.denom_b > 0.f ? p0.denom_b : 1.f, M, N, Mp, Np, Kp, p0.D, p0.ldd, epi, groups,
                       static_cast<hipStream_t>(stream));
}

extern "C" int ll_nvfp4_gemm_set_schedule(int schedule) {
  LL_REQUIRE(schedule >= LL_GEMM_AUTO && schedule <= LL_GEMM_TILES_COMPILED, "ll_nvfp4_gemm_set_schedule: unknown schedule %d", schedule);
  ll::g_gemm_schedule.store(schedule);
  return LL_OK;
}

extern "C" int ll_nvfp4_gemm_get_schedule(void) { return ll::g_gemm_schedule.load(); }

extern "C" int ll_nvfp4_gemm_plan(int64_t M, int64_t N, int64_t Kp, int n_products, int compute_units, int schedule,
                                  int* persistent, uint32_t* workgroups, uint32_t* tiles, uint32_t* k_steps) {
  LL_REQUIRE(M > 0 && N > 0 && Kp > 0 && Kp % 64 == 0 && n_products >= 1 && n_products <= ll::kMaxGemmGroups && compute_units > 0 &&
                 M < (1 << 30) && N < (1 << 30) && Kp < (1 << 30),
             "ll_nvfp4_gemm_plan: bad sizes");
  LL_REQUIRE(schedule >= LL_GEMM_AUTO && schedule <= LL_GEMM_TILES_COMPILED, "ll_nvfp4_gemm_plan: unknown schedule %d", schedule);
  const ll::PersistentPlan plan = ll::plan_persistent(M, N, Kp, n_products, compute_units, schedule);
  if (persistent) *persistent = plan.use ? 1 : 0;
  if (workgroups) *workgroups = plan.d.G;
  if (tiles) *tiles = plan.d.tiles;
  if (k_steps) *k_steps = plan.d.nk;
  return LL_OK;
}

extern "C" int ll_nvfp4_gemm_kernel(int64_t M, int64_t N, int64_t Kp, int n_products, int compute_units, int schedule,
                                    int* kernel, int* hand_scheduled) {
  LL_REQUIRE(M > 0 && N > 0 && Kp > 0 && Kp % 64 == 0 && n_products >= 1 && n_products <= ll::kMaxGemmGroups && compute_units > 0 &&
                 M < (1 << 30) && N < (1 << 30) && Kp < (1 << 30),
             "ll_nvfp4_gemm_kernel: bad sizes");
  LL_REQUIRE(schedule >= LL_GEMM_AUTO && schedule <= LL_GEMM_TILES_COMPILED, "ll_nvfp4_gemm_kernel: unknown schedule %d", schedule);
  if (ll::plan_persistent(M, N, Kp, n_products, compute_units, schedule).use) {
    if (kernel) *kernel = LL_GEMM_KERNEL_PERSISTENT;
    if (hand_scheduled) *hand_scheduled = 1;
    return LL_OK;
  }
  const ll::TileKernelChoice c = ll::choose_tile_kernel(M, N, Kp, n_products, compute_units, schedule);
  if (kernel) *kernel = c.kernel;
  if (hand_scheduled) *hand_scheduled = c.hand_scheduled ? 1 : 0;
  return LL_OK;
}

extern "C" int ll_nvfp4_gemm_reserve(int64_t M, int64_t N, int64_t Kp, int n_products, void* stream) {
  using namespace ll;
  LL_REQUIRE(M > 0 && N > 0 && Kp > 0 && Kp % 64 == 0 && n_products >= 1 && n_products <= kMaxGemmGroups && M < (1 << 30) &&
                 N < (1 << 30) && Kp < (1 << 30),
             "ll_nvfp4_gemm_reserve: bad sizes");
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    set_error("ll_nvfp4_gemm_reserve: hipGetDevice failed");
    return LL_ELAUNCH;
  }
  if (int rc = compute_units_of(dev, cus, "ll_nvfp4_gemm_reserve")) return rc;
  const PersistentPlan plan = plan_persistent(M, N, Kp, n_products, cus, g_gemm_schedule.load(std::memory_order_relaxed));
  if (!plan.use) return LL_OK;
  if (stream_is_capturing(static_cast<hipStream_t>(stream))) {
    set_error("ll_nvfp4_gemm_reserve: the stream is being captured; reserve before the recording starts");
    return LL_ENOSUP;
  }
  StreamScratch w;
  return stream_scratch(dev, static_cast<hipStream_t>(stream), persistent_record_bytes(plan.d), gemm_split_tiles(plan.d), true, w, nullptr,
                        "ll_nvfp4_gemm_reserve");
}
