// Normalization and NVFP4 quantization of the result in one launch for gfx950: the adaLN modulation
// (utils/adaln_triton.py:36-86) or the affine LayerNorm (wan_5b/modules/model.py:101-111) of the DiT block,
// followed by the activation quantization of the linear layer that reads the result
// (fouroversix/src/fouroversix/quantize/pytorch/reference.py:121-368).  The normalized tensor itself is never
// written: its rows stay in registers between the two halves of the kernel, and only packed values, block scales
// and the tensor amax leave.  The bytes are those of the separate operations (same row arithmetic, same block
// arithmetic).
//
// The block scales depend on the maximum of the whole tensor, so every workgroup has to see every other
// workgroup's maximum before it can quantize: all workgroups of the launch are resident at once (the host sizes
// the grid to what the device holds), each publishes its maximum into its own slot of the caller's amax sink
// under the launch's epoch, and each waits until all slots carry that epoch.  The wait is bounded: a workgroup that
// has not seen every slot after `spin_limit` looks computes the maxima of the missing workgroups' rows itself,
// which gives the same number, so the kernel finishes whatever the other workgroups do (amax_exchange.h).
#include "ll_common.h"
#include "amax_exchange.h"
#include "norm_rows.h"
#include "quantize_block.h"

#pragma clang fp contract(off)

namespace ll {

constexpr int kNqThreads = 256;
constexpr int kNqChunks = 6;  // 16-byte groups per lane: rows of up to 64 * 6 * 8 = 3072 elements
constexpr int kNqMaxRowLength = 64 * kNqChunks * 8;
constexpr int kNqAdaln = 0, kNqLayerNorm = 1;

struct NormQuantParams {
  const uint16_t* x;
  int64_t M, Mp, L;
  int C;
  const uint16_t* a;  // adaLN: scale rows; LayerNorm: weight or null
  const uint16_t* b;  // adaLN: shift rows; LayerNorm: bias or null
  int64_t a_sb, a_sf, b_sb, b_sf, frame_seqlen;
  float eps;
  int add_one;
  uint8_t* values;
  uint8_t* scales;
  float* amax_out;
  AmaxSink sink;
  uint32_t spin_limit;
  int recompute;  // every workgroup takes the bounded wait's way out (tests)
};

template <int MODE>
__device__ __forceinline__ float norm_row(const NormQuantParams& p, int64_t row, int lane, uint4 (&packed)[kNqChunks]) {
  const uint16_t* xr = p.x + row * (int64_t)p.C;
  if (MODE == kNqAdaln) {
    const int64_t b = row / p.L, l = row - b * p.L, f = l / p.frame_seqlen;
    return adaln_row<kNqChunks>(xr, p.a + b * p.a_sb + f * p.a_sf, p.b + b * p.b_sb + f * p.b_sf, p.C, p.eps, p.add_one,
                                lane, packed);
  }
  return layernorm_row<kNqChunks>(xr, p.a, p.b, p.C, p.eps, lane, packed);
}

// The value of the neighbouring lane (lane ^ 1): quad_perm [1, 0, 3, 2].
__device__ __forceinline__ uint32_t from_pair_lane(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, false);
}

// One workgroup = four waves, one wave = one row at a time, R rows per wave over the launch: row
// (r * gridDim.x + blockIdx.x) * 4 + wave.  Rows [M, Mp) are the zero padding of the quantized operand.
// Only R = 1 is launched (see launch_rule).
template <int RULE, int MODE, int R>
__global__ __launch_bounds__(kNqThreads) __attribute__((amdgpu_waves_per_eu(R == 1 ? 3 : 2)))
void norm_quantize_kernel(NormQuantParams p) {
  __shared__ AmaxExchangeSmem s_exchange;
  __shared__ ScaleEntry s_tab[128];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t G = gridDim.x;

  // ---- first half: the rows, kept as packed bf16, and their maximum
  uint4 kept[R][kNqChunks];
  float wave_part = 0.0f;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int64_t row = ((int64_t)r * G + blockIdx.x) * 4 + wave;
    if (row < p.M) {
      wave_part = fmaxf(wave_part, norm_row<MODE>(p, row, lane, kept[r]));
    } else {
#pragma unroll
      for (int i = 0; i < kNqChunks; ++i) kept[r][i] = make_uint4(0u, 0u, 0u, 0u);
    }
  }
  // ---- the maximum of the whole tensor: exchanged with the other workgroups through the sink; a missing
  // workgroup's rows are normalized here, wave w taking the row its wave w has
  const float amax = exchange_amax(p.sink, G, blockIdx.x, wave_part, p.spin_limit, p.recompute != 0, s_exchange, [&](uint32_t s) {
    float part = 0.0f;
#pragma unroll 1
    for (int r = 0; r < R; ++r) {
      const int64_t row = ((int64_t)r * G + s) * 4 + wave;
      if (row < p.M) {
        uint4 unused[kNqChunks];
        part = fmaxf(part, norm_row<MODE>(p, row, lane, unused));
      }
    }
    return part;
  });
  if (blockIdx.x == 0 && threadIdx.x == 0) p.amax_out[0] = amax;

  // ---- second half: quantize the kept rows (same constants and paths as quantize_kernel)
  constexpr bool kStaticRule = (RULE == LL_RULE_STATIC_6 || RULE == LL_RULE_STATIC_4);
  constexpr float kE2 = (RULE == LL_RULE_STATIC_4) ? 4.0f : 6.0f;
  constexpr float kE4 = kStaticRule ? 448.0f : 256.0f;
  const bool fast = amax >= 0x1p-100f && amax <= 0x1p100f;
  const bool approx_ok = amax >= 0x1p-30f && amax <= 0x1p30f;
  const float enc = (kE2 * kE4) / amax;
  const float dec = 1.0f / enc;
  if (fast) fill_scale_table<RULE>(s_tab, amax, dec);
  __syncthreads();

  // A block of 16 is two neighbouring groups of 8, which lie in the lanes 2p and 2p + 1 (same i).  The even lane
  // quantizes the blocks of i = 0, 2, 4, the odd lane those of i = 1, 3, 5; each receives the missing half from
  // its neighbour.
  const int nchunks = p.C >> 3;
  const int64_t vrow = p.C >> 1;           // bytes per row of packed values
  const uint32_t tiles_x = (uint32_t)(p.C >> 6);
  const bool odd = (lane & 1) != 0;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int64_t row = ((int64_t)r * G + blockIdx.x) * 4 + wave;
    if (row >= p.Mp) continue;  // uniform over the wave
    uint8_t* vdst = p.values + row * vrow;
    uint8_t* sdst = p.scales + (row >> 7) * (int64_t)tiles_x * 512 + (row & 31) * 16 + ((row >> 5) & 3) * 4;
#pragma unroll
    for (int k = 0; k < kNqChunks / 2; ++k) {
      const uint4 even_piece = kept[r][2 * k], odd_piece = kept[r][2 * k + 1];
      const uint4 send = odd ? even_piece : odd_piece;
      uint4 recv;
      recv.x = from_pair_lane(send.x);
      recv.y = from_pair_lane(send.y);
      recv.z = from_pair_lane(send.z);
      recv.w = from_pair_lane(send.w);
      const uint4 lo4 = odd ? recv : even_piece, hi4 = odd ? odd_piece : recv;
      const int c = lane + 64 * (2 * k + (odd ? 1 : 0));  // this lane's own group of the block
      if (c >= nchunks) continue;
      const int blk = c >> 1;
      const uint32_t w[8] = {lo4.x, lo4.y, lo4.z, lo4.w, hi4.x, hi4.y, hi4.z, hi4.w};
      float X[16];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        X[2 * i] = __uint_as_float(w[i] << 16);
        X[2 * i + 1] = __uint_as_float(w[i] & 0xFFFF0000u);
      }
      uint32_t lo, hi, sb;
      if (!fast || !quantize_block_fast<RULE>(X, enc, s_tab, approx_ok, __builtin_inff(), lo, hi, sb))
        quantize_block<RULE>(X, amax, enc, dec, lo, hi, sb);
      *reinterpret_cast<uint2*>(vdst + blk * 8) = make_uint2(lo, hi);
      sdst[(int64_t)(blk >> 2) * 512 + (blk & 3)] = (uint8_t)sb;
    }
  }
}

// Workgroups of norm_quantize_kernel<rule, mode, R> that the current device holds at once.
template <int RULE, int MODE, int R>
static int resident_of(int* out) {
  static std::atomic<int> cache[64];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    set_error("norm_quantize: hipGetDevice failed: %s", hipGetErrorString(e));
    return LL_ELAUNCH;
  }
  std::atomic<int>* slot = (dev >= 0 && dev < 64) ? &cache[dev] : nullptr;
  int n = slot ? slot->load(std::memory_order_relaxed) : 0;
  if (n == 0) {
    int per_cu = 0, cus = 0;
    e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, norm_quantize_kernel<RULE, MODE, R>, kNqThreads, 0);
    if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess || per_cu <= 0 || cus <= 0) {
      set_error("norm_quantize: occupancy query failed: %s", hipGetErrorString(e));
      return LL_ELAUNCH;
    }
    n = per_cu * cus;
    if (slot) slot->store(n, std::memory_order_relaxed);
  }
  *out = n;
  return LL_OK;
}

template <int RULE, int MODE, int R>
static int launch_with(NormQuantParams& p, hipStream_t stream, bool* fits) {
  int resident = 0;
  if (int rc = resident_of<RULE, MODE, R>(&resident)) return rc;
  const int64_t groups = p.Mp / 4;  // Mp is a multiple of 128
  int64_t grid = resident < kAmaxParts ? resident : kAmaxParts;
  if (grid > groups) grid = groups;
  *fits = grid * R >= groups;
  if (!*fits) return LL_OK;
  hipLaunchKernelGGL((norm_quantize_kernel<RULE, MODE, R>), dim3((unsigned)grid), dim3(kNqThreads), 0, stream, p);
  return LL_OK;
}

template <int RULE, int MODE>
static int launch_rule(NormQuantParams& p, hipStream_t stream, bool* fits) {
  // One row per wave, three waves per SIMD.  Variants that keep two or four rows per wave (and so take more rows
  // than the device holds waves) were measured: at 7040 rows the kernel then takes as long as the two separate
  // kernels (36 us), at two waves per SIMD, so those shapes are left to the separate operations.
  return launch_with<RULE, MODE, 1>(p, stream, fits);
}

template <int MODE>
static int launch_mode(NormQuantParams& p, int rule, hipStream_t stream, bool* fits) {
  switch (rule) {
    case LL_RULE_STATIC_6: return launch_rule<LL_RULE_STATIC_6, MODE>(p, stream, fits);
    case LL_RULE_STATIC_4: return launch_rule<LL_RULE_STATIC_4, MODE>(p, stream, fits);
    case LL_RULE_MAE: return launch_rule<LL_RULE_MAE, MODE>(p, stream, fits);
    case LL_RULE_MSE: return launch_rule<LL_RULE_MSE, MODE>(p, stream, fits);
    default: return launch_rule<LL_RULE_ABS_MAX, MODE>(p, stream, fits);
  }
}

static int norm_quantize(NormQuantParams& p, int mode, int rule, const ll_amax_sink* sink, int64_t spin_limit,
                         void* stream, const char* what) {
  LL_REQUIRE(p.x && p.values && p.scales && p.amax_out, "%s: null pointer", what);
  LL_REQUIRE(rule >= 0 && rule <= 4, "%s: unknown scale rule %d", what, rule);
  LL_REQUIRE(sink && sink->parts && sink_is_valid(sink),
             "%s: an amax sink (8-byte aligned buffer, non-zero epoch) is required: the workgroups exchange their "
             "maxima through it", what);
  LL_REQUIRE(p.M > 0 && p.M <= 0x7FFFFFFF, "%s: bad row count %lld", what, (long long)p.M);
  LL_REQUIRE(((reinterpret_cast<uintptr_t>(p.x) | reinterpret_cast<uintptr_t>(p.a) | reinterpret_cast<uintptr_t>(p.b)) & 15) == 0 &&
                 (reinterpret_cast<uintptr_t>(p.values) & 7) == 0 && (reinterpret_cast<uintptr_t>(p.amax_out) & 3) == 0,
             "%s: inputs must be 16-byte aligned, packed values 8-byte aligned", what);
  if (p.C <= 0 || p.C % 64 != 0 || p.C > kNqMaxRowLength) {
    set_error("%s: rows of %d elements are not supported in one launch (a multiple of 64 up to %d): use the separate "
              "operations", what, p.C, kNqMaxRowLength);
    return LL_ENOSUP;
  }
  p.Mp = round_up(p.M, 128);
  p.sink = make_sink(sink);
  p.spin_limit = spin_limit < 0 ? 0u : (spin_limit > 0x7FFFFFFF ? 0x7FFFFFFFu : (uint32_t)spin_limit);
  p.recompute = spin_limit < 0 ? 1 : 0;
  bool fits = false;
  const int rc = mode == kNqAdaln ? launch_mode<kNqAdaln>(p, rule, static_cast<hipStream_t>(stream), &fits)
                                  : launch_mode<kNqLayerNorm>(p, rule, static_cast<hipStream_t>(stream), &fits);
  if (rc) return rc;
  if (!fits) {
    set_error("%s: %lld rows are more than the device holds at once in this kernel: use the separate operations", what,
              (long long)p.M);
    return LL_ENOSUP;
  }
  LL_CHECK_LAUNCH("norm_quantize_kernel");
  return LL_OK;
}

}  // namespace ll

extern "C" int ll_adaln_quantize(const void* x, int64_t B, int64_t L, int C, const void* scale, const void* shift,
                                 int64_t scale_stride_b, int64_t scale_stride_f, int64_t shift_stride_b,
                                 int64_t shift_stride_f, int64_t frame_seqlen, float eps, int add_one_to_scale, int rule,
                                 uint8_t* values, uint8_t* scales, float* amax, const ll_amax_sink* amax_sink,
                                 int64_t spin_limit, void* stream) {
  using namespace ll;
  LL_REQUIRE(scale && shift, "ll_adaln_quantize: null pointer");
  LL_REQUIRE(B > 0 && L > 0 && frame_seqlen > 0 && L % frame_seqlen == 0 && B * L <= 0x7FFFFFFF,
             "ll_adaln_quantize: bad shape B=%lld L=%lld frame_seqlen=%lld", (long long)B, (long long)L,
             (long long)frame_seqlen);
  LL_REQUIRE(scale_stride_b % 8 == 0 && scale_stride_f % 8 == 0 && shift_stride_b % 8 == 0 && shift_stride_f % 8 == 0,
             "ll_adaln_quantize: strides must be multiples of 8 elements");
  NormQuantParams p{};
  p.x = static_cast<const uint16_t*>(x);
  p.M = B * L;
  p.L = L;
  p.C = C;
  p.a = static_cast<const uint16_t*>(scale);
  p.b = static_cast<const uint16_t*>(shift);
  p.a_sb = scale_stride_b;
  p.a_sf = scale_stride_f;
  p.b_sb = shift_stride_b;
  p.b_sf = shift_stride_f;
  p.frame_seqlen = frame_seqlen;
  p.eps = eps;
  p.add_one = add_one_to_scale;
  p.values = values;
  p.scales = scales;
  p.amax_out = amax;
  return norm_quantize(p, kNqAdaln, rule, amax_sink, spin_limit, stream, "ll_adaln_quantize");
}

extern "C" int ll_layer_norm_quantize(const void* x, int64_t rows, int C, const void* weight, const void* bias,
                                      float eps, int rule, uint8_t* values, uint8_t* scales, float* amax,
                                      const ll_amax_sink* amax_sink, int64_t spin_limit, void* stream) {
  using namespace ll;
  NormQuantParams p{};
  p.x = static_cast<const uint16_t*>(x);
  p.M = rows;
  p.L = rows > 0 ? rows : 1;
  p.C = C;
  p.a = static_cast<const uint16_t*>(weight);
  p.b = static_cast<const uint16_t*>(bias);
  p.frame_seqlen = 1;
  p.eps = eps;
  p.values = values;
  p.scales = scales;
  p.amax_out = amax;
  return norm_quantize(p, kNqLayerNorm, rule, amax_sink, spin_limit, stream, "ll_layer_norm_quantize");
}
