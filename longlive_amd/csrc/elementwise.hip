// Memory-bound fused kernels of the DiT block for gfx950: 3-D RoPE apply, adaLN modulate, RMSNorm.
// All of them read bf16 with 128-bit loads, compute in fp32 and round where the reference rounds.
#include "ll_common.h"
#include "norm_rows.h"

#pragma clang fp contract(off)

namespace ll {

// ----------------------------------------------------------------------------- RoPE
// utils/rope_triton.py:36-81.  One thread = 8 consecutive elements (4 rotation pairs) of one (token, head).
__global__ __launch_bounds__(256) void rope_kernel(const uint16_t* __restrict__ x, int64_t S, int N, int D,
                                                   int64_t xs, int64_t xn, const float* __restrict__ cosp,
                                                   const float* __restrict__ sinp, int64_t seq_len,
                                                   uint16_t* __restrict__ out) {
  const int gpr = D >> 3;  // groups per (token, head)
  const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t total = S * N * gpr;
  if (g >= total) return;
  const int64_t s = g / ((int64_t)N * gpr);
  const int rem = (int)(g - s * (int64_t)N * gpr);
  const int n = rem / gpr, c = (rem - n * gpr) * 8;
  const uint4 v = *reinterpret_cast<const uint4*>(x + s * xs + (int64_t)n * xn + c);
  uint4 o = v;
  if (s < seq_len) {
    float f[8], r[8];
    unpack8(v, f);
    const float4 cs = *reinterpret_cast<const float4*>(cosp + s * (D >> 1) + (c >> 1));
    const float4 sn = *reinterpret_cast<const float4*>(sinp + s * (D >> 1) + (c >> 1));
    const float cc[4] = {cs.x, cs.y, cs.z, cs.w}, ss[4] = {sn.x, sn.y, sn.z, sn.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float a = f[2 * i], b = f[2 * i + 1];
      r[2 * i] = a * cc[i] - b * ss[i];
      r[2 * i + 1] = a * ss[i] + b * cc[i];
    }
    o = pack8(r);
  }
  *reinterpret_cast<uint4*>(out + (s * N + n) * (int64_t)D + c) = o;
}

// ----------------------------------------------------------------------------- adaLN
// utils/adaln_triton.py:36-86.  One workgroup = one token row.
template <int NCH>
__global__ __launch_bounds__(kRowThreads) void adaln_kernel(const uint16_t* __restrict__ x, int64_t rows, int64_t L, int C,
                                                            const uint16_t* __restrict__ scale,
                                                            const uint16_t* __restrict__ shift, int64_t sc_sb,
                                                            int64_t sc_sf, int64_t sh_sb, int64_t sh_sf,
                                                            int64_t frame_seqlen, float eps, int add_one,
                                                            uint16_t* __restrict__ out, AmaxSink sink) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * kRowsPerWg + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int64_t b = row / L, l = row - b * L, f = l / frame_seqlen;
  uint4 packed[NCH];
  float out_max = adaln_row<NCH>(x + row * (int64_t)C, scale + b * sc_sb + f * sc_sf, shift + b * sh_sb + f * sh_sf, C, eps,
                                 add_one, lane, packed);
  uint16_t* orow = out + row * (int64_t)C;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = lane + i * 64;
    if (c < (C >> 3)) *reinterpret_cast<uint4*>(orow + c * 8) = packed[i];
  }
  if (sink.parts) {
    out_max = wave_max(out_max);
    if (lane == 0) amax_sink_update(sink, (uint32_t)row, out_max);
  }
}

// ----------------------------------------------------------------------------- LayerNorm with weight and bias
// wan_5b/modules/model.py:101-111 (nn.LayerNorm on bf16 tensors: statistics and the affine map in fp32, one
// rounding to bf16 at the end).  One wave = one row.
template <int NCH>
__global__ __launch_bounds__(kRowThreads) void layernorm_kernel(const uint16_t* __restrict__ x, int64_t rows, int C,
                                                                const uint16_t* __restrict__ w,
                                                                const uint16_t* __restrict__ b, float eps,
                                                                uint16_t* __restrict__ out, AmaxSink sink) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * kRowsPerWg + (threadIdx.x >> 6);
  if (row >= rows) return;
  uint4 packed[NCH];
  float out_max = layernorm_row<NCH>(x + row * (int64_t)C, w, b, C, eps, lane, packed);
  uint16_t* orow = out + row * (int64_t)C;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = lane + i * 64;
    if (c < (C >> 3)) *reinterpret_cast<uint4*>(orow + c * 8) = packed[i];
  }
  if (sink.parts) {
    out_max = wave_max(out_max);
    if (lane == 0) amax_sink_update(sink, (uint32_t)row, out_max);
  }
}

// ----------------------------------------------------------------------------- RMSNorm
// wan_5b/modules/model.py:82-98.
template <int NCH>
__global__ __launch_bounds__(kRowThreads) void rmsnorm_kernel(const uint16_t* __restrict__ x, int64_t rows, int C,
                                                              const uint16_t* __restrict__ w, float eps,
                                                              uint16_t* __restrict__ out) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * kRowsPerWg + (threadIdx.x >> 6);
  if (row >= rows) return;
  const uint16_t* xr = x + row * (int64_t)C;
  const int nchunks = C >> 3;
  float v[NCH][8];
  float sq = 0.0f;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = lane + i * 64;
    if (c < nchunks) {
      unpack8(*reinterpret_cast<const uint4*>(xr + c * 8), v[i]);
#pragma unroll
      for (int j = 0; j < 8; ++j) sq += v[i][j] * v[i][j];
    }
  }
  const float ms = wave_sum_dpp(sq) / (float)C;
  const float r = 1.0f / sqrtf(ms + eps);
  uint16_t* orow = out + row * (int64_t)C;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = lane + i * 64;
    if (c < nchunks) {
      float w8[8], y[8];
      unpack8(*reinterpret_cast<const uint4*>(w + c * 8), w8);
#pragma unroll
      for (int j = 0; j < 8; ++j) y[j] = round_to_bf16(v[i][j] * r) * w8[j];
      *reinterpret_cast<uint4*>(orow + c * 8) = pack8(y);
    }
  }
}


// ----------------------------------------------------------------------------- RMSNorm + RoPE (+ K smoothing)
// q / k path after the projections (wan_5b/modules/causal_model.py:362-368, 477-487): WanRMSNorm over the
// whole row, then the 3-D rotary embedding per head of 128, each with the roundings of the separate kernels
// above; optionally also k - mean(k over the head dimension) (utils/quant.py:797-798) as a second output,
// mean and difference rounded to bf16 like the two eager operations.  One wave = one token row; a head is
// held by 16 consecutive lanes.  blockIdx.y selects the tensor (q or k), so that both go in one launch.
struct QkProblem {  // one tensor of the q / k pair
  const uint16_t* x;
  const uint16_t* w;
  uint16_t* out;
  uint16_t* out_smooth;  // or null
  AmaxSink sink;         // receives max |out| when sink.parts is not null
};
struct QkProblems {
  QkProblem p[2];
};

template <int NCH>
__global__ __launch_bounds__(kRowThreads) void qk_norm_rope_kernel(QkProblems problems, int64_t rows, int C, float eps,
                                                                   const float* __restrict__ cosp,
                                                                   const float* __restrict__ sinp, int64_t seq_len) {
  const QkProblem& pr = problems.p[blockIdx.y];
  const uint16_t* __restrict__ x = pr.x;
  const uint16_t* __restrict__ w = pr.w;
  uint16_t* __restrict__ out = pr.out;
  uint16_t* __restrict__ out_smooth = pr.out_smooth;
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * kRowsPerWg + (threadIdx.x >> 6);
  if (row >= rows) return;
  const uint16_t* xr = x + row * (int64_t)C;
  const int nchunks = C >> 3;
  float v[NCH][8];
  float sq = 0.0f;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = lane + i * 64;
    if (c < nchunks) {
      unpack8(*reinterpret_cast<const uint4*>(xr + c * 8), v[i]);
#pragma unroll
      for (int j = 0; j < 8; ++j) sq += v[i][j] * v[i][j];
    }
  }
  const float ms = wave_sum_dpp(sq) / (float)C;
  const float r = 1.0f / sqrtf(ms + eps);
  const bool rotate = row < seq_len;
  float out_max = 0.0f;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = lane + i * 64;  // uniform over each group of 16 threads: c < nchunks or not
    if (c < nchunks) {
      float w8[8], y[8], o8[8];
      unpack8(*reinterpret_cast<const uint4*>(w + c * 8), w8);
#pragma unroll
      for (int j = 0; j < 8; ++j) y[j] = round_to_bf16(round_to_bf16(v[i][j] * r) * w8[j]);
      if (rotate) {
        const int pair0 = (c & 15) * 4;  // first rotation pair of this chunk inside its head
        const float4 cs = *reinterpret_cast<const float4*>(cosp + row * 64 + pair0);
        const float4 sn = *reinterpret_cast<const float4*>(sinp + row * 64 + pair0);
        const float cc[4] = {cs.x, cs.y, cs.z, cs.w}, ss[4] = {sn.x, sn.y, sn.z, sn.w};
#pragma unroll
        for (int p = 0; p < 4; ++p) {
          const float a = y[2 * p], b = y[2 * p + 1];
          o8[2 * p] = round_to_bf16(a * cc[p] - b * ss[p]);
          o8[2 * p + 1] = round_to_bf16(a * ss[p] + b * cc[p]);
        }
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) o8[j] = y[j];
      }
      const uint4 packed = pack8(o8);
      *reinterpret_cast<uint4*>(out + row * (int64_t)C + c * 8) = packed;
      out_max = abs_max_bf16x8(packed, out_max);
      if (out_smooth) {
        float part = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) part += o8[j];
#pragma unroll
        for (int m = 1; m < 16; m <<= 1) part += __shfl_xor(part, m, 64);
        const float mean = round_to_bf16(part * (1.0f / 128.0f));
        float s8[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) s8[j] = o8[j] - mean;
        *reinterpret_cast<uint4*>(out_smooth + row * (int64_t)C + c * 8) = pack8(s8);
      }
    }
  }
  if (pr.sink.parts) {
    out_max = wave_max(out_max);
    if (lane == 0) amax_sink_update(pr.sink, (uint32_t)row, out_max);
  }
}

// ----------------------------------------------------------------------------- gated residual
// x + y * gate of the DiT block (wan_5b/modules/causal_model.py:889, 919-920): the product is rounded to
// bf16, then the sum, as the two separate bf16 operations of the reference do.  gate is indexed
// [b, l / frame_seqlen, :].  One thread = 8 consecutive channels.
__global__ __launch_bounds__(256) void gate_residual_kernel(const uint16_t* __restrict__ x,
                                                           const uint16_t* __restrict__ y,
                                                           const uint16_t* __restrict__ gate, int64_t L, int C,
                                                           int64_t g_sb, int64_t g_sf, int64_t frame_seqlen,
                                                           int64_t total_chunks, uint16_t* __restrict__ out) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total_chunks) return;
  const int cpr = C >> 3;  // chunks per row
  const int64_t row = idx / cpr;
  const int c = (int)(idx - row * cpr);
  const int64_t b = row / L, l = row - b * L, f = l / frame_seqlen;
  float xv[8], yv[8], gv[8];
  unpack8(*reinterpret_cast<const uint4*>(x + row * (int64_t)C + c * 8), xv);
  unpack8(*reinterpret_cast<const uint4*>(y + row * (int64_t)C + c * 8), yv);
  unpack8(*reinterpret_cast<const uint4*>(gate + b * g_sb + f * g_sf + c * 8), gv);
  float r[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) r[j] = xv[j] + round_to_bf16(yv[j] * gv[j]);
  *reinterpret_cast<uint4*>(out + row * (int64_t)C + c * 8) = pack8(r);
}

}  // namespace ll

extern "C" int ll_rope_apply(const void* x, int64_t S, int N, int D, int64_t x_stride_s, int64_t x_stride_n,
                             const float* cos, const float* sin, int64_t seq_len, void* out, void* stream) {
  using namespace ll;
  LL_REQUIRE(x && cos && sin && out, "ll_rope_apply: null pointer");
  LL_REQUIRE(S > 0 && N > 0 && D > 0 && D % 16 == 0 && seq_len >= 0 && seq_len <= S,
             "ll_rope_apply: bad shape S=%lld N=%d D=%d seq_len=%lld (D must be a multiple of 16)", (long long)S, N, D,
             (long long)seq_len);
  LL_REQUIRE(x_stride_s % 8 == 0 && x_stride_n % 8 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 &&
                 (reinterpret_cast<uintptr_t>(out) & 15) == 0 && (reinterpret_cast<uintptr_t>(cos) & 15) == 0 &&
                 (reinterpret_cast<uintptr_t>(sin) & 15) == 0,
             "ll_rope_apply: pointers must be 16-byte aligned and strides multiples of 8 elements");
  const int64_t groups = S * N * (D / 8);
  hipLaunchKernelGGL(rope_kernel, dim3((unsigned)((groups + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<const uint16_t*>(x), S, N, D, x_stride_s,
                     x_stride_n, cos, sin, seq_len, static_cast<uint16_t*>(out));
  LL_CHECK_LAUNCH("rope_kernel");
  return LL_OK;
}

extern "C" int ll_adaln_modulate(const void* x, int64_t B, int64_t L, int C, const void* scale, const void* shift,
                                 int64_t scale_stride_b, int64_t scale_stride_f, int64_t shift_stride_b,
                                 int64_t shift_stride_f, int64_t frame_seqlen, float eps, int add_one_to_scale,
                                 void* out, void* stream) {
  return ll_adaln_modulate_amax(x, B, L, C, scale, shift, scale_stride_b, scale_stride_f, shift_stride_b,
                                shift_stride_f, frame_seqlen, eps, add_one_to_scale, out, nullptr, stream);
}

extern "C" int ll_adaln_modulate_amax(const void* x, int64_t B, int64_t L, int C, const void* scale,
                                      const void* shift, int64_t scale_stride_b, int64_t scale_stride_f,
                                      int64_t shift_stride_b, int64_t shift_stride_f, int64_t frame_seqlen, float eps,
                                      int add_one_to_scale, void* out, const ll_amax_sink* amax_sink, void* stream) {
  using namespace ll;
  LL_REQUIRE(sink_is_valid(amax_sink), "ll_adaln_modulate_amax: amax sink needs 8-byte alignment and a non-zero epoch");
  const AmaxSink sink = make_sink(amax_sink);
  LL_REQUIRE(x && scale && shift && out, "ll_adaln_modulate: null pointer");
  LL_REQUIRE(B > 0 && L > 0 && C > 0 && C % 8 == 0 && C <= kMaxRowLength && frame_seqlen > 0 &&
                 L % frame_seqlen == 0,
             "ll_adaln_modulate: bad shape B=%lld L=%lld C=%d frame_seqlen=%lld (C %% 8 == 0, C <= %d)", (long long)B,
             (long long)L, C, (long long)frame_seqlen, kMaxRowLength);
  LL_REQUIRE(scale_stride_b % 8 == 0 && scale_stride_f % 8 == 0 && shift_stride_b % 8 == 0 && shift_stride_f % 8 == 0 &&
                 ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(scale) |
                   reinterpret_cast<uintptr_t>(shift) | reinterpret_cast<uintptr_t>(out)) & 15) == 0,
             "ll_adaln_modulate: pointers must be 16-byte aligned and strides multiples of 8 elements");
  LL_REQUIRE(B * L <= 0x7FFFFFFF, "ll_adaln_modulate: too many rows");
  const dim3 grid((unsigned)((B * L + kRowsPerWg - 1) / kRowsPerWg));
#define LL_LAUNCH_ADALN(NCH)                                                                                    \
  hipLaunchKernelGGL(adaln_kernel<NCH>, grid, dim3(kRowThreads), 0, static_cast<hipStream_t>(stream),           \
                     static_cast<const uint16_t*>(x), B * L, L, C, static_cast<const uint16_t*>(scale),         \
                     static_cast<const uint16_t*>(shift), scale_stride_b, scale_stride_f, shift_stride_b,       \
                     shift_stride_f, frame_seqlen, eps, add_one_to_scale, static_cast<uint16_t*>(out), sink)
  if (C <= 64 * 6 * 8) {
    LL_LAUNCH_ADALN(6);
  } else {
    LL_LAUNCH_ADALN(kMaxChunks);
  }
#undef LL_LAUNCH_ADALN
  LL_CHECK_LAUNCH("adaln_kernel");
  return LL_OK;
}

extern "C" int ll_layer_norm(const void* x, int64_t rows, int C, const void* weight, const void* bias, float eps,
                             void* out, const ll_amax_sink* amax_sink, void* stream) {
  using namespace ll;
  LL_REQUIRE(x && out, "ll_layer_norm: null pointer");
  LL_REQUIRE(rows > 0 && rows <= 0x7FFFFFFF && C > 0 && C % 8 == 0 && C <= kMaxRowLength,
             "ll_layer_norm: bad shape rows=%lld C=%d", (long long)rows, C);
  LL_REQUIRE(((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(weight) | reinterpret_cast<uintptr_t>(bias) |
               reinterpret_cast<uintptr_t>(out)) & 15) == 0,
             "ll_layer_norm: pointers must be 16-byte aligned");
  LL_REQUIRE(sink_is_valid(amax_sink), "ll_layer_norm: amax sink needs 8-byte alignment and a non-zero epoch");
  const AmaxSink sink = make_sink(amax_sink);
  const dim3 grid((unsigned)((rows + kRowsPerWg - 1) / kRowsPerWg));
#define LL_LAUNCH_LN(NCH)                                                                                        \
  hipLaunchKernelGGL(layernorm_kernel<NCH>, grid, dim3(kRowThreads), 0, static_cast<hipStream_t>(stream),        \
                     static_cast<const uint16_t*>(x), rows, C, static_cast<const uint16_t*>(weight),             \
                     static_cast<const uint16_t*>(bias), eps, static_cast<uint16_t*>(out), sink)
  if (C <= 64 * 6 * 8) {
    LL_LAUNCH_LN(6);
  } else {
    LL_LAUNCH_LN(kMaxChunks);
  }
#undef LL_LAUNCH_LN
  LL_CHECK_LAUNCH("layernorm_kernel");
  return LL_OK;
}

extern "C" int ll_rms_norm(const void* x, int64_t rows, int C, const void* weight, float eps, void* out,
                           void* stream) {
  using namespace ll;
  LL_REQUIRE(x && weight && out, "ll_rms_norm: null pointer");
  LL_REQUIRE(rows > 0 && rows <= 0x7FFFFFFF && C > 0 && C % 8 == 0 && C <= kMaxRowLength,
             "ll_rms_norm: bad shape rows=%lld C=%d", (long long)rows, C);
  LL_REQUIRE(((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(weight) |
               reinterpret_cast<uintptr_t>(out)) & 15) == 0,
             "ll_rms_norm: pointers must be 16-byte aligned");
  const dim3 grid((unsigned)((rows + kRowsPerWg - 1) / kRowsPerWg));
#define LL_LAUNCH_RMS(NCH)                                                                                       \
  hipLaunchKernelGGL(rmsnorm_kernel<NCH>, grid, dim3(kRowThreads), 0, static_cast<hipStream_t>(stream),          \
                     static_cast<const uint16_t*>(x), rows, C, static_cast<const uint16_t*>(weight), eps,        \
                     static_cast<uint16_t*>(out))
  if (C <= 64 * 6 * 8) {
    LL_LAUNCH_RMS(6);
  } else {
    LL_LAUNCH_RMS(kMaxChunks);
  }
#undef LL_LAUNCH_RMS
  LL_CHECK_LAUNCH("rmsnorm_kernel");
  return LL_OK;
}

extern "C" int ll_gate_residual(const void* x, const void* y, int64_t B, int64_t L, int C, const void* gate,
                                int64_t gate_stride_b, int64_t gate_stride_f, int64_t frame_seqlen, void* out,
                                void* stream) {
  using namespace ll;
  LL_REQUIRE(x && y && gate && out, "ll_gate_residual: null pointer");
  LL_REQUIRE(B > 0 && L > 0 && C > 0 && C % 8 == 0 && frame_seqlen > 0, "ll_gate_residual: bad shape B=%lld L=%lld C=%d",
             (long long)B, (long long)L, C);
  LL_REQUIRE(gate_stride_b % 8 == 0 && gate_stride_f % 8 == 0 &&
                 ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(gate) |
                   reinterpret_cast<uintptr_t>(out)) & 15) == 0,
             "ll_gate_residual: pointers must be 16-byte aligned and strides multiples of 8 elements");
  const int64_t chunks = B * L * (C >> 3);
  LL_REQUIRE((chunks + 255) / 256 <= 0x7FFFFFFF, "ll_gate_residual: tensor too large");
  hipLaunchKernelGGL(gate_residual_kernel, dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<const uint16_t*>(x),
                     static_cast<const uint16_t*>(y), static_cast<const uint16_t*>(gate), L, C, gate_stride_b,
                     gate_stride_f, frame_seqlen, chunks, static_cast<uint16_t*>(out));
  LL_CHECK_LAUNCH("gate_residual_kernel");
  return LL_OK;
}

static int launch_qk_norm_rope(const ll::QkProblems& problems, int n_problems, int64_t rows, int num_heads, float eps,
                               const float* cos, const float* sin, int64_t seq_len, void* stream) {
  using namespace ll;
  const int64_t C = (int64_t)num_heads * 128;
  LL_REQUIRE(cos && sin, "ll_qk_norm_rope: null pointer");
  LL_REQUIRE(rows > 0 && rows <= 0x7FFFFFFF && num_heads > 0 && C <= kMaxRowLength && seq_len >= 0,
             "ll_qk_norm_rope: bad shape rows=%lld heads=%d", (long long)rows, num_heads);
  uintptr_t bits = reinterpret_cast<uintptr_t>(cos) | reinterpret_cast<uintptr_t>(sin);
  for (int i = 0; i < n_problems; ++i) {
    const QkProblem& q = problems.p[i];
    LL_REQUIRE(q.x && q.w && q.out, "ll_qk_norm_rope: null pointer");
    bits |= reinterpret_cast<uintptr_t>(q.x) | reinterpret_cast<uintptr_t>(q.w) | reinterpret_cast<uintptr_t>(q.out) |
            reinterpret_cast<uintptr_t>(q.out_smooth);
  }
  LL_REQUIRE((bits & 15) == 0, "ll_qk_norm_rope: pointers must be 16-byte aligned");
  const dim3 grid((unsigned)((rows + kRowsPerWg - 1) / kRowsPerWg), (unsigned)n_problems);
#define LL_LAUNCH_QK(NCH)                                                                                       \
  hipLaunchKernelGGL(qk_norm_rope_kernel<NCH>, grid, dim3(kRowThreads), 0, static_cast<hipStream_t>(stream),    \
                     problems, rows, (int)C, eps, cos, sin, seq_len)
  if (C <= 64 * 6 * 8) {
    LL_LAUNCH_QK(6);
  } else {
    LL_LAUNCH_QK(kMaxChunks);
  }
#undef LL_LAUNCH_QK
  LL_CHECK_LAUNCH("qk_norm_rope_kernel");
  return LL_OK;
}

extern "C" int ll_qk_norm_rope(const void* x, int64_t rows, int num_heads, const void* weight, float eps,
                               const float* cos, const float* sin, int64_t seq_len, void* out, void* out_smooth,
                               void* stream) {
  ll::QkProblems problems{};
  problems.p[0] = {static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(weight), static_cast<uint16_t*>(out),
                   static_cast<uint16_t*>(out_smooth), ll::AmaxSink{}};
  return launch_qk_norm_rope(problems, 1, rows, num_heads, eps, cos, sin, seq_len, stream);
}

extern "C" int ll_qk_norm_rope_pair(const void* q, const void* k, int64_t rows, int num_heads, const void* q_weight,
                                    const void* k_weight, float eps, const float* cos, const float* sin,
                                    int64_t seq_len, void* q_out, void* k_out, void* k_out_smooth, void* stream) {
  return ll_qk_norm_rope_pair_amax(q, k, rows, num_heads, q_weight, k_weight, eps, cos, sin, seq_len, q_out, k_out,
                                   k_out_smooth, nullptr, stream);
}

extern "C" int ll_qk_norm_rope_pair_amax(const void* q, const void* k, int64_t rows, int num_heads,
                                         const void* q_weight, const void* k_weight, float eps, const float* cos,
                                         const float* sin, int64_t seq_len, void* q_out, void* k_out,
                                         void* k_out_smooth, const ll_amax_sink* k_amax_sink, void* stream) {
  LL_REQUIRE(ll::sink_is_valid(k_amax_sink), "ll_qk_norm_rope_pair_amax: amax sink needs 8-byte alignment and a non-zero epoch");
  ll::QkProblems problems{};
  problems.p[0] = {static_cast<const uint16_t*>(q), static_cast<const uint16_t*>(q_weight),
                   static_cast<uint16_t*>(q_out), nullptr, ll::AmaxSink{}};
  problems.p[1] = {static_cast<const uint16_t*>(k), static_cast<const uint16_t*>(k_weight),
                   static_cast<uint16_t*>(k_out), static_cast<uint16_t*>(k_out_smooth), ll::make_sink(k_amax_sink)};
  return launch_qk_norm_rope(problems, 2, rows, num_heads, eps, cos, sin, seq_len, stream);
}
