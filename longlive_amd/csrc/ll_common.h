// Shared device/host helpers for the gfx950 NVFP4 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include <atomic>

#include "../../include/ll_nvfp4.h"

namespace ll {

// ----------------------------------------------------------------------------- errors
void set_error(const char* fmt, ...);

#define LL_REQUIRE(cond, ...)      \
  do {                             \
    if (!(cond)) {                 \
      ll::set_error(__VA_ARGS__);  \
      return LL_EINVAL;            \
    }                              \
  } while (0)

#define LL_CHECK_LAUNCH(name)                                              \
  do {                                                                     \
    hipError_t e__ = hipGetLastError();                                    \
    if (e__ != hipSuccess) {                                               \
      ll::set_error("%s: launch failed: %s", name, hipGetErrorString(e__)); \
      return LL_ELAUNCH;                                                   \
    }                                                                      \
  } while (0)

inline int64_t round_up(int64_t x, int64_t m) { return (x + m - 1) / m * m; }

// ----------------------------------------------------------------------------- memory of the library's own (stream_scratch.hip)
// Records for partial tiles and arrival counters, one set per (device, stream).
struct StreamScratch {
  uint8_t* records = nullptr;
  size_t record_bytes = 0;
  int* counters = nullptr;  // zero whenever no launch is running
  size_t n_counters = 0;
};
// A set with at least record_bytes and `counters` counters.  may_allocate false (the stream is being captured into
// a graph): only a set that is already large enough is handed out, and *missing says that there is none.
int stream_scratch(int dev, hipStream_t stream, size_t record_bytes, size_t counters, bool may_allocate, StreamScratch& out,
                   bool* missing, const char* what);
int release_stream_scratch(int dev, hipStream_t stream);
// Whether work submitted to `stream` is being recorded into a graph instead of run.  A failing query (the legacy
// stream while another stream of the thread captures) counts as recording: then nothing may be allocated either.
bool stream_is_capturing(hipStream_t stream);
int compute_units_of(int dev, int& cus, const char* what);

// Kernels that need more than 64 KB of dynamic LDS have to be told so with hipFuncSetAttribute, and that setting
// holds per device.  `done` (one per kernel, zero-initialised) keeps one bit per device ordinal so that the call
// is made once for every device the kernel is launched on; two threads racing here both make the same call.
inline int allow_dynamic_lds(const void* kernel, size_t bytes, std::atomic<uint64_t>& done, const char* what) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    set_error("%s: hipGetDevice failed: %s", what, hipGetErrorString(e));
    return LL_ELAUNCH;
  }
  const uint64_t bit = 1ull << (dev & 63);
  if (dev < 64 && (done.load(std::memory_order_acquire) & bit)) return LL_OK;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  if (e != hipSuccess) {
    set_error("%s: cannot reserve %zu bytes of LDS: %s", what, bytes, hipGetErrorString(e));
    return LL_ELAUNCH;
  }
  if (dev < 64) done.fetch_or(bit, std::memory_order_release);
  return LL_OK;
}

// ----------------------------------------------------------------------------- formats
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

// fp32 -> bf16 bits, round to nearest even, with the hardware conversion of gfx950 (v_cvt_pk_bf16_f32;
// NaN becomes a quiet NaN).
typedef __bf16 bf16x2_hw __attribute__((ext_vector_type(2)));
typedef float f32x2_hw __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  return (uint32_t)__builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
}
// Two values at once: lo in bits 0-15, hi in bits 16-31.
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const f32x2_hw v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_hw));
}
__device__ __forceinline__ float round_to_bf16(float f) { return __uint_as_float(f32_to_bf16_bits(f) << 16); }

// e4m3fn byte -> fp32 (exact). 0x7F / 0xFF decode to NaN.
__device__ __forceinline__ float e4m3_to_f32(uint32_t b) {
  uint32_t e = (b >> 3) & 0xFu, m = b & 7u;
  float v;
  if (e == 0) {
    v = (float)m * 0.001953125f;  // m * 2^-9
  } else if (e == 15 && m == 7) {
    v = __uint_as_float(0x7FC00000u);
  } else {
    v = __uint_as_float(((e + 120u) << 23) | (m << 20));
  }
  return (b & 0x80u) ? -v : v;
}

// fp32 -> e4m3fn byte, round to nearest even, |x| > 464 -> NaN (0x7F): the value torch's
// float8_e4m3fn cast produces.
__device__ __forceinline__ uint32_t f32_to_e4m3(float x) {
  uint32_t u = __float_as_uint(x);
  uint32_t sign = (u >> 24) & 0x80u;
  u &= 0x7FFFFFFFu;
  float a = __uint_as_float(u);
  if (!(a <= 464.0f)) return sign | 0x7Fu;  // NaN, inf, overflow
  if (a >= 0.015625f) {                     // normal range: keep 3 mantissa bits
    uint32_t r = (u + 0x7FFFFu + ((u >> 20) & 1u)) >> 20;
    return sign | (r - (120u << 3));
  }
  return sign | (uint32_t)__builtin_rintf(a * 512.0f);  // sub-normal grid 2^-9, 8 -> 2^-6
}

__device__ __constant__ const float kE2M1[16] = {0.0f,  0.5f,  1.0f,  1.5f,  2.0f,  3.0f,  4.0f,  6.0f,
                                                 -0.0f, -0.5f, -1.0f, -1.5f, -2.0f, -3.0f, -4.0f, -6.0f};

// Offset of scale (r, c) of a [rows, cols] e4m3 matrix stored in 128x4 blocked order.
__host__ __device__ __forceinline__ int64_t blocked_scale_offset(int64_t r, int64_t c, int64_t cols) {
  int64_t rb = r >> 7, ri = r & 127, cb = c >> 2, ci = c & 3;
  return ((rb * (cols >> 2) + cb) * 32 + (ri & 31)) * 16 + (ri >> 5) * 4 + ci;
}

__host__ __device__ __forceinline__ void rule_limits(int rule, float& e2, float& e4) {
  e2 = (rule == LL_RULE_STATIC_4) ? 4.0f : 6.0f;
  e4 = (rule == LL_RULE_STATIC_6 || rule == LL_RULE_STATIC_4) ? 448.0f : 256.0f;
}

// 1 / (e2m1_max * e4m3_max) of a KV-cache slot as the reference's fused dequantization forms it: the reciprocal
// in double, rounded to fp32 once (utils/kernel/kv_dequant_cuda.cu:216); the slot scale is amax times this.
inline float kv_inverse_denominator(float e2m1_max, float e4m3_max) {
  return static_cast<float>(1.0 / (static_cast<double>(e2m1_max) * static_cast<double>(e4m3_max)));
}

// ----------------------------------------------------------------------------- wave helpers
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
// Sum over the wave with data-parallel-primitive moves instead of LDS permutes: partial sums travel down
// each row of 16 lanes (row_shr 1, 2, 3, then 4 and 8 under bank masks), then across the rows (row_bcast 15
// and 31), which leaves the total in lane 63; every lane returns that value.  Lanes that a move does not
// reach contribute 0 (bound_ctrl).
#define LL_DPP_ADD(v, ctrl, row_mask, bank_mask)                                                                 \
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, row_mask, bank_mask, true))
__device__ __forceinline__ float wave_sum_dpp(float v) {
  LL_DPP_ADD(v, 0x111, 0xF, 0xF);  // row_shr:1
  LL_DPP_ADD(v, 0x112, 0xF, 0xF);  // row_shr:2
  LL_DPP_ADD(v, 0x114, 0xF, 0xE);  // row_shr:4, lanes 4-15 of each row
  LL_DPP_ADD(v, 0x118, 0xF, 0xC);  // row_shr:8, lanes 8-15 of each row
  LL_DPP_ADD(v, 0x142, 0xA, 0xF);  // row_bcast:15 into rows 1 and 3
  LL_DPP_ADD(v, 0x143, 0xC, 0xF);  // row_bcast:31 into rows 2 and 3
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
#undef LL_DPP_ADD

// max(m, |v|) over the 8 bf16 values of a packed 16-byte group
__device__ __forceinline__ float abs_max_bf16x8(const uint4& v, float m) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    m = fmaxf(m, fabsf(__uint_as_float(w[i] << 16)));
    m = fmaxf(m, fabsf(__uint_as_float(w[i] & 0xFFFF0000u)));
  }
  return m;
}
// Amax sink: a kernel that writes a tensor leaves partial absolute maxima of it in LL_AMAX_PARTS 64-bit
// slots, each holding (epoch << 32) | float bits and raised with a 64-bit atomic max.  A value of a newer
// epoch beats every older one, so the slots never need clearing; the reader ignores slots of other epochs.
// (The bit patterns of non-negative floats order like unsigned integers.)
constexpr int kAmaxParts = LL_AMAX_PARTS;
struct AmaxSink {
  unsigned long long* parts;     // null: no sink
  uint32_t epoch;
  const uint32_t* epoch_offset;  // device word added to epoch when the kernel runs (launches replayed from a graph), or null
};
__device__ __forceinline__ uint32_t amax_sink_epoch(uint32_t epoch, const uint32_t* epoch_offset) {
  return epoch + (epoch_offset ? *epoch_offset : 0u);
}
__device__ __forceinline__ void amax_sink_update(const AmaxSink& sink, uint32_t slot, float v) {
  const uint32_t epoch = amax_sink_epoch(sink.epoch, sink.epoch_offset);
  atomicMax(sink.parts + (slot & (kAmaxParts - 1)), ((unsigned long long)epoch << 32) | __float_as_uint(v));
}
// The kernel-side sink of a caller's ll_amax_sink (null or without a buffer: no sink).
inline AmaxSink make_sink(const ll_amax_sink* s) {
  AmaxSink k{};
  if (s && s->parts) {
    k.parts = reinterpret_cast<unsigned long long*>(s->parts);
    k.epoch = s->epoch;
    k.epoch_offset = s->epoch_offset;
  }
  return k;
}
inline bool sink_is_valid(const ll_amax_sink* s) {
  return !s || !s->parts ||
         ((reinterpret_cast<uintptr_t>(s->parts) & 7) == 0 && s->epoch != 0 && (reinterpret_cast<uintptr_t>(s->epoch_offset) & 3) == 0);
}
__device__ __forceinline__ float amax_sink_read(const unsigned long long* parts, uint32_t epoch, int slot) {
  const unsigned long long v = parts[slot];
  return (uint32_t)(v >> 32) == epoch ? __uint_as_float((uint32_t)v) : 0.0f;
}

}  // namespace ll
