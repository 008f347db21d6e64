// Test-only library (libll_nvfp4_testhooks.so), not part of the product ABI: applies the gfx950 conversion
// instructions the quantizer's fast path relies on to raw floats, so that the GPU tests can compare them with the
// software e4m3 / e2m1 codecs value by value; and runs the attention kernel's work-division arithmetic
// (attention_split.h, the very functions the kernel calls) on the host, so that the CPU tests can check that every
// (tile, iteration) of a launch is covered exactly once.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "attention_split.h"

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

// The segments of workgroup g, in the order the kernel walks them, as (tile, begin, end) triples; returns their
// number (at most max_segments are written).
extern "C" int ll_test_attention_segments(uint32_t G, uint32_t units, uint32_t whole_rounds, uint32_t n_iter,
                                          uint32_t g, int32_t* out, int max_segments) {
  ll::WorkCursor at = ll::start_of_work(g, G, units);
  ll::Segment seg;
  int n = 0;
  while (ll::next_segment(at, g, G, units, whole_rounds, n_iter, seg)) {
    if (n < max_segments) {
      out[3 * n] = (int32_t)seg.tile;
      out[3 * n + 1] = seg.begin;
      out[3 * n + 2] = seg.end;
    }
    ++n;
  }
  return n;
}

// First and last workgroup with a part of split tile `split_tile`, and the record workgroup g uses for its part.
extern "C" void ll_test_attention_parts(uint32_t split_tile, uint32_t G, uint32_t units, uint32_t n_iter,
                                        uint32_t* g_first, uint32_t* g_last) {
  ll::parts_of_tile(split_tile, G, units, n_iter, *g_first, *g_last);
}
extern "C" uint32_t ll_test_attention_record(uint32_t g, uint32_t split_tile, uint32_t G, uint32_t units,
                                             uint32_t n_iter) {
  return ll::record_of_part(g, split_tile, G, units, n_iter);
}
