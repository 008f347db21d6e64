// Test-only library (libll_nvfp4_testhooks.so), not part of the product ABI: applies the gfx950 conversion
// instructions the quantizer's fast path relies on to raw floats, so that the GPU tests can compare them with the
// software e4m3 / e2m1 codecs value by value; and runs the attention kernel's work-division arithmetic
// (attention_split.h, the very functions the kernel calls) on the host, so that the CPU tests can check that every
// (tile, iteration) of a launch is covered exactly once - and on the device, so that the GPU tests can check that both
// sides compute the same numbers.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "attention_split.h"
#include "gemm_split.h"

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

// A division travels as seven numbers: G, whole_rounds, extra, n_iter, units, full_units, light.
static ll::Division division_of(const uint32_t* d) { return ll::Division{d[0], d[1], d[2], d[3], d[4], d[5], d[6]}; }

// The segments of workgroup g, in the order the kernel walks them, as (tile, begin, end) triples; returns their
// number (at most max_segments are written).
extern "C" int ll_test_attention_segments(const uint32_t* division, uint32_t g, int32_t* out, int max_segments) {
  const ll::Division d = division_of(division);
  ll::WorkCursor at = ll::start_of_work(g, d);
  ll::Segment seg;
  int n = 0;
  while (ll::next_segment(at, g, d, seg)) {
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
extern "C" void ll_test_attention_parts(uint32_t split_tile, const uint32_t* division, uint32_t* g_first, uint32_t* g_last) {
  ll::parts_of_tile(split_tile, division_of(division), *g_first, *g_last);
}
extern "C" uint32_t ll_test_attention_record(uint32_t g, uint32_t split_tile, const uint32_t* division) {
  return ll::record_of_part(g, split_tile, division_of(division));
}

// The launcher's whole choice for a shape: out = mode, n_qtiles, full_qtiles, split_tiles, then the division's
// seven numbers.
extern "C" void ll_test_attention_full_plan(int64_t Lq, int H, int64_t n_keys, int cus, int policy, uint32_t* out) {
  const ll::AttentionPlan plan = ll::plan_attention(Lq, H, n_keys, cus, policy);
  out[0] = (uint32_t)plan.mode;
  out[1] = (uint32_t)plan.n_qtiles;
  out[2] = (uint32_t)plan.full_qtiles;
  out[3] = (uint32_t)plan.split_tiles;
  const uint32_t d[7] = {plan.d.G, plan.d.whole_rounds, plan.d.extra, plan.d.n_iter, plan.d.units, plan.d.full_units, plan.d.light};
  for (int i = 0; i < 7; ++i) out[4 + i] = d[i];
}

// The same arithmetic evaluated on the device: out[g] = first_unit_of(g) for g = 0 .. G, then for every split tile
// its first and last holder (2 * split_tiles numbers).  Returns 0, -2 when the launch fails.
__global__ void division_kernel(ll::Division d, uint32_t split_tiles, uint32_t* __restrict__ out) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i <= d.G) out[i] = ll::first_unit_of(i, d);
  if (i < split_tiles) ll::parts_of_tile(i, d, out[d.G + 1 + 2 * i], out[d.G + 2 + 2 * i]);
}
extern "C" int ll_test_attention_division_on_device(const uint32_t* division, uint32_t split_tiles, uint32_t* out,
                                                    void* stream) {
  const ll::Division d = division_of(division);
  const uint32_t n = d.G + 1 > split_tiles ? d.G + 1 : split_tiles;
  hipLaunchKernelGGL(division_kernel, dim3((n + 255) / 256), dim3(256), 0, static_cast<hipStream_t>(stream), d,
                     split_tiles, out);
  return hipGetLastError() == hipSuccess ? 0 : -2;
}

// Host counterpart of first_unit_of for the comparison.
extern "C" uint32_t ll_test_attention_first_unit(uint32_t g, const uint32_t* division) {
  return ll::first_unit_of(g, division_of(division));
}

// ---- the persistent GEMM's division (gemm_split.h) on the host.  A division travels as four numbers: G, tiles, nk,
// whole_rounds.
static ll::GemmDivision gemm_division_of(const uint32_t* d) { return ll::GemmDivision{d[0], d[1], d[2], d[3]}; }

// The segments of workgroup g, in the order the kernel walks them, as (tile, begin, end) triples; returns their number.
extern "C" int ll_test_gemm_segments(const uint32_t* division, uint32_t g, int32_t* out, int max_segments) {
  const ll::GemmDivision d = gemm_division_of(division);
  ll::GemmCursor at = ll::gemm_start_of_work(g, d);
  ll::GemmSegment seg;
  int n = 0;
  while (ll::gemm_next_segment(at, g, d, seg)) {
    if (n < max_segments) {
      out[3 * n] = (int32_t)seg.tile;
      out[3 * n + 1] = (int32_t)seg.begin;
      out[3 * n + 2] = (int32_t)seg.end;
    }
    ++n;
  }
  return n;
}
extern "C" void ll_test_gemm_parts(uint32_t split_tile, const uint32_t* division, uint32_t* g_first, uint32_t* g_last) {
  ll::gemm_parts_of_tile(split_tile, gemm_division_of(division), *g_first, *g_last);
}
extern "C" uint32_t ll_test_gemm_record(uint32_t g, uint32_t split_tile, const uint32_t* division) {
  return ll::gemm_record_of_part(g, split_tile, gemm_division_of(division));
}
// The launcher's choice for a shape: out = use, G, tiles, nk, whole_rounds, tiles_m, tiles_n_each.
extern "C" void ll_test_gemm_plan(int64_t M, int64_t N, int64_t Kp, int n_products, int cus, int schedule, uint32_t* out) {
  const ll::PersistentPlan plan = ll::plan_persistent(M, N, Kp, n_products, cus, schedule);
  out[0] = plan.use ? 1u : 0u;
  out[1] = plan.d.G;
  out[2] = plan.d.tiles;
  out[3] = plan.d.nk;
  out[4] = plan.d.whole_rounds;
  out[5] = (uint32_t)plan.tiles_m;
  out[6] = (uint32_t)plan.tiles_n_each;
}
