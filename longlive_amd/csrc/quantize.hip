// NVFP4 quantization for gfx950: tensor amax, block-16 e4m3 scales, e2m1 codes, and the
// four-over-six per-block choice.  Arithmetic follows the reference's PyTorch backend
// (fouroversix/src/fouroversix/quantize/pytorch/reference.py:121-368) operation by operation, so
// the packed bytes are identical to what that backend produces on a CPU.
//
// This file must be compiled without floating-point contraction: every product and sum below is
// rounded separately, as the eager PyTorch graph rounds it.
#include "ll_common.h"
#include "quantize_block.h"

#pragma clang fp contract(off)

namespace ll {

constexpr int kThreads = 256;

// ----------------------------------------------------------------------------- amax
// Each workgroup folds a grid-strided share of x into one partial maximum; the quantize kernel
// reduces the kAmaxParts partials again, so no atomics and no zero-initialised state are needed.
__global__ __launch_bounds__(kThreads) void amax_partial_kernel(const uint16_t* __restrict__ x, int64_t M, int64_t K,
                                                                 int64_t ldx, float* __restrict__ parts) {
  float m = 0.0f;
  const int64_t tid = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  const int64_t nthreads = (int64_t)gridDim.x * kThreads;
  const bool vec = ((K & 7) == 0) && ((ldx & 7) == 0) && ((reinterpret_cast<uintptr_t>(x) & 15) == 0);
  if (vec) {
    const int64_t kc = K >> 3;
    const int64_t nchunks = M * kc;
    for (int64_t c = tid; c < nchunks; c += nthreads) {
      const int64_t r = c / kc, cc = c - r * kc;
      const uint4 v = *reinterpret_cast<const uint4*>(x + r * ldx + cc * 8);
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        m = fmaxf(m, fabsf(__uint_as_float(w[i] << 16)));
        m = fmaxf(m, fabsf(__uint_as_float(w[i] & 0xFFFF0000u)));
      }
    }
  } else {
    const int64_t n = M * K;
    for (int64_t i = tid; i < n; i += nthreads) {
      const int64_t r = i / K, c = i - r * K;
      m = fmaxf(m, fabsf(bf16_bits_to_f32(x[r * ldx + c])));
    }
  }
  m = wave_max(m);
  __shared__ float sm[kThreads / 64];
  if ((threadIdx.x & 63) == 0) sm[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
    float r = sm[0];
    for (int i = 1; i < kThreads / 64; ++i) r = fmaxf(r, sm[i]);
    parts[blockIdx.x] = r;
  }
}

// ----------------------------------------------------------------------------- quantize kernel
// One workgroup = a 128-row x 64-column tile = 512 blocks of 16 = one 512-byte tile of the blocked
// scale layout, which is staged in LDS and written with coalesced 4-byte stores.
// GENERIC = false: x is 16-byte aligned with ldx a multiple of 8 and K a multiple of 64, so every block is two
// whole 16-byte pieces and only rows beyond M need care (zeros).  GENERIC = true handles any K, ldx and
// alignment element by element at the edges.
// What differs between the tensors of one launch (one or two tensors of the same shape: the K and V of a chunk).
struct QuantJob {
  const uint16_t* x;
  uint8_t* values;
  uint8_t* scales;
  float* amax_io;
  const float* parts;
  const unsigned long long* sink_parts;
  uint32_t sink_epoch_base;
  const uint32_t* sink_epoch_offset;
};
struct QuantJobs {
  QuantJob j[2];
  int n;  // the first half of the workgroups takes j[0], the second half j[1]
};

template <int RULE, bool GENERIC>
__global__ __launch_bounds__(kThreads) void quantize_kernel(QuantJobs jobs, int64_t M, int64_t K, int64_t ldx, int64_t Kp,
                                                            int amax_given, int64_t total_tiles) {
  // The tensor this workgroup works on (uniform selects, no indexing of the argument block).
  const uint32_t per_job = jobs.n == 2 ? gridDim.x >> 1 : gridDim.x;
  const bool second = jobs.n == 2 && blockIdx.x >= per_job;
  const uint32_t wg_in_job = second ? blockIdx.x - per_job : blockIdx.x;
  const uint16_t* __restrict__ x = second ? jobs.j[1].x : jobs.j[0].x;
  uint8_t* __restrict__ values = second ? jobs.j[1].values : jobs.j[0].values;
  uint8_t* __restrict__ scales = second ? jobs.j[1].scales : jobs.j[0].scales;
  float* __restrict__ amax_io = second ? jobs.j[1].amax_io : jobs.j[0].amax_io;
  const float* __restrict__ parts = second ? jobs.j[1].parts : jobs.j[0].parts;
  const unsigned long long* __restrict__ sink_parts = second ? jobs.j[1].sink_parts : jobs.j[0].sink_parts;
  const uint32_t sink_epoch_base = second ? jobs.j[1].sink_epoch_base : jobs.j[0].sink_epoch_base;
  const uint32_t* __restrict__ sink_epoch_offset = second ? jobs.j[1].sink_epoch_offset : jobs.j[0].sink_epoch_offset;
  __shared__ float s_red[kThreads / 64];
  __shared__ uint32_t s_scales[2][128];  // two staged 512-byte scale tiles in blocked order
  __shared__ ScaleEntry s_tab[128];
  static_assert(kThreads == 256 && kAmaxParts == 4 * kThreads, "four waves, four partial maxima per thread");

  // ---- tensor amax: given, or the maximum of the kAmaxParts partial maxima (every wave folds its share, the four
  // wave results meet in LDS and every thread folds those itself: one barrier)
  float amax;
  if (amax_given) {
    amax = amax_io[0];
  } else {
    float4 p;
    if (sink_parts) {
      const uint32_t sink_epoch = amax_sink_epoch(sink_epoch_base, sink_epoch_offset);
      p = make_float4(amax_sink_read(sink_parts, sink_epoch, 4 * threadIdx.x),
                      amax_sink_read(sink_parts, sink_epoch, 4 * threadIdx.x + 1),
                      amax_sink_read(sink_parts, sink_epoch, 4 * threadIdx.x + 2),
                      amax_sink_read(sink_parts, sink_epoch, 4 * threadIdx.x + 3));
    } else {
      p = reinterpret_cast<const float4*>(parts)[threadIdx.x];
    }
    const float m = wave_max(fmaxf(fmaxf(p.x, p.y), fmaxf(p.z, p.w)));
    if ((threadIdx.x & 63) == 0) s_red[threadIdx.x >> 6] = m;
    __syncthreads();
    amax = fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3]));
    if (wg_in_job == 0 && threadIdx.x == 0) amax_io[0] = amax;
  }

  // The fast path needs every block maximum to stay below amax (so block scales stay within e4m3 range: true by
  // construction when the amax was computed here, checked block by block when the caller supplied it) and amax far
  // from the ends of the fp32 range (so powers of two scale exactly; uniform over the launch); otherwise the exact
  // path is taken.
  constexpr bool kStaticRule = (RULE == LL_RULE_STATIC_6 || RULE == LL_RULE_STATIC_4);
  constexpr float kE2 = (RULE == LL_RULE_STATIC_4) ? 4.0f : 6.0f;
  constexpr float kE4 = kStaticRule ? 448.0f : 256.0f;
  const bool fast = amax >= 0x1p-100f && amax <= 0x1p100f;
  const float bound = amax_given ? amax : __builtin_inff();
  const bool approx_ok = amax >= 0x1p-30f && amax <= 0x1p30f;  // squares of errors stay normal fp32 numbers
  const float enc = (kE2 * kE4) / amax;
  const float dec = 1.0f / enc;
  if (fast) fill_scale_table<RULE>(s_tab, amax, dec);
  __syncthreads();

  const bool vec = ((ldx & 7) == 0) && ((reinterpret_cast<uintptr_t>(x) & 15) == 0);
  const uint32_t tiles_x = (uint32_t)(Kp >> 6);

  // Tiles are dealt to the resident workgroups round-robin, so the prologue above (amax reduction,
  // scale table) is paid once per workgroup and not once per tile.
  // A tile's rows receive 32 packed bytes each, a quarter of a 128-byte line; the four tiles that complete
  // the lines are consecutive in tile order.  Consecutive workgroup ids are dealt round-robin to the 8 XCDs,
  // each with an L2 of its own, so the four tiles go to workgroups v, v + 8, v + 16, v + 24, which start on
  // the same XCD at about the same time and let that L2 merge the partial lines before they are written back.
  // The grid is a multiple of 32 workgroups, so a workgroup's next tile is its current one plus the grid size:
  // the tile's row and column advance by constants, and no division is left in the loop.
  const uint32_t n_tiles = (uint32_t)total_tiles;
  const uint32_t grid = per_job, wg = wg_in_job;
  const uint32_t first_tile = ((wg >> 5) * 8u + (wg & 7u)) * 4u + ((wg >> 3) & 3u);
  const uint32_t step_y = grid / tiles_x, step_x = grid - step_y * tiles_x;

  // The thread's two blocks of a tile: block b = threadIdx.x + it * kThreads, row b / 4, column block b % 4.
  const int r0 = threadIdx.x >> 2, cb = threadIdx.x & 3;
  const int64_t vrow = Kp >> 1;                                   // bytes per row of packed values
  const int64_t thread_x = (int64_t)r0 * ldx + cb * 16;           // elements, from the tile's first element
  const int64_t thread_v = (int64_t)r0 * vrow + cb * 8;           // bytes, from the tile's first packed byte
  const int s_off0 = (r0 & 31) * 16 + (r0 >> 5) * 4 + cb;         // staged scale byte of the block of it = 0; it = 1: + 8
  // The 32 bytes of one block as they lie in memory (16 bf16 values); blocks that stick out of the tensor are
  // completed with zeros, like the reference's zero padding.
  struct Raw {
    uint4 lo, hi;
  };
  struct Tile {
    uint32_t index, ty, tx;
  };
  auto load_block = [&](const Tile& t, int it, Raw& raw) {
    const int64_t row0 = (int64_t)t.ty * 128, col0 = (int64_t)t.tx * 64;
    if (!GENERIC || (vec && col0 + 64 <= K)) {  // whole 16-byte pieces; rows beyond M are zeros
      if (row0 + r0 + it * 64 < M) {
        const uint4* p = reinterpret_cast<const uint4*>(x + (row0 * ldx + col0) + thread_x + (int64_t)it * 64 * ldx);
        raw.lo = p[0];
        raw.hi = p[1];
      } else {
        raw.lo = raw.hi = make_uint4(0u, 0u, 0u, 0u);
      }
    } else {
      const int64_t row = row0 + r0 + it * 64, col = col0 + cb * 16;
      uint32_t w[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const uint32_t e0 = (row < M && col + 2 * i < K) ? x[row * ldx + col + 2 * i] : 0u;
        const uint32_t e1 = (row < M && col + 2 * i + 1 < K) ? x[row * ldx + col + 2 * i + 1] : 0u;
        w[i] = e0 | (e1 << 16);
      }
      raw.lo = make_uint4(w[0], w[1], w[2], w[3]);
      raw.hi = make_uint4(w[4], w[5], w[6], w[7]);
    }
  };
  // Quantize one block and store its 8 packed bytes; the scale byte goes to the staged 128x4 scale tile.
  auto quantize_store = [&](const Tile& t, int it, const Raw& raw, uint8_t* s_bytes) {
    const uint32_t w[8] = {raw.lo.x, raw.lo.y, raw.lo.z, raw.lo.w, raw.hi.x, raw.hi.y, raw.hi.z, raw.hi.w};
    float X[16];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      X[2 * i] = __uint_as_float(w[i] << 16);
      X[2 * i + 1] = __uint_as_float(w[i] & 0xFFFF0000u);
    }
    uint32_t lo, hi, sb;
    if (!fast || !quantize_block_fast<RULE>(X, enc, s_tab, approx_ok, bound, lo, hi, sb)) quantize_block<RULE>(X, amax, enc, dec, lo, hi, sb);
    uint8_t* dst = values + ((int64_t)t.ty * 128 * vrow + (int64_t)t.tx * 32) + thread_v + (int64_t)it * 64 * vrow;
    *reinterpret_cast<uint2*>(dst) = make_uint2(lo, hi);
    s_bytes[s_off0 + it * 8] = (uint8_t)sb;
  };
  auto advance = [&](Tile& t) {
    t.index += grid;
    t.ty += step_y;
    t.tx += step_x;
    if (t.tx >= tiles_x) {
      t.tx -= tiles_x;
      ++t.ty;
    }
  };

  // One barrier per tile: the staged scale tile is double-buffered.
  Tile cur;
  cur.index = first_tile;
  cur.ty = first_tile / tiles_x;
  cur.tx = first_tile - cur.ty * tiles_x;
  int parity = 0;
#pragma unroll 1
  while (cur.index < n_tiles) {
    uint8_t* s_bytes = reinterpret_cast<uint8_t*>(s_scales[parity]);
#pragma unroll 1
    for (int it = 0; it < 2; ++it) {
      Raw raw;
      load_block(cur, it, raw);
      quantize_store(cur, it, raw, s_bytes);
    }
    __syncthreads();
    if (threadIdx.x < 128)
      reinterpret_cast<uint32_t*>(scales)[(int64_t)cur.index * 128 + threadIdx.x] = s_scales[parity][threadIdx.x];
    parity ^= 1;  // the next tile stages into the other buffer; this one is rewritten two barriers from now
    advance(cur);
  }
}

}  // namespace ll

extern "C" size_t ll_nvfp4_quantize_workspace_floats(void) { return ll::kAmaxParts; }

// Workgroups of quantize_kernel<rule, generic> that fit on the current device at once (occupancy per CU from the
// runtime, times the CU count), looked up once per device and kernel.
static int resident_workgroups(int rule, bool generic, int64_t* out) {
  using namespace ll;
  static std::atomic<int> cache[64][5][2];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    set_error("ll_nvfp4_quantize: hipGetDevice failed: %s", hipGetErrorString(e));
    return LL_ELAUNCH;
  }
  std::atomic<int>* slot = (dev >= 0 && dev < 64) ? &cache[dev][rule][generic ? 1 : 0] : nullptr;
  int n = slot ? slot->load(std::memory_order_relaxed) : 0;
  if (n == 0) {
    int per_cu = 0, cus = 0;
#define LL_OCC(R)                                                                                                        \
  e = generic ? hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, quantize_kernel<R, true>, kThreads, 0)            \
              : hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, quantize_kernel<R, false>, kThreads, 0)
    switch (rule) {
      case LL_RULE_STATIC_6: LL_OCC(LL_RULE_STATIC_6); break;
      case LL_RULE_STATIC_4: LL_OCC(LL_RULE_STATIC_4); break;
      case LL_RULE_MAE: LL_OCC(LL_RULE_MAE); break;
      case LL_RULE_MSE: LL_OCC(LL_RULE_MSE); break;
      default: LL_OCC(LL_RULE_ABS_MAX); break;
    }
#undef LL_OCC
    if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess || per_cu <= 0 || cus <= 0) {
      set_error("ll_nvfp4_quantize: occupancy query failed: %s", hipGetErrorString(e));
      return LL_ELAUNCH;
    }
    n = per_cu * cus;
    if (n < 32) n = 32;
    if (slot) slot->store(n, std::memory_order_relaxed);
  }
  *out = n;
  return LL_OK;
}

// One host-side description per tensor of a launch.
struct QuantRequest {
  const void* x;
  uint8_t* values;
  uint8_t* scales;
  float* amax;
  float* workspace;
  const ll_amax_sink* sink;
};

// n = 1 or 2 tensors of the same shape, leading dimension, rule and source of the amax, in one launch: the
// resident workgroups are split evenly between them.
static int quantize_impl(const QuantRequest* req, int n, int64_t M, int64_t K, int64_t ldx, int rule, int amax_given,
                         void* stream) {
  using namespace ll;
  LL_REQUIRE(n == 1 || n == 2, "ll_nvfp4_quantize: %d tensors in one launch (1 or 2)", n);
  LL_REQUIRE(M > 0 && K > 0 && ldx >= K, "ll_nvfp4_quantize: bad shape M=%lld K=%lld ldx=%lld", (long long)M,
             (long long)K, (long long)ldx);
  LL_REQUIRE(rule >= 0 && rule <= 4, "ll_nvfp4_quantize: unknown scale rule %d", rule);
  const int64_t Mp = round_up(M, 128), Kp = round_up(K, 64);
  const int64_t total_tiles = (Kp / 64) * (Mp / 128);
  LL_REQUIRE(total_tiles < (1ll << 31), "ll_nvfp4_quantize: tensor too large for one launch");
  hipStream_t s = static_cast<hipStream_t>(stream);
  QuantJobs jobs{};
  jobs.n = n;
  bool generic = (K % 64) != 0 || (ldx % 8) != 0;
  for (int i = 0; i < n; ++i) {
    const QuantRequest& r = req[i];
    LL_REQUIRE(r.x && r.values && r.scales && r.amax, "ll_nvfp4_quantize: null pointer");
    LL_REQUIRE(amax_given || r.workspace || r.sink, "ll_nvfp4_quantize: workspace required to compute amax");
    LL_REQUIRE(!r.sink || (r.sink->parts && sink_is_valid(r.sink)),
               "ll_nvfp4_quantize_from_sink: amax sink needs an 8-byte aligned buffer and a non-zero epoch");
    LL_REQUIRE((reinterpret_cast<uintptr_t>(r.values) & 7) == 0 && (reinterpret_cast<uintptr_t>(r.scales) & 3) == 0,
               "ll_nvfp4_quantize: outputs must be 8-byte (values) / 4-byte (scales) aligned");
    generic = generic || (reinterpret_cast<uintptr_t>(r.x) & 15) != 0;
    QuantJob& j = jobs.j[i];
    j.x = static_cast<const uint16_t*>(r.x);
    j.values = r.values;
    j.scales = r.scales;
    j.amax_io = r.amax;
    j.parts = r.workspace;
    j.sink_parts = r.sink ? reinterpret_cast<const unsigned long long*>(r.sink->parts) : nullptr;
    j.sink_epoch_base = r.sink ? r.sink->epoch : 0u;
    j.sink_epoch_offset = r.sink ? r.sink->epoch_offset : nullptr;
    if (!amax_given && !r.sink) {
      hipLaunchKernelGGL(amax_partial_kernel, dim3(kAmaxParts), dim3(kThreads), 0, s, j.x, M, K, ldx, r.workspace);
      LL_CHECK_LAUNCH("amax_partial_kernel");
    }
  }
  // One workgroup per tile up to what the chip holds at once (the launch is persistent: every workgroup has to be
  // resident from the start, or the ones that wait would run after the others have finished).
  int64_t resident = 0;
  if (int rc = resident_workgroups(rule, generic, &resident)) return rc;
  const int64_t padded_tiles = (total_tiles + 31) & ~(int64_t)31;  // whole groups of 32 for the XCD-aware tile order
  int64_t share = (resident / n) & ~(int64_t)31;                  // workgroups per tensor
  if (share < 32) share = 32;
  const dim3 grid((unsigned)((padded_tiles < share ? padded_tiles : share) * n));
#define LL_LAUNCH_Q(R)                                                                                                  \
  do {                                                                                                                  \
    if (generic)                                                                                                        \
      hipLaunchKernelGGL((quantize_kernel<R, true>), grid, dim3(kThreads), 0, s, jobs, M, K, ldx, Kp, amax_given,      \
                         total_tiles);                                                                                  \
    else                                                                                                                \
      hipLaunchKernelGGL((quantize_kernel<R, false>), grid, dim3(kThreads), 0, s, jobs, M, K, ldx, Kp, amax_given,     \
                         total_tiles);                                                                                  \
  } while (0)
  switch (rule) {
    case LL_RULE_STATIC_6: LL_LAUNCH_Q(LL_RULE_STATIC_6); break;
    case LL_RULE_STATIC_4: LL_LAUNCH_Q(LL_RULE_STATIC_4); break;
    case LL_RULE_MAE: LL_LAUNCH_Q(LL_RULE_MAE); break;
    case LL_RULE_MSE: LL_LAUNCH_Q(LL_RULE_MSE); break;
    default: LL_LAUNCH_Q(LL_RULE_ABS_MAX); break;
  }
#undef LL_LAUNCH_Q
  LL_CHECK_LAUNCH("quantize_kernel");
  return LL_OK;
}

extern "C" int ll_nvfp4_quantize(const void* x, int64_t M, int64_t K, int64_t ldx, int rule, uint8_t* values,
                                 uint8_t* scales, float* amax, int amax_given, float* workspace, void* stream) {
  const QuantRequest r{x, values, scales, amax, workspace, nullptr};
  return quantize_impl(&r, 1, M, K, ldx, rule, amax_given, stream);
}

// One workgroup of kAmaxParts threads.  Every thread reads the word before anyone writes it, so all agree on
// whether the slots have to be cleared.
__global__ __launch_bounds__(ll::kAmaxParts) void amax_epoch_advance_kernel(uint32_t* epoch_offset, uint32_t step,
                                                                            unsigned long long* parts) {
  const uint32_t current = *epoch_offset;
  __syncthreads();
  const bool restart = current > 0xE0000000u - step;  // epochs stay clear of 2^32 whatever the base epochs are (< 2^28)
  if (restart) parts[threadIdx.x] = 0ull;
  if (threadIdx.x == 0) *epoch_offset = restart ? 0u : current + step;
}

extern "C" int ll_amax_epoch_advance(uint32_t* epoch_offset, uint32_t step, uint64_t* parts, void* stream) {
  LL_REQUIRE(epoch_offset && parts && (reinterpret_cast<uintptr_t>(epoch_offset) & 3) == 0 &&
                 (reinterpret_cast<uintptr_t>(parts) & 7) == 0,
             "ll_amax_epoch_advance: epoch_offset (4-byte aligned) and parts (8-byte aligned) are required");
  LL_REQUIRE(step > 0 && step <= (1u << 28), "ll_amax_epoch_advance: step %u outside 1..2^28", step);
  hipLaunchKernelGGL(amax_epoch_advance_kernel, dim3(1), dim3(ll::kAmaxParts), 0, static_cast<hipStream_t>(stream),
                     epoch_offset, step, reinterpret_cast<unsigned long long*>(parts));
  LL_CHECK_LAUNCH("amax_epoch_advance_kernel");
  return LL_OK;
}

extern "C" int ll_nvfp4_quantize_from_sink(const void* x, int64_t M, int64_t K, int64_t ldx, int rule,
                                           uint8_t* values, uint8_t* scales, float* amax,
                                           const ll_amax_sink* amax_sink, void* stream) {
  using namespace ll;
  LL_REQUIRE(amax_sink, "ll_nvfp4_quantize_from_sink: null amax sink");
  const QuantRequest r{x, values, scales, amax, nullptr, amax_sink};
  return quantize_impl(&r, 1, M, K, ldx, rule, 0, stream);
}

extern "C" int ll_nvfp4_quantize_pair_from_sinks(const void* x0, const void* x1, int64_t M, int64_t K, int64_t ldx,
                                                 int rule, uint8_t* values0, uint8_t* values1, uint8_t* scales0,
                                                 uint8_t* scales1, float* amax0, float* amax1,
                                                 const ll_amax_sink* amax_sink0, const ll_amax_sink* amax_sink1,
                                                 void* stream) {
  using namespace ll;
  LL_REQUIRE(amax_sink0 && amax_sink1, "ll_nvfp4_quantize_pair_from_sinks: null amax sink");
  LL_REQUIRE(values0 != values1 && scales0 != scales1 && amax0 != amax1,
             "ll_nvfp4_quantize_pair_from_sinks: the two tensors need outputs of their own");
  const QuantRequest r[2] = {{x0, values0, scales0, amax0, nullptr, amax_sink0},
                             {x1, values1, scales1, amax1, nullptr, amax_sink1}};
  return quantize_impl(r, 2, M, K, ldx, rule, 0, stream);
}

// ----------------------------------------------------------------------------- entry point that allocates nothing
// ll_nvfp4_quantize needs kAmaxParts floats of device scratch for the partial maxima of its amax pass.  For callers
// that cannot allocate, the same floats exist once per GPU as a file-scope device array.  In host code the array's
// name is only a handle: its device address is looked up once per device (hipGetSymbolAddress, with that device
// current) and kept; kernels receive that address like any other workspace pointer.
static __device__ __align__(256) float scratch[LL_AMAX_PARTS];

namespace {
constexpr int kMaxDevices = 64;
std::atomic<float*> g_scratch_ptr[kMaxDevices];

int scratch_address(float** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    ll::set_error("ll_nvfp4_quantize_noalloc: hipGetDevice failed: %s", hipGetErrorString(e));
    return LL_ELAUNCH;
  }
  if (dev < 0 || dev >= kMaxDevices) {
    ll::set_error("ll_nvfp4_quantize_noalloc: device ordinal %d not supported (at most %d devices)", dev, kMaxDevices);
    return LL_ENOSUP;
  }
  float* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    void* addr = nullptr;
    e = hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !addr) {
      ll::set_error("ll_nvfp4_quantize_noalloc: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
      return LL_ELAUNCH;
    }
    p = static_cast<float*>(addr);
    g_scratch_ptr[dev].store(p, std::memory_order_release);  // racing threads store the same address
  }
  *out = p;
  return LL_OK;
}
}  // namespace

extern "C" int64_t ll_nvfp4_quantize_noalloc_max_elements(void) { return LL_NOALLOC_MAX_ELEMENTS; }

extern "C" int ll_nvfp4_quantize_noalloc(const void* x, int64_t M, int64_t K, int64_t ldx, int rule, uint8_t* values,
                                         uint8_t* scales, float* amax, void* stream) {
  using namespace ll;
  LL_REQUIRE(M > 0 && K > 0, "ll_nvfp4_quantize_noalloc: bad shape M=%lld K=%lld", (long long)M, (long long)K);
  LL_REQUIRE(K <= LL_NOALLOC_MAX_ELEMENTS && M <= LL_NOALLOC_MAX_ELEMENTS / K,
             "ll_nvfp4_quantize_noalloc: %lld x %lld elements exceed the limit of %lld of this entry point; use "
             "ll_nvfp4_quantize with a caller-provided workspace",
             (long long)M, (long long)K, (long long)LL_NOALLOC_MAX_ELEMENTS);
  float* ws = nullptr;
  if (int rc = scratch_address(&ws)) return rc;
  const QuantRequest r{x, values, scales, amax, ws, nullptr};
  return quantize_impl(&r, 1, M, K, ldx, rule, 0, stream);
}
