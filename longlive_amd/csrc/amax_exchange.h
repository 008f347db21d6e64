// The workgroups of one resident launch agree on the maximum of a tensor that they produce together: each
// publishes the maximum of its own share into its own slot of an amax sink under the launch's epoch, and each
// waits - a bounded number of looks - until all slots carry that epoch.  A workgroup whose wait runs out (another
// stream may hold compute units for milliseconds, and a workgroup that has not started cannot publish) computes
// the maxima of the missing workgroups' shares itself, through a function the kernel supplies: the same numbers,
// so every workgroup reaches the end with the same result whatever the others do.
#pragma once
#include "ll_common.h"

namespace ll {

struct AmaxExchangeSmem {
  float red[16];                                    // one partial per wave
  float amax;
  int alone;
  unsigned long long missing[kAmaxParts / 64];      // one bit per slot that did not carry the epoch at the last look
};

// Called by every thread of the workgroup (at most 16 waves).  `thread_part`: the thread's share of the maximum of
// this workgroup's share; `slot` < G <= kAmaxParts: this workgroup's slot; `share_max(s)`: the calling thread's
// part of the maximum of the share of workgroup s, evaluated by all threads of the workgroup together (uniform
// control flow) when s is missing.  spin_limit + 1 looks at most; `everything`: skip the wait and compute all
// shares (tests of that path).  Returns the tensor maximum.
template <class ShareMax>
__device__ __forceinline__ float exchange_amax(const AmaxSink& sink, uint32_t G, uint32_t slot, float thread_part,
                                               uint32_t spin_limit, bool everything, AmaxExchangeSmem& sm,
                                               ShareMax&& share_max) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n_waves = (blockDim.x + 63) >> 6;
  const uint32_t epoch = amax_sink_epoch(sink.epoch, sink.epoch_offset);
  auto over_waves = [&](float v) {  // maximum over the workgroup; the value is valid in every thread
    v = wave_max(v);
    __syncthreads();  // the previous use of sm.red is over
    if (lane == 0) sm.red[wave] = v;
    __syncthreads();
    float r = sm.red[0];
    for (int w = 1; w < n_waves; ++w) r = fmaxf(r, sm.red[w]);
    return r;
  };
  const float mine = over_waves(thread_part);
  if (threadIdx.x == 0) amax_sink_update(sink, slot, mine);

  // wave 0 looks at the G slots until all carry this launch's epoch
  if (wave == 0) {
    bool all_here = false;
    float m = 0.0f;
#pragma unroll 1
    for (uint32_t look = 0;; ++look) {
      unsigned long long any_missing = 0ull;
      m = 0.0f;
      for (uint32_t k = 0; k * 64 < G; ++k) {
        const uint32_t s = lane + 64 * k;
        bool here = s >= G;
        if (s < G && !everything) {
          const unsigned long long v = __hip_atomic_load(sink.parts + s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          here = (uint32_t)(v >> 32) == epoch;
          if (here) m = fmaxf(m, __uint_as_float((uint32_t)v));
        }
        const unsigned long long missing = __builtin_amdgcn_ballot_w64(!here);
        if (lane == 0) sm.missing[k] = missing;
        any_missing |= missing;
      }
      if (any_missing == 0ull) {
        all_here = true;
        break;
      }
      if (everything || look >= spin_limit) break;
      __builtin_amdgcn_s_sleep(8);
    }
    m = wave_max(m);
    if (lane == 0) {
      sm.amax = m;
      sm.alone = all_here ? 0 : 1;
    }
  }
  __syncthreads();
  float amax = sm.amax;  // the maximum over the workgroups that have arrived
  if (sm.alone) {        // uniform over the workgroup
    float part = 0.0f;
#pragma unroll 1
    for (uint32_t k = 0; k * 64 < G; ++k) {
      const unsigned long long word = sm.missing[k];
      uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)word), hi = __builtin_amdgcn_readfirstlane((uint32_t)(word >> 32));
#pragma unroll 1
      while ((lo | hi) != 0u) {
        const uint32_t bit = lo != 0u ? (uint32_t)__builtin_ctz(lo) : 32u + (uint32_t)__builtin_ctz(hi);
        if (lo != 0u) lo &= lo - 1u; else hi &= hi - 1u;
        part = fmaxf(part, share_max(64 * k + bit));
      }
    }
    amax = fmaxf(amax, over_waves(part));
  }
  return amax;
}

}  // namespace ll
