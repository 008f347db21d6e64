// Chunk attention over an NVFP4 KV cache for gfx950, with the dequantization fused into the K/V tile
// load:  out = softmax(q k^T * scale) v  over  [ cached tokens (FP4 slots) | current chunk (bf16) ].
//
// Replaces "dequantize the whole cache to bf16, copy the chunk in, call flash attention"
// (wan_5b/modules/causal_model.py:557-567, 628-671, 781; utils/quant.py:731-768).
//
// Workgroup = one head x 128 queries, 8 waves = two per SIMD.  Wave w owns 32 queries (w & 3) and every
// second 64-key tile (w >> 2); the two halves of the key range are merged at the end.  A wave needs at most
// 256 registers (64 for O^T, 32 for S^T, 32 for its Q fragments, the rest for tile fragments, raw FP4 data
// and addressing), which is what lets two waves share a SIMD: while one wave converts FP4 data or evaluates
// exponentials, the other one's MFMAs run.  Per iteration all 512 threads decode 128 keys of K and V
// ((e2m1 x e4m3) x slot scale -> bf16: bit for bit the values the reference's fused cache dequantization and
// ll_kv_dequantize_blocks produce, utils/kernel/kv_dequant_cuda.cu:95-106) into LDS, both
// row-major (one row per key), with the same thread layout and the same byte offsets for K and V.  The MFMAs
// compute S^T = K Q^T and O^T = V^T P^T (v_mfma_f32_32x32x16_bf16), so every lane owns one query column: row max /
// row sum need no cross-lane traffic beyond one swap between the wave halves, and the online-softmax rescale is
// a per-lane scalar.  The V^T operand (a lane needs eight consecutive keys of one head-dim column) comes out of
// the row-major tile through ds_read_b64_tr_b16, the LDS read that transposes 16-bit elements across 16 lanes.
#include "ll_common.h"

namespace ll {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef float float2v __attribute__((ext_vector_type(2)));

constexpr int kHeadDim = 128;
constexpr int kTileKeys = 64;                  // keys per wave tile
constexpr int kIterKeys = 2 * kTileKeys;       // keys decoded per iteration (one tile per key-parity)
constexpr int kWgQueries = 128;
constexpr int kWaveQueries = 32;
constexpr int kKPitch = 272;                   // bytes per key row of K in LDS (256 + 16 pad)
constexpr int kVPitch = 288;                   // bytes per key row of V in LDS (256 + 32 pad: four rows of a transposing read hit 32 different banks)
constexpr int kKTileBytes = kTileKeys * kKPitch;
constexpr int kVTileBytes = kTileKeys * kVPitch;
constexpr int kStageBytes = 2 * kKTileBytes + 2 * kVTileBytes;
constexpr int kMaxSlots = 64;
constexpr int kAttnThreads = 512;

struct AttnParams {
  const uint16_t* q;
  int64_t Lq;
  int H;
  const uint64_t *kv_ptrs, *ks_ptrs, *ka_ptrs, *vv_ptrs, *vs_ptrs, *va_ptrs;
  int64_t n_cached, n_new;
  int bts, n_slots;
  float inv_denom;
  const uint16_t *k_new, *v_new;
  float scale_log2;  // softmax scale * log2(e)
  uint16_t* out;
  AmaxSink sink;  // receives max |out| when sink.parts is not null
  int n_qtiles;
};

struct SlotTable {
  const uint8_t* kv[kMaxSlots];
  const uint8_t* ks[kMaxSlots];
  const uint8_t* vv[kMaxSlots];
  const uint8_t* vs[kMaxSlots];
  float kg[kMaxSlots];
  float vg[kMaxSlots];
};

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) { return pack_bf16x2(a, b); }

// max(v[lane], v[lane ^ 32]) in every lane: one v_permlane32_swap (register file only) instead of a
// permute through LDS, whose result would also wait for every LDS read issued before it.
__device__ __forceinline__ float max_over_wave_halves(float v) {
  const uint32_t u = __float_as_uint(v);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);  // r[0] = lower half twice, r[1] = upper half twice
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

typedef _Float16 half2v __attribute__((ext_vector_type(2)));

// The two e4m3 block scales in the low 16 bits of `word`, as f16 pairs (s, s) ready for a packed multiply.
__device__ __forceinline__ void block_scales_f16(uint32_t word, half2v (&s2)[2]) {
  const half2v sc = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(word, 1.0f, false);
  s2[0] = half2v{sc[0], sc[0]};
  s2[1] = half2v{sc[1], sc[1]};
}

// f32(t.lo) * g and f32(t.hi) * g with one instruction each: the mixed-precision fused multiply-add widens
// the selected f16 half on the way in (op_sel_hi marks source 0 as f16, op_sel picks its upper half).  The
// addend is -0, which leaves the product untouched, signed zeros included.
__device__ __forceinline__ float widen_mul_lo(half2v t, float g) {
  float r;
  asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel_hi:[1,0,0]" : "=v"(r) : "v"(t), "v"(g), "s"(-0.0f));
  return r;
}
__device__ __forceinline__ float widen_mul_hi(half2v t, float g) {
  float r;
  asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(r) : "v"(t), "v"(g), "s"(-0.0f));
  return r;
}

// 8 e2m1 codes (one dword) of a block with scale s2 = (s, s) and slot scale gs -> the 8 fp32 values
// (code * s) * gs, the expression of the reference's fused cache dequantization (utils/kernel/kv_dequant_cuda.cu:
// 97-106).  code * s has at most six significant bits and lies within [2^-10, 2688], so the packed f16 product is
// exact; the multiplication by gs is the only rounding, done in fp32.
__device__ __forceinline__ void fp4x8_to_f32(uint32_t w, half2v s2, float gs, float (&o)[8]) {
  const half2v t0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 0) * s2;
  const half2v t1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 1) * s2;
  const half2v t2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 2) * s2;
  const half2v t3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 3) * s2;
  o[0] = widen_mul_lo(t0, gs); o[1] = widen_mul_hi(t0, gs);
  o[2] = widen_mul_lo(t1, gs); o[3] = widen_mul_hi(t1, gs);
  o[4] = widen_mul_lo(t2, gs); o[5] = widen_mul_hi(t2, gs);
  o[6] = widen_mul_lo(t3, gs); o[7] = widen_mul_hi(t3, gs);
}

// Raw FP4 data prefetched one iteration ahead.  Only packed bytes and scale bytes are held in registers
// across the MFMA phase; everything else (slot scale, kind of key, bf16 source rows of the current chunk)
// is re-derived from the key index when the data is decoded.
struct KRaw {         // K or V of one key, one quarter of the head dimension (32 elements)
  uint4 v;            // 16 packed bytes
  uint32_t scales;    // 2 e4m3 block scales (low 16 bits)
};

// Load through a pointer that is known to address global memory.  Slot pointers come out of a table, so
// the compiler would otherwise emit flat loads, whose completion also counts as an LDS event and stalls
// the first LDS wait that follows.
template <typename T>
__device__ __forceinline__ T load_global(const void* ptr) {
  return *(const __attribute__((address_space(1))) T*)ptr;
}
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 load_global_b128(const void* ptr) {
  const u32x4 v = load_global<u32x4>(ptr);
  return make_uint4(v[0], v[1], v[2], v[3]);
}

// Raw FP4 loads.  vo / so are byte offsets of the thread's data inside the slot's value / scale arrays;
// the caller keeps them up to date incrementally (both advance by a constant per iteration inside a slot).
__device__ __forceinline__ void fetch_row(const uint8_t* values, const uint8_t* scales, uint32_t vo, uint32_t so, KRaw& f) {
  f.v = load_global_b128(values + vo);
  f.scales = load_global<uint16_t>(scales + so);
}

// 4 bytes per lane from global memory straight into LDS at lds_base + 4 * lane (lds_base wave-uniform).  An asm
// statement on purpose: for the builtin the compiler's wait-count pass, which cannot tell the two LDS stages apart,
// makes later LDS reads of the *other* stage wait for the load.  The kernel waits for these loads itself
// (vmcnt(0) ahead of the barrier that hands the stage over).
__device__ __forceinline__ void load_to_lds_b32(const void* src, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(src), "s"(lds_base) : "memory");
}
__device__ __forceinline__ uint32_t lds_address(const void* p) {
  return __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)p);
}

// Decode 32 elements of one key (K or V) to bf16 and store the 64 bytes into the key's LDS row.
// kind: 0 = fp4 slot data in f (gs = slot amax * f32(1 / (e2m1_max * e4m3_max))), 1 = bf16 row at src, 2 = zeros.
__device__ __forceinline__ void store_row(const KRaw& f, int kind, float gs, const uint4* src, uint8_t* dst) {
  uint4* d4 = reinterpret_cast<uint4*>(dst);
  if (kind == 0) {
    const uint32_t w[4] = {f.v.x, f.v.y, f.v.z, f.v.w};
    half2v s2[2];
    block_scales_f16(f.scales, s2);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float v8[8];
      fp4x8_to_f32(w[j], s2[j >> 1], gs, v8);
      d4[j] = make_uint4(pack_bf16(v8[0], v8[1]), pack_bf16(v8[2], v8[3]), pack_bf16(v8[4], v8[5]), pack_bf16(v8[6], v8[7]));
    }
  } else if (kind == 1) {
#pragma unroll
    for (int i = 0; i < 4; ++i) d4[i] = src[i];
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) d4[i] = make_uint4(0, 0, 0, 0);
  }
}

__global__ __launch_bounds__(kAttnThreads) void kv_attention_kernel(AttnParams p) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  SlotTable& tab = *reinterpret_cast<SlotTable*>(smem + 2 * kStageBytes);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, lh = lane >> 5;
  const int qq = wave & 3, kp = wave >> 2;  // query quarter (32 queries), key parity

  int wg = blockIdx.x;
  {
    const int total = p.H * p.n_qtiles;
    if (total % 8 == 0) wg = (wg & 7) * (total / 8) + (wg >> 3);
  }
  const int head = wg / p.n_qtiles, qtile = wg - head * p.n_qtiles;

  if (tid < p.n_slots) {
    tab.kv[tid] = reinterpret_cast<const uint8_t*>(p.kv_ptrs[tid]);
    tab.ks[tid] = reinterpret_cast<const uint8_t*>(p.ks_ptrs[tid]);
    tab.vv[tid] = reinterpret_cast<const uint8_t*>(p.vv_ptrs[tid]);
    tab.vs[tid] = reinterpret_cast<const uint8_t*>(p.vs_ptrs[tid]);
    tab.kg[tid] = load_global<float>(reinterpret_cast<const void*>(p.ka_ptrs[tid])) * p.inv_denom;
    tab.vg[tid] = load_global<float>(reinterpret_cast<const void*>(p.va_ptrs[tid])) * p.inv_denom;
  }

  bf16x8 qf[8];
  {
    int64_t query = (int64_t)qtile * kWgQueries + qq * kWaveQueries + l32;
    if (query >= p.Lq) query = p.Lq - 1;
    const uint16_t* src = p.q + (query * p.H + head) * kHeadDim + 8 * lh;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) qf[ks] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(src + 16 * ks));
  }

  float16v o[4];
#pragma unroll
  for (int dt = 0; dt < 4; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[dt][i] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;

  const int n_iter = (int)((p.n_cached + p.n_new + kIterKeys - 1) / kIterKeys);
  __syncthreads();

  // ---- decode plan.  Thread = (key_local = tid / 4, quarter of the head dim = tid % 4), the same for K and V.
  // Schedule of iteration `it`: the MFMAs work on LDS stage it & 1 while the raw FP4 bytes of iteration
  // it + 1 (already in registers) are decoded into the other stage during the S phase.  As soon as the raw
  // registers are free the bytes of iteration it + 2 are requested, which gives each load most of an
  // iteration to land.  Position of the data the raw registers hold (or will hold next): iter_base = first
  // key of that iteration; per thread the key iter_base + k_local as (slot, offset in slot) plus the byte
  // offsets of its packed values and scales in the slot, which K and V share.
  KRaw kf, vf;
  const int n_cached = (int)p.n_cached, Lk_i = (int)(p.n_cached + p.n_new);
  const int k_local = tid >> 2, k_quarter = tid & 3;
  const uint32_t row_bytes = (uint32_t)p.H * 64u;
  const uint32_t step_vo = (uint32_t)kIterKeys * row_bytes;
  const uint32_t step_so = (uint32_t)p.H * 1024u;
  const int k_dst_off = (k_local >> 6) * kKTileBytes + (k_local & 63) * kKPitch + k_quarter * 64;
  const int v_dst_off = 2 * kKTileBytes + (k_local >> 6) * kVTileBytes + (k_local & 63) * kVPitch + k_quarter * 64;
  int iter_base = 0;
  int k_slot = k_local / p.bts, k_off = k_local - k_slot * p.bts;
  uint32_t k_vo, k_so;
  float k_gs, v_gs;  // slot scale amax * f32(1 / (e2m1_max * e4m3_max)) of the thread's key, for K and for V
  auto locate = [&]() __attribute__((always_inline)) {
    const int64_t row = (int64_t)k_off * p.H + head;
    k_vo = (uint32_t)row * 64u + k_quarter * 16u;
    k_so = (uint32_t)blocked_scale_offset(row, k_quarter * 2, 8);
    k_gs = tab.kg[min(k_slot, kMaxSlots - 1)];
    v_gs = tab.vg[min(k_slot, kMaxSlots - 1)];
  };
  locate();
  auto fetch_next = [&]() __attribute__((always_inline)) {
    if (iter_base + k_local < n_cached) {
      fetch_row(tab.kv[k_slot], tab.ks[k_slot], k_vo, k_so, kf);
      fetch_row(tab.vv[k_slot], tab.vs[k_slot], k_vo, k_so, vf);
    }
  };
  auto advance = [&]() __attribute__((always_inline)) {
    iter_base += kIterKeys;
    k_off += kIterKeys;
    k_vo += step_vo;
    k_so += step_so;
    if (k_off >= p.bts) {
      do {
        k_off -= p.bts;
        ++k_slot;
      } while (k_off >= p.bts);
      locate();
    }
  };
  auto decode_any = [&](int stage) __attribute__((always_inline)) {
    const int key = iter_base + k_local;
    const int kind = key < n_cached ? 0 : (key < Lk_i ? 1 : 2);
    const int64_t src_off = ((int64_t)(key - n_cached) * p.H + head) * kHeadDim + k_quarter * 32;
    store_row(kf, kind, k_gs, reinterpret_cast<const uint4*>(p.k_new + src_off), smem + stage * kStageBytes + k_dst_off);
    store_row(vf, kind, v_gs, reinterpret_cast<const uint4*>(p.v_new + src_off), smem + stage * kStageBytes + v_dst_off);
  };

  // Reference point of the exponentials.  m_run is not the exact running maximum: it is raised only when
  // the maximum has grown by more than kRescaleStep (in the exp2 domain) since it was last raised, so P can
  // reach 2^kRescaleStep instead of 1 (harmless in fp32 / bf16) and the 64 accumulator registers per lane
  // are rescaled a handful of times per kernel instead of at almost every tile.  The final division by
  // the row sum, which is accumulated against the same reference, makes the result independent of it.
  constexpr float kRescaleStep = 8.0f;

  // Second half of an iteration: reference point of the exponentials over the wave's 64 keys (S^T in sc:
  // register r of tile kt <-> key 32 kt + 8 (r / 4) + 4 lh + r % 4), then the PV phase in four steps of 16
  // keys, the exponentials of step j + 1 computed under the four MFMAs of step j.
  auto softmax_pv = [&](float16v (&sc)[2], const uint8_t* vt_base) __attribute__((always_inline)) {
    float neg;
    {
      float mx = sc[0][0];
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, sc[kt][r]);
      mx = max_over_wave_halves(mx);
      const bool raise = (mx - m_run) * p.scale_log2 > kRescaleStep;
      const float m_new = raise ? mx : m_run;
      const float alpha = raise ? __builtin_amdgcn_exp2f((m_run - m_new) * p.scale_log2) : 1.0f;
      neg = -m_new * p.scale_log2;
      m_run = m_new;
      if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
        l_run *= alpha;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
          for (int i = 0; i < 16; ++i) o[dt][i] *= alpha;
      }
    }
    float sum = 0.0f;
    auto make_p = [&](int step, bf16x8& dst) __attribute__((always_inline)) {
      const int kt = step >> 1, hf = step & 1;
      uint32_t w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p0 = __builtin_amdgcn_exp2f(fmaf(sc[kt][8 * hf + 2 * i], p.scale_log2, neg));
        const float p1 = __builtin_amdgcn_exp2f(fmaf(sc[kt][8 * hf + 2 * i + 1], p.scale_log2, neg));
        sum += p0 + p1;
        w[i] = pack_bf16(p0, p1);
      }
      dst = __builtin_bit_cast(bf16x8, make_uint4(w[0], w[1], w[2], w[3]));
    };
    // V^T fragment of step `step` (16 keys), head-dim tile dt: lane l needs column d = 32 dt + l % 32 for the keys
    // 16 step + 8 j + 4 (l / 32) + 0..3 (j = 0, 1: the order of P's registers).  One transposing read serves a
    // 16-lane group: source lane i points at row key0 + i / 4, columns d0 + 4 (i % 4) .. + 3, and every lane of
    // the group receives column d0 + i of the four rows.
    typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) bf16x4* lds_bf16x4_t;
    const uint8_t* vt_lane = vt_base + (4 * lh + ((lane & 15) >> 2)) * kVPitch + (16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;
    auto read_v = [&](int step, bf16x4 (&dst)[4][2]) __attribute__((always_inline)) {
#pragma unroll
      for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          dst[dt][j] = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
              (lds_bf16x4_t)(vt_lane + (16 * step + 8 * j) * kVPitch + dt * 64));
    };
    bf16x8 pb[2];
    bf16x4 vfr[2][4][2];
    read_v(0, vfr[0]);
    make_p(0, pb[0]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int step = 0; step < 4; ++step) {
      if (step < 3) read_v(step + 1, vfr[(step + 1) & 1]);
#pragma unroll
      for (int dt = 0; dt < 4; ++dt) {
        const bf16x4(&v)[2] = vfr[step & 1][dt];
        const bf16x8 a = __builtin_shufflevector(v[0], v[1], 0, 1, 2, 3, 4, 5, 6, 7);
        o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pb[step & 1], o[dt], 0, 0, 0);
      }
      if (step < 3) {
        make_p(step + 1, pb[(step + 1) & 1]);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
          __builtin_amdgcn_sched_group_barrier(0x400, 2, 0);  // two exponentials
          __builtin_amdgcn_sched_group_barrier(0x002, 5, 0);  // their multiply-adds, sums and packing
        }
      }
    }
    l_run += sum;
  };

  // prologue: stage 0 <- iteration 0, raw registers <- iteration 1
  fetch_next();
  decode_any(0);
  advance();
  if (n_iter > 1) fetch_next();
  __syncthreads();
  // Every load issued so far (Q fragments, first tiles) has to have landed before the loop: otherwise the
  // compiler's wait-count bookkeeping carries them into the loop and makes the MFMA phase wait for the
  // prefetch loads it has just issued.  0x0F70 = vmcnt(0), other counters untouched.
  __builtin_amdgcn_s_waitcnt(0x0F70);

  // Iterations whose own 128 keys all exist and whose successor is all FP4 form a prefix of the key range;
  // they run the interleaved body: S^T (64 keys x 32 queries) = 16 MFMAs in eight steps of two, each step
  // also converting one dword of the prefetched K row (even steps) or V row (odd steps) into the other LDS
  // stage.  The rest (the bf16 chunk, the tail) runs the plain
  // body in a loop of its own.
  int n_fast = n_cached / kIterKeys - 1;
  n_fast = n_fast < 0 ? 0 : (n_fast > n_iter ? n_iter : n_fast);
  int it = 0;
  for (; it < n_fast; ++it) {
    const uint8_t* cur = smem + (it & 1) * kStageBytes;
    uint8_t* nxt = smem + ((it + 1) & 1) * kStageBytes;
    const uint8_t* vt_base = cur + 2 * kKTileBytes + kp * kVTileBytes;
    const bool has_next2 = it + 2 < n_iter;
    float16v sc[2];
    {
      const uint32_t wk[4] = {kf.v.x, kf.v.y, kf.v.z, kf.v.w}, wv[4] = {vf.v.x, vf.v.y, vf.v.z, vf.v.w};
      half2v ks2[2], vs2[2];
      block_scales_f16(kf.scales, ks2);
      block_scales_f16(vf.scales, vs2);
      uint8_t* kdst = nxt + k_dst_off;
      uint8_t* vdst = nxt + v_dst_off;
      const uint8_t* krow0 = cur + kp * kKTileBytes + l32 * kKPitch + lh * 16;
      const uint8_t* krow1 = krow0 + 32 * kKPitch;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) sc[kt][i] = 0.0f;
      uint4 a0 = *reinterpret_cast<const uint4*>(krow0), a1 = *reinterpret_cast<const uint4*>(krow1);
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        uint4 n0 = a0, n1 = a1;
        if (ks < 7) {
          n0 = *reinterpret_cast<const uint4*>(krow0 + (ks + 1) * 32);
          n1 = *reinterpret_cast<const uint4*>(krow1 + (ks + 1) * 32);
        }
        const bf16x8 fa0 = __builtin_bit_cast(bf16x8, a0), fa1 = __builtin_bit_cast(bf16x8, a1);
        sc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa0, qf[ks], sc[0], 0, 0, 0);
        sc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa1, qf[ks], sc[1], 0, 0, 0);
        {  // one dword (8 elements) of the prefetched row per step: K in the even steps, V in the odd ones
          const int j = ks >> 1;
          const bool is_k = (ks & 1) == 0;
          float v8[8];
          fp4x8_to_f32(is_k ? wk[j] : wv[j], is_k ? ks2[j >> 1] : vs2[j >> 1], is_k ? k_gs : v_gs, v8);
          reinterpret_cast<uint4*>(is_k ? kdst : vdst)[j] = make_uint4(pack_bf16(v8[0], v8[1]), pack_bf16(v8[2], v8[3]),
                                                                       pack_bf16(v8[4], v8[5]), pack_bf16(v8[6], v8[7]));
        }
        a0 = n0;
        a1 = n1;
      }
    }
    advance();
    if (has_next2) fetch_next();
    softmax_pv(sc, vt_base);
    __syncthreads();
  }

  // Plain body: the S phase without interleaved conversion, masking in the last tile, and the successor tile
  // decoded after the MFMAs (or, for the chunk's own bf16 tiles, brought in ahead of them).
  for (; it < n_iter; ++it) {
    const uint8_t* cur = smem + (it & 1) * kStageBytes;
    const uint8_t* vt_base = cur + 2 * kKTileBytes + kp * kVTileBytes;
    const int tile_base = it * kIterKeys + kp * kTileKeys;
    // A successor that lies wholly in the bf16 chunk is brought in ahead of the MFMAs: its K rows go
    // and V rows go straight from global memory into the other stage (one 256-byte row per wave instruction,
    // 16 rows of each per wave).
    const bool next_is_chunk = iter_base >= n_cached && iter_base + kIterKeys <= Lk_i;  // iter_base = first key of tile it + 1
    if (next_is_chunk) {
      uint8_t* nxt = smem + ((it + 1) & 1) * kStageBytes;
      const int64_t src_off = ((int64_t)(iter_base + wave * 16 - n_cached) * p.H + head) * kHeadDim + lane * 2;
      const int64_t src_step = (int64_t)p.H * kHeadDim;
      uint8_t* kdst = nxt + (wave >> 2) * kKTileBytes + ((wave & 3) * 16) * kKPitch;
      uint8_t* vdst = nxt + 2 * kKTileBytes + (wave >> 2) * kVTileBytes + ((wave & 3) * 16) * kVPitch;
      const uint32_t kdst_lds = lds_address(kdst), vdst_lds = lds_address(vdst);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        load_to_lds_b32(p.k_new + src_off + r * src_step, kdst_lds + r * kKPitch);
        load_to_lds_b32(p.v_new + src_off + r * src_step, vdst_lds + r * kVPitch);
      }
    }
    if (tile_base < Lk_i) {
      float16v sc[2];
      const uint8_t* krow0 = cur + kp * kKTileBytes + l32 * kKPitch + lh * 16;
      const uint8_t* krow1 = krow0 + 32 * kKPitch;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) sc[kt][i] = 0.0f;
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        const bf16x8 fa0 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(krow0 + ks * 32));
        const bf16x8 fa1 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(krow1 + ks * 32));
        sc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa0, qf[ks], sc[0], 0, 0, 0);
        sc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa1, qf[ks], sc[1], 0, 0, 0);
      }
      if (tile_base + kTileKeys > Lk_i) {
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int key = tile_base + kt * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
            if (key >= Lk_i) sc[kt][r] = -INFINITY;
          }
      }
      softmax_pv(sc, vt_base);
    }
    if (next_is_chunk) {
      iter_base += kIterKeys;  // the slot bookkeeping of advance() has no use beyond the cache
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the rows have landed in LDS
    } else if (it + 1 < n_iter) {
      decode_any((it + 1) & 1);
      advance();
      if (it + 2 < n_iter) fetch_next();
    }
    __syncthreads();
  }

  // ---- merge the two key-parity halves and write out.  Row sums are per wave half so far.
  l_run += __shfl_xor(l_run, 32, 64);
  float* xo = reinterpret_cast<float*>(smem);   // [qq][64 regs][64 lanes]
  float* xm = xo + 4 * 64 * 64;                  // [qq][64]
  float* xl = xm + 4 * 64;
  if (kp == 1) {
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int i = 0; i < 16; ++i) xo[(qq * 64 + dt * 16 + i) * 64 + lane] = o[dt][i];
    xm[qq * 64 + lane] = m_run;
    xl[qq * 64 + lane] = l_run;
  }
  __syncthreads();
  if (kp == 0) {
    float out_max = 0.0f;
    const float m1 = xm[qq * 64 + lane], l1 = xl[qq * 64 + lane];
    const float m = fmaxf(m_run, m1);
    const float a0 = __builtin_amdgcn_exp2f((m_run - m) * p.scale_log2);
    const float a1 = (m1 == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f((m1 - m) * p.scale_log2);
    const float inv_l = 1.0f / (l_run * a0 + l1 * a1);
    const int64_t query = (int64_t)qtile * kWgQueries + qq * kWaveQueries + l32;
    if (query < p.Lq) {
      uint16_t* dst = p.out + (query * p.H + head) * kHeadDim;
#pragma unroll
      for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
          float v[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float o1 = xo[(qq * 64 + dt * 16 + 4 * rg + i) * 64 + lane];
            v[i] = (o[dt][4 * rg + i] * a0 + o1 * a1) * inv_l;
          }
          const int d = dt * 32 + 8 * rg + 4 * lh;
          const uint2 packed = make_uint2(pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]));
          *reinterpret_cast<uint2*>(dst + d) = packed;
          out_max = abs_max_bf16x8(make_uint4(packed.x, packed.y, 0u, 0u), out_max);
        }
    }
    if (p.sink.parts) {
      out_max = wave_max(out_max);
      if (lane == 0) amax_sink_update(p.sink, blockIdx.x * 4 + qq, out_max);
    }
  }
}

static int launch_attention(const AttnParams& p_in, hipStream_t stream) {
  AttnParams p = p_in;
  p.n_qtiles = (int)((p.Lq + kWgQueries - 1) / kWgQueries);
  const size_t smem = 2 * kStageBytes + sizeof(SlotTable);
  static std::atomic<uint64_t> lds_allowed{0};
  if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(&kv_attention_kernel), smem, lds_allowed, "ll_kv_attention")) return rc;
  hipLaunchKernelGGL(kv_attention_kernel, dim3((unsigned)(p.H * p.n_qtiles)), dim3(kAttnThreads), smem, stream, p);
  LL_CHECK_LAUNCH("kv_attention_kernel");
  return LL_OK;
}

}  // namespace ll

extern "C" int ll_kv_attention(const void* q, int64_t Lq, int num_heads, const uint64_t* k_values_ptrs,
                               const uint64_t* k_scales_ptrs, const uint64_t* k_amax_ptrs,
                               const uint64_t* v_values_ptrs, const uint64_t* v_scales_ptrs,
                               const uint64_t* v_amax_ptrs, int64_t n_cached, int block_token_size, float e2m1_max,
                               float e4m3_max, const void* k_new, const void* v_new, int64_t n_new,
                               float softmax_scale, void* out, void* stream) {
  return ll_kv_attention_amax(q, Lq, num_heads, k_values_ptrs, k_scales_ptrs, k_amax_ptrs, v_values_ptrs,
                              v_scales_ptrs, v_amax_ptrs, n_cached, block_token_size, e2m1_max, e4m3_max, k_new, v_new,
                              n_new, softmax_scale, out, nullptr, stream);
}

extern "C" int ll_kv_attention_amax(const void* q, int64_t Lq, int num_heads, const uint64_t* k_values_ptrs,
                                    const uint64_t* k_scales_ptrs, const uint64_t* k_amax_ptrs,
                                    const uint64_t* v_values_ptrs, const uint64_t* v_scales_ptrs,
                                    const uint64_t* v_amax_ptrs, int64_t n_cached, int block_token_size,
                                    float e2m1_max, float e4m3_max, const void* k_new, const void* v_new,
                                    int64_t n_new, float softmax_scale, void* out, const ll_amax_sink* amax_sink,
                                    void* stream) {
  using namespace ll;
  LL_REQUIRE(q && out, "ll_kv_attention: null q/out");
  LL_REQUIRE(Lq > 0 && num_heads > 0 && n_cached >= 0 && n_new >= 0 && n_cached + n_new > 0,
             "ll_kv_attention: bad sizes Lq=%lld H=%d n_cached=%lld n_new=%lld", (long long)Lq, num_heads,
             (long long)n_cached, (long long)n_new);
  LL_REQUIRE(n_new == 0 || (k_new && v_new), "ll_kv_attention: n_new > 0 needs k_new and v_new");
  LL_REQUIRE(n_cached + n_new < (1ll << 30) && Lq < (1ll << 30), "ll_kv_attention: sequence too long");
  int n_slots = 0;
  if (n_cached > 0) {
    LL_REQUIRE(k_values_ptrs && k_scales_ptrs && k_amax_ptrs && v_values_ptrs && v_scales_ptrs && v_amax_ptrs,
               "ll_kv_attention: n_cached > 0 needs the six slot pointer tables");
    LL_REQUIRE(block_token_size >= 4 && e2m1_max > 0.f && e4m3_max > 0.f, "ll_kv_attention: bad slot geometry");
    LL_REQUIRE((int64_t)block_token_size * num_heads * 64 < (1ll << 31), "ll_kv_attention: slot too large");
    LL_REQUIRE(((int64_t)block_token_size * num_heads) % 128 == 0,
               "ll_kv_attention: slot rows (block_token_size*num_heads = %lld) must be a multiple of 128",
               (long long)block_token_size * num_heads);
    n_slots = (int)((n_cached + block_token_size - 1) / block_token_size);
    LL_REQUIRE(n_slots <= kMaxSlots, "ll_kv_attention: at most %d cache slots, got %d", kMaxSlots, n_slots);
  }
  LL_REQUIRE(((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(k_new) |
               reinterpret_cast<uintptr_t>(v_new)) & 15) == 0,
             "ll_kv_attention: q, out, k_new, v_new must be 16-byte aligned");
  AttnParams p{};
  p.q = static_cast<const uint16_t*>(q);
  p.Lq = Lq;
  p.H = num_heads;
  p.kv_ptrs = k_values_ptrs; p.ks_ptrs = k_scales_ptrs; p.ka_ptrs = k_amax_ptrs;
  p.vv_ptrs = v_values_ptrs; p.vs_ptrs = v_scales_ptrs; p.va_ptrs = v_amax_ptrs;
  p.n_cached = n_cached;
  p.n_new = n_new;
  p.bts = n_cached > 0 ? block_token_size : (1 << 30);
  p.n_slots = n_slots;
  p.inv_denom = n_cached > 0 ? kv_inverse_denominator(e2m1_max, e4m3_max) : 0.f;
  p.k_new = static_cast<const uint16_t*>(k_new);
  p.v_new = static_cast<const uint16_t*>(v_new);
  p.scale_log2 = softmax_scale * 1.4426950408889634f;
  p.out = static_cast<uint16_t*>(out);
  if (amax_sink && amax_sink->parts) {
    p.sink.parts = reinterpret_cast<unsigned long long*>(amax_sink->parts);
    p.sink.epoch = amax_sink->epoch;
  }
  return launch_attention(p, static_cast<hipStream_t>(stream));
}

extern "C" int ll_attention_bf16(const void* q, const void* k, const void* v, int64_t Lq, int64_t Lk, int num_heads,
                                 float softmax_scale, void* out, void* stream) {
  return ll_kv_attention(q, Lq, num_heads, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0, 6.f, 256.f, k,
                         v, Lk, softmax_scale, out, stream);
}
