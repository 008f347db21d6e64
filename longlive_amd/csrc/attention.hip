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
// (e2m1 x e4m3 x amax/(6*256) -> bf16, the values the reference's dequantized bf16 cache holds) into LDS:
// K row-major, V transposed.  The MFMAs compute S^T = K Q^T and O^T = V^T P^T (v_mfma_f32_32x32x16_bf16), so
// every lane owns one query column: row max / row sum need no cross-lane traffic beyond one swap between the
// wave halves, and the online-softmax rescale is a per-lane scalar.
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
constexpr int kVPitch = 136;                   // bytes per d row of V^T in LDS (128 + 8 pad)
constexpr int kKTileBytes = kTileKeys * kKPitch;
constexpr int kVTileBytes = kHeadDim * kVPitch;
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

__device__ __forceinline__ float fp8_byte_to_f32(uint32_t word, int byte) {
  typedef float float2v_ __attribute__((ext_vector_type(2)));
  const float2v_ lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)word, false);
  const float2v_ hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)word, true);
  return byte == 0 ? lo[0] : byte == 1 ? lo[1] : byte == 2 ? hi[0] : hi[1];
}

// 8 e2m1 codes (one dword) times sf -> 8 floats
__device__ __forceinline__ void fp4x8_to_f32(uint32_t w, float sf, float (&o)[8]) {
  const float2v q0 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 0);
  const float2v q1 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 1);
  const float2v q2 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 2);
  const float2v q3 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 3);
  o[0] = q0[0] * sf; o[1] = q0[1] * sf; o[2] = q1[0] * sf; o[3] = q1[1] * sf;
  o[4] = q2[0] * sf; o[5] = q2[1] * sf; o[6] = q3[0] * sf; o[7] = q3[1] * sf;
}

// Raw FP4 data prefetched one iteration ahead.  Only packed bytes and scale bytes are held in registers
// across the MFMA phase; everything else (slot scale, kind of key, bf16 source rows of the current chunk)
// is re-derived from the key index when the data is decoded.
struct KRaw {         // K of one key, one quarter of the head dimension (32 elements)
  uint4 v;            // 16 packed bytes
  uint32_t scales;    // 2 e4m3 block scales (low 16 bits)
};
struct VRaw {         // V of one key, half a 16-element block
  uint32_t v;         // 4 packed bytes
  uint32_t scale;     // e4m3 block scale byte
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
__device__ __forceinline__ void fetch_k(const SlotTable& tab, int slot, uint32_t vo, uint32_t so, KRaw& f) {
  f.v = load_global_b128(tab.kv[slot] + vo);
  f.scales = load_global<uint16_t>(tab.ks[slot] + so);
}
__device__ __forceinline__ void fetch_v(const SlotTable& tab, int slot, uint32_t vo, uint32_t so, VRaw& f) {
  f.v = load_global<uint32_t>(tab.vv[slot] + vo);
  f.scale = load_global<uint8_t>(tab.vs[slot] + so);
}

// Decode K (32 elements of one key) to bf16 and store the 64 bytes into the key's LDS row.
// kind: 0 = fp4 slot data in f (gs = slot amax / (e2m1_max * e4m3_max)), 1 = bf16 row at src, 2 = zeros.
__device__ __forceinline__ void store_k(const KRaw& f, int kind, float gs, const uint4* src, uint8_t* dst) {
  uint4* d4 = reinterpret_cast<uint4*>(dst);
  if (kind == 0) {
    const uint32_t w[4] = {f.v.x, f.v.y, f.v.z, f.v.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float sf = fp8_byte_to_f32(f.scales, j >> 1) * gs;
      float v8[8];
      fp4x8_to_f32(w[j], sf, v8);
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

// 8 head-dim elements of 4 consecutive keys -> for every element one 8-byte run of 4 bf16 along the key
// axis, written into the transposed V tile.  vt_tile points at the tile, row0 = first d row.
// kind / gs / src per key as in store_k (src = the key's 8 bf16 elements).
__device__ __forceinline__ void store_v4(const VRaw (&f)[4], const int (&kind)[4], const float (&gs)[4],
                                         const uint4* const (&src)[4], uint8_t* vt_tile, int row0, int chunk) {
  uint32_t w[4][4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) {
    if (kind[kk] == 0) {
      const float sf = fp8_byte_to_f32(f[kk].scale, 0) * gs[kk];
      float v8[8];
      fp4x8_to_f32(f[kk].v, sf, v8);
#pragma unroll
      for (int i = 0; i < 4; ++i) w[kk][i] = pack_bf16(v8[2 * i], v8[2 * i + 1]);
    } else if (kind[kk] == 1) {
      const uint4 a = src[kk][0];
      w[kk][0] = a.x; w[kk][1] = a.y; w[kk][2] = a.z; w[kk][3] = a.w;
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) w[kk][i] = 0;
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t e01 = __builtin_amdgcn_perm(w[1][i], w[0][i], 0x05040100u);
    const uint32_t e23 = __builtin_amdgcn_perm(w[3][i], w[2][i], 0x05040100u);
    const uint32_t o01 = __builtin_amdgcn_perm(w[1][i], w[0][i], 0x07060302u);
    const uint32_t o23 = __builtin_amdgcn_perm(w[3][i], w[2][i], 0x07060302u);
    *reinterpret_cast<uint2*>(vt_tile + (row0 + 2 * i) * kVPitch + chunk * 8) = make_uint2(e01, e23);
    *reinterpret_cast<uint2*>(vt_tile + (row0 + 2 * i + 1) * kVPitch + chunk * 8) = make_uint2(o01, o23);
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

  // ---- decode plan.  K: thread = (key_local = tid / 4, quarter of the head dim = tid % 4).
  //                    V: key tile = wave / 4; a thread owns 8 elements (half lane / 32 of the 16-element
  //                       block 2 (wave % 4) + lane / 16 % 2) of 4 consecutive keys 4 (lane % 16): for one
  //                       head-dim row 16 lanes write one full 128-byte row of V^T, which the 136-byte pitch
  //                       spreads over all LDS banks.
  // Schedule of iteration `it`: the MFMAs work on LDS stage it & 1 while the raw FP4 bytes of iteration
  // it + 1 (already in registers) are decoded into the other stage during the S phase.  As soon as the raw
  // registers are free the bytes of iteration it + 2 are requested, which gives each load most of an
  // iteration to land.  Position of the data the raw registers hold (or will hold next): iter_base = first
  // key of that iteration; per thread the K key iter_base + k_local and the four V keys
  // iter_base + v_local + 0..3, each as (slot, offset in slot) plus the byte offsets of its packed values and
  // scale(s) in the slot.
  KRaw kf;
  VRaw vf[4];
  const int n_cached = (int)p.n_cached, Lk_i = (int)(p.n_cached + p.n_new);
  // lanes 0-31 of a wave (one pass of an 8-byte LDS write) get rows 16 apart = 32 banks apart
  const int v_blk = 2 * (wave & 3) + ((lane >> 4) & 1), v_half = lane >> 5;
  const int v_chunk = lane & 15, v_tile = wave >> 2;
  const int k_local = tid >> 2, k_quarter = tid & 3, v_local = v_tile * kTileKeys + 4 * v_chunk;
  const uint32_t row_bytes = (uint32_t)p.H * 64u;
  const uint32_t step_vo = (uint32_t)kIterKeys * row_bytes;
  const uint32_t step_so = (uint32_t)p.H * 1024u;
  const uint32_t slot_bytes = (uint32_t)p.bts * row_bytes;
  const int k_dst_off = (k_local >> 6) * kKTileBytes + (k_local & 63) * kKPitch + k_quarter * 64;
  const int v_row0 = v_blk * 16 + v_half * 8;
  const int v_dst_off = 2 * kKTileBytes + v_tile * kVTileBytes + v_row0 * kVPitch + v_chunk * 8;
  int iter_base = 0;
  int k_slot = k_local / p.bts, k_off = k_local - k_slot * p.bts;
  int v_slot = v_local / p.bts, v_off = v_local - v_slot * p.bts;
  uint32_t k_vo, k_so, v_vo, v_so[4];
  float k_gs, v_gs[4];  // slot scale amax / (e2m1_max * e4m3_max) of the thread's K key and of its four V keys
  auto locate_k = [&]() __attribute__((always_inline)) {
    const int64_t row = (int64_t)k_off * p.H + head;
    k_vo = (uint32_t)row * 64u + k_quarter * 16u;
    k_so = (uint32_t)blocked_scale_offset(row, k_quarter * 2, 8);
    k_gs = tab.kg[min(k_slot, kMaxSlots - 1)];
  };
  auto locate_v = [&]() __attribute__((always_inline)) {
    v_vo = ((uint32_t)v_off * p.H + head) * 64u + v_blk * 8u + v_half * 4u;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      int oo = v_off + kk;
      if (oo >= p.bts) oo -= p.bts;
      v_so[kk] = (uint32_t)blocked_scale_offset((int64_t)oo * p.H + head, v_blk, 8);
      v_gs[kk] = tab.vg[min(v_slot + (v_off + kk >= p.bts ? 1 : 0), kMaxSlots - 1)];
    }
  };
  locate_k();
  locate_v();
  auto fetch_k_next = [&]() __attribute__((always_inline)) {
    if (iter_base + k_local < n_cached) fetch_k(tab, k_slot, k_vo, k_so, kf);
  };
  auto fetch_v_next = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      const bool wrap = v_off + kk >= p.bts;
      if (iter_base + v_local + kk < n_cached)
        fetch_v(tab, v_slot + (wrap ? 1 : 0), v_vo + kk * row_bytes - (wrap ? slot_bytes : 0u), v_so[kk], vf[kk]);
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
      locate_k();
    }
    v_off += kIterKeys;
    v_vo += step_vo;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) v_so[kk] += step_so;
    if (v_off + 3 >= p.bts) {
      while (v_off >= p.bts) {
        v_off -= p.bts;
        ++v_slot;
      }
      locate_v();
    }
  };
  auto decode_k_any = [&](int stage) __attribute__((always_inline)) {
    const int k_key = iter_base + k_local;
    const int kind = k_key < n_cached ? 0 : (k_key < Lk_i ? 1 : 2);
    const float gs = kind == 0 ? k_gs : 0.0f;
    const uint4* src = reinterpret_cast<const uint4*>(
        p.k_new + ((int64_t)(k_key - n_cached) * p.H + head) * kHeadDim + k_quarter * 32);
    store_k(kf, kind, gs, src, smem + stage * kStageBytes + k_dst_off);
  };
  auto decode_v_any = [&](int stage) __attribute__((always_inline)) {
    int kind[4];
    float gs[4];
    const uint4* src[4];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      const int key = iter_base + v_local + kk;
      kind[kk] = key < n_cached ? 0 : (key < Lk_i ? 1 : 2);
      gs[kk] = kind[kk] == 0 ? v_gs[kk] : 0.0f;
      src[kk] = reinterpret_cast<const uint4*>(p.v_new + ((int64_t)(key - n_cached) * p.H + head) * kHeadDim + v_row0);
    }
    store_v4(vf, kind, gs, src, smem + stage * kStageBytes + 2 * kKTileBytes + v_tile * kVTileBytes, v_row0, v_chunk);
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
    auto read_v = [&](int step, uint2 (&dst)[4][2]) __attribute__((always_inline)) {
      const int chunk0 = (step >> 1) * 8 + (step & 1) * 4 + lh;
#pragma unroll
      for (int dt = 0; dt < 4; ++dt) {
        const uint8_t* src = vt_base + (dt * 32 + l32) * kVPitch;
        dst[dt][0] = *reinterpret_cast<const uint2*>(src + chunk0 * 8);
        dst[dt][1] = *reinterpret_cast<const uint2*>(src + (chunk0 + 2) * 8);
      }
    };
    bf16x8 pb[2];
    uint2 vfr[2][4][2];
    read_v(0, vfr[0]);
    make_p(0, pb[0]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int step = 0; step < 4; ++step) {
      if (step < 3) read_v(step + 1, vfr[(step + 1) & 1]);
#pragma unroll
      for (int dt = 0; dt < 4; ++dt) {
        const uint2(&v)[2] = vfr[step & 1][dt];
        const bf16x8 a = __builtin_bit_cast(bf16x8, make_uint4(v[0].x, v[0].y, v[1].x, v[1].y));
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
  fetch_k_next();
  fetch_v_next();
  decode_k_any(0);
  decode_v_any(0);
  advance();
  if (n_iter > 1) {
    fetch_k_next();
    fetch_v_next();
  }
  __syncthreads();
  // Every load issued so far (Q fragments, first tiles) has to have landed before the loop: otherwise the
  // compiler's wait-count bookkeeping carries them into the loop and makes the MFMA phase wait for the
  // prefetch loads it has just issued.  0x0F70 = vmcnt(0), other counters untouched.
  __builtin_amdgcn_s_waitcnt(0x0F70);

  // Iterations whose own 128 keys all exist and whose successor is all FP4 form a prefix of the key range;
  // they run the interleaved body: S^T (64 keys x 32 queries) = 16 MFMAs in eight steps of two, each step
  // also converting one dword of the prefetched K row (even steps) or two elements of the prefetched V data
  // for four keys (odd steps) into the other LDS stage.  The rest (the bf16 chunk, the tail) runs the plain
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
      const float gsk = k_gs;
      float sfv[4];
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) sfv[kk] = fp8_byte_to_f32(vf[kk].scale, 0) * v_gs[kk];
      const uint32_t w[4] = {kf.v.x, kf.v.y, kf.v.z, kf.v.w};
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
        if ((ks & 1) == 0) {  // K: dword ks / 2 of the quarter row
          const int j = ks >> 1;
          const float sf = fp8_byte_to_f32(kf.scales, j >> 1) * gsk;
          float v8[8];
          fp4x8_to_f32(w[j], sf, v8);
          reinterpret_cast<uint4*>(kdst)[j] = make_uint4(pack_bf16(v8[0], v8[1]), pack_bf16(v8[2], v8[3]),
                                                          pack_bf16(v8[4], v8[5]), pack_bf16(v8[6], v8[7]));
        } else {  // V: elements 2 j, 2 j + 1 of the thread's 8, for its 4 keys -> two rows of V^T
          const int j = ks >> 1;
          float e[4][2];
#pragma unroll
          for (int kk = 0; kk < 4; ++kk) {
            float2v q;
            switch (j) {
              case 0: q = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(vf[kk].v, 1.0f, 0); break;
              case 1: q = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(vf[kk].v, 1.0f, 1); break;
              case 2: q = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(vf[kk].v, 1.0f, 2); break;
              default: q = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(vf[kk].v, 1.0f, 3); break;
            }
            e[kk][0] = q[0] * sfv[kk];
            e[kk][1] = q[1] * sfv[kk];
          }
#pragma unroll
          for (int jj = 0; jj < 2; ++jj)
            *reinterpret_cast<uint2*>(vdst + (2 * j + jj) * kVPitch) =
                make_uint2(pack_bf16(e[0][jj], e[1][jj]), pack_bf16(e[2][jj], e[3][jj]));
        }
        a0 = n0;
        a1 = n1;
      }
    }
    advance();
    if (has_next2) {
      fetch_k_next();
      fetch_v_next();
    }
    softmax_pv(sc, vt_base);
    __syncthreads();
  }

  // Plain body: the S phase without interleaved conversion, masking in the last tile, and the successor tile
  // decoded after the MFMAs (or, for the chunk's own bf16 tiles, brought in ahead of them).
  typedef __attribute__((address_space(1))) const void* gptr_t;
  typedef __attribute__((address_space(3))) void* lptr_t;
  for (; it < n_iter; ++it) {
    const uint8_t* cur = smem + (it & 1) * kStageBytes;
    const uint8_t* vt_base = cur + 2 * kKTileBytes + kp * kVTileBytes;
    const int tile_base = it * kIterKeys + kp * kTileKeys;
    // A successor that lies wholly in the bf16 chunk is brought in ahead of the MFMAs: its K rows go
    // straight from global memory into the other stage (one 256-byte row per wave instruction, 16 rows per
    // wave), its V pieces are requested now and transposed into LDS after the PV phase.
    const bool next_is_chunk = iter_base >= n_cached && iter_base + kIterKeys <= Lk_i;  // iter_base = first key of tile it + 1
    uint4 vraw[4];
    if (next_is_chunk) {
      uint8_t* nxt = smem + ((it + 1) & 1) * kStageBytes;
      const uint16_t* ksrc = p.k_new + ((int64_t)(iter_base + wave * 16 - n_cached) * p.H + head) * kHeadDim + lane * 2;
      uint8_t* kdst = nxt + (wave >> 2) * kKTileBytes + ((wave & 3) * 16) * kKPitch;
#pragma unroll
      for (int r = 0; r < 16; ++r)
        __builtin_amdgcn_global_load_lds((gptr_t)(ksrc + (int64_t)r * p.H * kHeadDim), (lptr_t)(kdst + r * kKPitch), 4, 0, 0);
#pragma unroll
      for (int kk = 0; kk < 4; ++kk)
        vraw[kk] = load_global_b128(p.v_new + ((int64_t)(iter_base + v_local + kk - n_cached) * p.H + head) * kHeadDim + v_row0);
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
      uint8_t* vdst = smem + ((it + 1) & 1) * kStageBytes + v_dst_off;
      const uint32_t w[4][4] = {{vraw[0].x, vraw[0].y, vraw[0].z, vraw[0].w}, {vraw[1].x, vraw[1].y, vraw[1].z, vraw[1].w},
                                {vraw[2].x, vraw[2].y, vraw[2].z, vraw[2].w}, {vraw[3].x, vraw[3].y, vraw[3].z, vraw[3].w}};
#pragma unroll
      for (int i = 0; i < 4; ++i) {  // elements 2 i, 2 i + 1 of the thread's 8, for its 4 keys -> two rows of V^T
        // v_perm_b32: bytes 0-3 come from the second operand, 4-7 from the first
        *reinterpret_cast<uint2*>(vdst + (2 * i) * kVPitch) =
            make_uint2(__builtin_amdgcn_perm(w[1][i], w[0][i], 0x05040100u), __builtin_amdgcn_perm(w[3][i], w[2][i], 0x05040100u));
        *reinterpret_cast<uint2*>(vdst + (2 * i + 1) * kVPitch) =
            make_uint2(__builtin_amdgcn_perm(w[1][i], w[0][i], 0x07060302u), __builtin_amdgcn_perm(w[3][i], w[2][i], 0x07060302u));
      }
      iter_base += kIterKeys;  // the slot bookkeeping of advance() has no use beyond the cache
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the K rows have landed in LDS
    } else if (it + 1 < n_iter) {
      decode_k_any((it + 1) & 1);
      decode_v_any((it + 1) & 1);
      advance();
      if (it + 2 < n_iter) {
        fetch_k_next();
        fetch_v_next();
      }
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
  static bool configured = false;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&kv_attention_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) {
      set_error("ll_kv_attention: cannot reserve %zu bytes of LDS: %s", smem, hipGetErrorString(e));
      return LL_ELAUNCH;
    }
    configured = true;
  }
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
  p.inv_denom = n_cached > 0 ? 1.0f / (e2m1_max * e4m3_max) : 0.f;
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
