// Chunk attention over an NVFP4 KV cache for gfx950, with the dequantization fused into the K/V tile
// load:  out = softmax(q k^T * scale) v  over  [ cached tokens (FP4 slots) | current chunk (bf16) ].
//
// Replaces "dequantize the whole cache to bf16, copy the chunk in, call flash attention"
// (wan_5b/modules/causal_model.py:557-567, 628-671, 781; utils/quant.py:731-768).
//
// A workgroup is 8 waves = two per SIMD, in one of two shapes (template parameter WIDE):
//   * one head x 128 queries: wave w owns 32 queries (w & 3) and every second 64-key tile (w >> 2); the two
//     halves of the key range are merged at the end;
//   * one head x 256 queries: wave w owns 32 queries and walks both 64-key tiles of an iteration, so a decoded
//     tile serves twice as many MFMAs.  A launch of this shape may hand a workgroup whole tiles, parts of the
//     key range of tiles (combined through device memory), or both: attention_split.h.  Where a head's last
//     group of queries fills at most four of the eight waves, the waves without queries do no matrix work and
//     the division counts such a tile as the lighter load it is.
// A wave needs at most 256 registers (64 for O^T, 32 for S^T, 32 for its Q fragments, the rest for tile
// fragments, raw FP4 data and addressing), which is what lets two waves share a SIMD: while one wave converts
// FP4 data or evaluates exponentials, the other one's MFMAs run.  Per iteration all 512 threads decode 128 keys of K and V
// ((e2m1 x e4m3) x slot scale -> bf16: bit for bit the values the reference's fused cache dequantization and
// ll_kv_dequantize_blocks produce, utils/kernel/kv_dequant_cuda.cu:95-106) into LDS, both
// row-major (one row per key), with the same thread layout and the same byte offsets for K and V.  The MFMAs
// compute S^T = K Q^T and O^T = V^T P^T (v_mfma_f32_32x32x16_bf16), so every lane owns one query column: row max /
// row sum need no cross-lane traffic beyond one swap between the wave halves, and the online-softmax rescale is
// a per-lane scalar.  The V^T operand (a lane needs eight consecutive keys of one head-dim column) comes out of
// the row-major tile through ds_read_b64_tr_b16, the LDS read that transposes 16-bit elements across 16 lanes.
#include "ll_common.h"
#include "attention_split.h"

#include <map>
#include <mutex>
#include <utility>

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
constexpr int kPartialFloats = 8 * 66 * 64;    // a workgroup's partial result: per wave 64 O^T registers, reference point and row sum, per lane

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
  int n_qtiles;     // groups of queries per head
  int full_qtiles;  // tile t < H * full_qtiles is (head t / full_qtiles, group t % full_qtiles); the tiles behind are
                    // the heads' last groups, (head t - H * full_qtiles, group full_qtiles)
  // Division of the launch between its d.G workgroups (attention_split.h).  One workgroup per tile is
  // whole_rounds = 1, extra = 0, units = 0; `partials` / `arrivals` serve the split part (256-query kernel only).
  Division d;
  float* partials;  // [2 G] records of kPartialFloats floats
  int* arrivals;    // [tiles] counters, zero between launches
};

struct SlotTable {
  const uint8_t* kv[kMaxSlots];
  const uint8_t* ks[kMaxSlots];
  const uint8_t* vv[kMaxSlots];
  const uint8_t* vs[kMaxSlots];
  float kg[kMaxSlots];
  float vg[kMaxSlots];
  int last_arrival;  // whether this workgroup completed the tile it just left a partial result for
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

// The kernel's arguments, read again from the argument segment at the point of use.  What is needed only between
// two segments of work (output pointers, the split of the units) then occupies no scalar registers during the main
// loops, which need all of them; the empty asm statement keeps the compiler from moving the reads to the kernel's start.
__device__ __forceinline__ const __attribute__((address_space(4))) AttnParams& reread_params() {
  const __attribute__((address_space(4))) AttnParams* a =
      (const __attribute__((address_space(4))) AttnParams*)__builtin_amdgcn_kernarg_segment_ptr();
  asm volatile("" : "+s"(a));
  return *a;
}
// The launch's division as an ordinary value (seven scalar loads from the argument segment).
__device__ __forceinline__ Division division_of(const __attribute__((address_space(4))) AttnParams& c) {
  return Division{c.d.G, c.d.whole_rounds, c.d.extra, c.d.n_iter, c.d.units, c.d.full_units, c.d.light};
}
// threadIdx.x as a value the compiler knows nothing about: what is derived from it inside a segment's prologue or
// epilogue is then computed there, and not ahead of the loop over segments, where it would occupy registers
// throughout the main loops.
__device__ __forceinline__ int fresh_thread_index() {
  int t = threadIdx.x;
  asm volatile("" : "+v"(t));
  return t;
}
// Partial results travel between workgroups on different XCDs, whose L2 caches do not see each other's lines.
// Device-scope relaxed atomic accesses go past the L2 (the stores write through, the loads fetch from memory), so
// the exchange needs no device-scope fence - a fence would write back and invalidate the XCD's whole L2, which at
// that moment holds the K/V tiles the other 31 workgroups of the XCD are working through.
__device__ __forceinline__ void store_shared_f32(float* ptr, float v) {
  __hip_atomic_store(reinterpret_cast<uint32_t*>(ptr), __float_as_uint(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_shared_f32(const float* ptr) {
  return __uint_as_float(__hip_atomic_load(reinterpret_cast<const uint32_t*>(ptr), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}
// This workgroup's number in the order in which the work is handed out: consecutive hardware workgroup numbers go
// to different XCDs; every XCD gets a contiguous range of the work instead, so that workgroups that share an L2
// read the same heads.
__device__ __forceinline__ uint32_t group_number(uint32_t G) {
  uint32_t b = blockIdx.x;
  asm volatile("" : "+s"(b));
  return G % 8 == 0 ? (b & 7) * (G / 8) + (b >> 3) : b;
}

template <bool WIDE>
__global__ __launch_bounds__(kAttnThreads) void kv_attention_kernel(AttnParams p) {
  constexpr int kQueries = WIDE ? 2 * kWgQueries : kWgQueries;  // queries per workgroup
  constexpr int kHalves = WIDE ? 2 : 1;                          // 64-key tiles a wave works through per iteration
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  SlotTable& tab = *reinterpret_cast<SlotTable*>(smem + 2 * kStageBytes);

  const int n_iter = (int)((p.n_cached + p.n_new + kIterKeys - 1) / kIterKeys);
  WorkCursor at;  // where this workgroup is in its work (attention_split.h)
  {
    const auto& c = reread_params();
    at = start_of_work(group_number(c.d.G), division_of(c));
  }

  if (const int tid = threadIdx.x; tid < p.n_slots) {
    tab.kv[tid] = reinterpret_cast<const uint8_t*>(p.kv_ptrs[tid]);
    tab.ks[tid] = reinterpret_cast<const uint8_t*>(p.ks_ptrs[tid]);
    tab.vv[tid] = reinterpret_cast<const uint8_t*>(p.vv_ptrs[tid]);
    tab.vs[tid] = reinterpret_cast<const uint8_t*>(p.vs_ptrs[tid]);
    tab.kg[tid] = load_global<float>(reinterpret_cast<const void*>(p.ka_ptrs[tid])) * p.inv_denom;
    tab.vg[tid] = load_global<float>(reinterpret_cast<const void*>(p.va_ptrs[tid])) * p.inv_denom;
  }

  __syncthreads();

  // After its whole tiles (workgroups that share an XCD run neighbouring tiles of a round side by side, in step
  // through the key range), a workgroup's share of the units is cut at tile boundaries into segments: iterations
  // [seg_begin, seg_end) of one tile (head x group of queries).  A segment that is a whole tile ends with the normalised output; the
  // others leave (O, reference point, row sum) in `partials`, and the workgroup that finishes a tile's last
  // segment combines them.  The segments are taken from the share's end backwards: a share is typically the
  // tail of one tile followed by the head of the next, and with the head (keys from 0) first and the tail
  // (keys up to the end) last, all workgroups of the launch move through the key range together, a few
  // iterations apart at most, which is what lets those of one head find each other's K/V lines in the L2.
  for (;;) {
  int tile_id, seg_begin, seg_end;
  bf16x8 qf[8];
  {
    const auto& c = reread_params();
    Segment seg;
    if (!next_segment(at, group_number(c.d.G), division_of(c), seg)) break;
    tile_id = (int)seg.tile;
    seg_begin = seg.begin;
    seg_end = seg.end;
  }
  int head, qtile;
  if (const int n_full = p.H * p.full_qtiles; tile_id < n_full) {
    head = tile_id / p.full_qtiles;
    qtile = tile_id - head * p.full_qtiles;
  } else {
    head = tile_id - n_full;
    qtile = p.full_qtiles;
  }
  // The thread's coordinates, derived anew in every segment (see fresh_thread_index).
  const int tid = fresh_thread_index(), lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, lh = lane >> 5;
  const int qq = WIDE ? wave : (wave & 3), kp = WIDE ? 0 : (wave >> 2);  // group of 32 queries, key parity
  // 256-query kernel: when the tile holds at most 128 queries (the last group of queries of a head is rarely
  // full), its waves 4..7 have none, and each wave that has some then has its SIMD to itself (waves w and w + 4
  // share one).  The waves without queries take their part in bringing K and V into LDS and in every barrier, and
  // nothing else: no MFMAs, no exponentials, no fragment reads.  With more than 128 queries some SIMD carries two
  // busy waves whatever the others do, and nothing would be gained (in the 128-query kernel, where the two waves
  // of a SIMD serve the same queries, never).
  bool wave_idle = false;
  if constexpr (WIDE) {
    const auto& c = reread_params();
    const int64_t first = (int64_t)qtile * kQueries;
    wave_idle = __builtin_amdgcn_readfirstlane((int)(c.Lq - first <= 128 && first + qq * kWaveQueries >= c.Lq)) != 0;
  }
  {
    const auto& c = reread_params();
    int64_t query = (int64_t)qtile * kQueries + qq * kWaveQueries + l32;
    if (query >= c.Lq) query = c.Lq - 1;
    const uint16_t* src = c.q + (query * p.H + head) * kHeadDim + 8 * lh;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) qf[ks] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(src + 16 * ks));
  }

  float16v o[4];
#pragma unroll
  for (int dt = 0; dt < 4; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[dt][i] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;

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
  int iter_base = seg_begin * kIterKeys;
  int k_slot = (iter_base + k_local) / p.bts, k_off = iter_base + k_local - k_slot * p.bts;
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
    bf16x4 vfr[2][4][2];
    read_v(0, vfr[0]);
    __builtin_amdgcn_sched_barrier(0);
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
    // The scheduling barriers keep every LDS read where it is written: a whole step ahead of the MFMAs that use
    // it.  Left alone, the compiler moves each read down to just ahead of its MFMA to shorten register live
    // ranges, and the wave then sits out the LDS latency a dozen times per tile.
    bf16x8 pb[2];
    make_p(0, pb[0]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int step = 0; step < 4; ++step) {
      if (step < 3) read_v(step + 1, vfr[(step + 1) & 1]);
      __builtin_amdgcn_sched_barrier(0);
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
      __builtin_amdgcn_sched_barrier(0);
    }
    l_run += sum;
  };

  // prologue: the segment's first iteration into its stage, raw registers <- the second one
  fetch_next();
  decode_any(seg_begin & 1);
  advance();
  if (seg_begin + 1 < seg_end) fetch_next();
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
  const int n_fast = min(n_cached / kIterKeys, seg_end) - 1;
  int it = seg_begin;
  if (wave_idle) {
    // A wave without queries: the conversion of its rows, the same number of barriers, nothing else.
    for (; it < n_fast; ++it) {
      uint8_t* nxt = smem + ((it + 1) & 1) * kStageBytes;
      const bool has_next2 = it + 2 < seg_end;
      const uint32_t wk[4] = {kf.v.x, kf.v.y, kf.v.z, kf.v.w}, wv[4] = {vf.v.x, vf.v.y, vf.v.z, vf.v.w};
      half2v ks2[2], vs2[2];
      block_scales_f16(kf.scales, ks2);
      block_scales_f16(vf.scales, vs2);
      uint8_t* kdst = nxt + k_dst_off;
      uint8_t* vdst = nxt + v_dst_off;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float v8[8];
        fp4x8_to_f32(wk[j], ks2[j >> 1], k_gs, v8);
        reinterpret_cast<uint4*>(kdst)[j] = make_uint4(pack_bf16(v8[0], v8[1]), pack_bf16(v8[2], v8[3]),
                                                       pack_bf16(v8[4], v8[5]), pack_bf16(v8[6], v8[7]));
        fp4x8_to_f32(wv[j], vs2[j >> 1], v_gs, v8);
        reinterpret_cast<uint4*>(vdst)[j] = make_uint4(pack_bf16(v8[0], v8[1]), pack_bf16(v8[2], v8[3]),
                                                       pack_bf16(v8[4], v8[5]), pack_bf16(v8[6], v8[7]));
      }
      advance();
      if (has_next2) fetch_next();
      __syncthreads();
    }
  }
  for (; it < n_fast; ++it) {
    const uint8_t* cur = smem + (it & 1) * kStageBytes;
    uint8_t* nxt = smem + ((it + 1) & 1) * kStageBytes;
    const bool has_next2 = it + 2 < seg_end;
    const uint32_t wk[4] = {kf.v.x, kf.v.y, kf.v.z, kf.v.w}, wv[4] = {vf.v.x, vf.v.y, vf.v.z, vf.v.w};
    half2v ks2[2], vs2[2];
    block_scales_f16(kf.scales, ks2);
    block_scales_f16(vf.scales, vs2);
    uint8_t* kdst = nxt + k_dst_off;
    uint8_t* vdst = nxt + v_dst_off;
#pragma unroll
    for (int h = 0; h < kHalves; ++h) {
      const int tile = WIDE ? h : kp;
      float16v sc[2];
      const uint8_t* krow0 = cur + tile * kKTileBytes + l32 * kKPitch + lh * 16;
      const uint8_t* krow1 = krow0 + 32 * kKPitch;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) sc[kt][i] = 0.0f;
      // K fragments two steps ahead of their MFMAs, three sets in rotation, held in place by scheduling barriers.
      uint4 fk[3][2];
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        fk[ks][0] = *reinterpret_cast<const uint4*>(krow0 + ks * 32);
        fk[ks][1] = *reinterpret_cast<const uint4*>(krow1 + ks * 32);
      }
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        if (ks < 6) {
          fk[(ks + 2) % 3][0] = *reinterpret_cast<const uint4*>(krow0 + (ks + 2) * 32);
          fk[(ks + 2) % 3][1] = *reinterpret_cast<const uint4*>(krow1 + (ks + 2) * 32);
        }
        __builtin_amdgcn_sched_barrier(0);
        const bf16x8 fa0 = __builtin_bit_cast(bf16x8, fk[ks % 3][0]), fa1 = __builtin_bit_cast(bf16x8, fk[ks % 3][1]);
        sc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa0, qf[ks], sc[0], 0, 0, 0);
        sc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa1, qf[ks], sc[1], 0, 0, 0);
        // One dword (8 elements) of the prefetched rows at a time.  One tile per wave: K in the even steps, V in the
        // odd ones.  Two tiles per wave: every second step, K under the first tile's MFMAs and V under the second's.
        if (!WIDE || (ks & 1) == 0) {
          const int j = ks >> 1;
          const bool is_k = WIDE ? h == 0 : (ks & 1) == 0;
          float v8[8];
          fp4x8_to_f32(is_k ? wk[j] : wv[j], is_k ? ks2[j >> 1] : vs2[j >> 1], is_k ? k_gs : v_gs, v8);
          reinterpret_cast<uint4*>(is_k ? kdst : vdst)[j] = make_uint4(pack_bf16(v8[0], v8[1]), pack_bf16(v8[2], v8[3]),
                                                                       pack_bf16(v8[4], v8[5]), pack_bf16(v8[6], v8[7]));
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      if (h == kHalves - 1) {
        advance();
        if (has_next2) fetch_next();
      }
      softmax_pv(sc, cur + 2 * kKTileBytes + tile * kVTileBytes);
    }
    __syncthreads();
  }

  // Plain body: the S phase without interleaved conversion, masking in the last tile, and the successor tile
  // decoded after the MFMAs (or, for the chunk's own bf16 tiles, brought in ahead of them).
  for (; it < seg_end; ++it) {
    const uint8_t* cur = smem + (it & 1) * kStageBytes;
    // A successor that lies wholly in the bf16 chunk is brought in ahead of the MFMAs: its K rows go
    // and V rows go straight from global memory into the other stage (one 256-byte row per wave instruction,
    // 16 rows of each per wave).
    const bool next_is_chunk = it + 1 < seg_end && iter_base >= n_cached && iter_base + kIterKeys <= Lk_i;  // iter_base = first key of tile it + 1
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
#pragma unroll 1
    for (int h = 0; h < kHalves; ++h) {
      const int tile = WIDE ? h : kp;
      const int tile_base = it * kIterKeys + tile * kTileKeys;
      if (tile_base >= Lk_i || wave_idle) break;
      float16v sc[2];
      const uint8_t* krow0 = cur + tile * kKTileBytes + l32 * kKPitch + lh * 16;
      const uint8_t* krow1 = krow0 + 32 * kKPitch;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) sc[kt][i] = 0.0f;
      uint4 fk[3][2];  // K fragments two steps ahead, as in the loop above
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        fk[ks][0] = *reinterpret_cast<const uint4*>(krow0 + ks * 32);
        fk[ks][1] = *reinterpret_cast<const uint4*>(krow1 + ks * 32);
      }
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        if (ks < 6) {
          fk[(ks + 2) % 3][0] = *reinterpret_cast<const uint4*>(krow0 + (ks + 2) * 32);
          fk[(ks + 2) % 3][1] = *reinterpret_cast<const uint4*>(krow1 + (ks + 2) * 32);
        }
        __builtin_amdgcn_sched_barrier(0);
        sc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fk[ks % 3][0]), qf[ks], sc[0], 0, 0, 0);
        sc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fk[ks % 3][1]), qf[ks], sc[1], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
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
      softmax_pv(sc, cur + 2 * kKTileBytes + tile * kVTileBytes);
    }
    if (next_is_chunk) {
      iter_base += kIterKeys;  // the slot bookkeeping of advance() has no use beyond the cache
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the rows have landed in LDS
    } else if (it + 1 < seg_end) {
      decode_any((it + 1) & 1);
      advance();
      if (it + 2 < seg_end) fetch_next();
    }
    __syncthreads();
  }

  l_run += __shfl_xor(l_run, 32, 64);  // row sums were per wave half so far
  {  // epilogue of the segment, with its own copies of the thread's coordinates (see fresh_thread_index)
  const auto& c = reread_params();
  const int tid = fresh_thread_index(), lane = tid & 63, wave = tid >> 6, l32 = lane & 31, lh = lane >> 5;
  const int qq = WIDE ? wave : (wave & 3), kp = WIDE ? 0 : (wave >> 2);
  if constexpr (WIDE) {
    // Every wave has seen its segment of the key range for its 32 queries.
    bool write_out = true;
    if (seg_begin != 0 || seg_end != n_iter) {
      // Part of a tile.  Whoever arrives last at a tile combines the parts; the others leave their state in a
      // record (two records per workgroup: one for the first tile it touches, one for the last) and count
      // their arrival.  The parts are combined from the end of the key range backwards whoever does it, so
      // the result does not depend on the order of arrival.  The workgroup that holds the last part is
      // normally also the last to arrive (the segments are walked backwards, see above): if a look at the
      // counter shows that, it goes on from its registers without writing a record.
      const uint32_t wg = group_number(c.d.G);
      const uint32_t split_tile = (uint32_t)tile_id - c.d.whole_rounds * c.d.G - c.d.extra;  // the tile's number among the split ones
      auto record_of = [&](uint32_t g) {
        return c.partials + (size_t)record_of_part(g, split_tile, division_of(c)) * kPartialFloats + wave * (66 * 64) + lane;
      };
      uint32_t g_first, g_last;
      parts_of_tile(split_tile, division_of(c), g_first, g_last);
      const int others = (int)(g_last - g_first);
      if (tid == 0)
        tab.last_arrival = wg == g_last && __hip_atomic_load(c.arrivals + split_tile, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == others;
      __syncthreads();
      const bool from_registers = tab.last_arrival != 0;
      write_out = from_registers;
      if (!from_registers) {
        if (!wave_idle) {
          float* mine = record_of(wg);
#pragma unroll
          for (int dt = 0; dt < 4; ++dt)
#pragma unroll
            for (int i = 0; i < 16; ++i) store_shared_f32(mine + (dt * 16 + i) * 64, o[dt][i]);
          store_shared_f32(mine + 64 * 64, m_run);
          store_shared_f32(mine + 65 * 64, l_run);
        }
        // Every wave waits until its own record stores are complete (vmcnt(0): a write-through store is
        // acknowledged once it is visible device-wide) before it reaches the barrier; thread 0 counts the arrival
        // behind that barrier, so no workgroup can see the count without the whole record being in memory.
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __syncthreads();
        if (tid == 0)
          tab.last_arrival = __hip_atomic_fetch_add(c.arrivals + split_tile, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == others;
        __syncthreads();
        write_out = tab.last_arrival != 0;
      }
      if (write_out) {
        if (tid == 0) __hip_atomic_store(c.arrivals + split_tile, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
        if (!from_registers) {  // start from nothing; the first step below turns that into the last part exactly
          m_run = -INFINITY;
          l_run = 0.0f;
#pragma unroll
          for (int dt = 0; dt < 4; ++dt)
#pragma unroll
            for (int i = 0; i < 16; ++i) o[dt][i] = 0.0f;
        }
        for (int g = (int)g_last - (from_registers ? 1 : 0); g >= (int)g_first && !wave_idle; --g) {
          const float* theirs = record_of((uint32_t)g);
          const float m1 = load_shared_f32(theirs + 64 * 64), l1 = load_shared_f32(theirs + 65 * 64);
          const float m = fmaxf(m_run, m1);
          const float a0 = (m_run == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f((m_run - m) * p.scale_log2);
          const float a1 = (m1 == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f((m1 - m) * p.scale_log2);
          l_run = l_run * a0 + l1 * a1;
          m_run = m;
#pragma unroll
          for (int dt = 0; dt < 4; ++dt)
#pragma unroll
            for (int i = 0; i < 16; ++i) o[dt][i] = o[dt][i] * a0 + load_shared_f32(theirs + (dt * 16 + i) * 64) * a1;
        }
      }
    }
    if (write_out) {
      float out_max = 0.0f;
      const float inv_l = 1.0f / l_run;
      const int64_t query = (int64_t)qtile * kQueries + qq * kWaveQueries + l32;
      if (query < c.Lq) {
        uint16_t* dst = c.out + (query * p.H + head) * kHeadDim;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
          for (int rg = 0; rg < 4; ++rg) {
            const uint2 packed = make_uint2(pack_bf16(o[dt][4 * rg] * inv_l, o[dt][4 * rg + 1] * inv_l),
                                            pack_bf16(o[dt][4 * rg + 2] * inv_l, o[dt][4 * rg + 3] * inv_l));
            *reinterpret_cast<uint2*>(dst + dt * 32 + 8 * rg + 4 * lh) = packed;
            out_max = abs_max_bf16x8(make_uint4(packed.x, packed.y, 0u, 0u), out_max);
          }
      }
      if (c.sink.parts) {
        out_max = wave_max(out_max);
        if (lane == 0) amax_sink_update(AmaxSink{c.sink.parts, c.sink.epoch, c.sink.epoch_offset}, (uint32_t)tile_id * 8 + wave, out_max);
      }
    }
  } else {
    // ---- merge the two key-parity halves through LDS and write out.
    float* xo = reinterpret_cast<float*>(smem);   // [qq][64 regs][64 lanes]
    float* xm = xo + 4 * 64 * 64;                  // [qq][64]
    float* xl = xm + 4 * 64;
    if (kp == 1 && !wave_idle) {
#pragma unroll
      for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) xo[(qq * 64 + dt * 16 + i) * 64 + lane] = o[dt][i];
      xm[qq * 64 + lane] = m_run;
      xl[qq * 64 + lane] = l_run;
    }
    __syncthreads();
    if (kp == 0 && !wave_idle) {
      float out_max = 0.0f;
      const float m1 = xm[qq * 64 + lane], l1 = xl[qq * 64 + lane];
      const float m = fmaxf(m_run, m1);
      const float a0 = __builtin_amdgcn_exp2f((m_run - m) * p.scale_log2);
      const float a1 = (m1 == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f((m1 - m) * p.scale_log2);
      const float inv_l = 1.0f / (l_run * a0 + l1 * a1);
      const int64_t query = (int64_t)qtile * kQueries + qq * kWaveQueries + l32;
      if (query < c.Lq) {
        uint16_t* dst = c.out + (query * p.H + head) * kHeadDim;
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
      if (c.sink.parts) {
        out_max = wave_max(out_max);
        if (lane == 0) amax_sink_update(AmaxSink{c.sink.parts, c.sink.epoch, c.sink.epoch_offset}, (uint32_t)tile_id * 4 + qq, out_max);
      }
    }
  }
  }
  __syncthreads();  // the stages (and the merge area) are free for the next segment
  }  // segments
}

static std::atomic<int> g_attention_policy{LL_ATTENTION_AUTO};

// Three ways to run a launch, all one workgroup per compute unit at a time (LDS):
//  * 128 queries per workgroup, the key range halved between two sets of waves; one workgroup per tile;
//  * 256 queries per workgroup (every decoded K/V tile serves twice as many MFMAs: an iteration takes about 1.64
//    times as long for twice the work), one workgroup per tile;
//  * 256 queries per workgroup, whole rounds of tiles first and the (tile, iteration) sequence of the tiles behind
//    them cut into one equal share per compute unit; tiles that straddle two shares are combined by the workgroup
//    that finishes last.
// plan_attention (attention_split.h) chooses.
static int launch_attention(const AttnParams& p_in, hipStream_t stream) {
  AttnParams p = p_in;
  const size_t smem = 2 * kStageBytes + sizeof(SlotTable);
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    set_error("ll_kv_attention: hipGetDevice failed");
    return LL_ELAUNCH;
  }
  if (int rc = compute_units_of(dev, cus, "ll_kv_attention")) return rc;
  const int64_t n_iter = (p.n_cached + p.n_new + kIterKeys - 1) / kIterKeys;
  LL_REQUIRE(p.H * ((p.Lq + kWgQueries - 1) / kWgQueries) * n_iter < (1ll << 32), "ll_kv_attention: too many (tile, iteration) units");
  const int policy = g_attention_policy.load(std::memory_order_relaxed);
  AttentionPlan plan = plan_attention(p.Lq, p.H, p.n_cached + p.n_new, cus, policy);
  StreamScratch w;
  if (plan.mode == LL_ATTENTION_SPLIT) {
    // The split division passes partial tiles through device memory of the library's own.  While the stream is
    // being captured nothing may be allocated (and the clearing of a new set must not become a graph node): a set
    // that an earlier launch or ll_kv_attention_reserve left on this stream is used as it is; without one the
    // automatic choice falls back to the cheaper of the two divisions that need no memory, and an explicit
    // request for the split division is refused.
    const bool capturing = stream_is_capturing(stream);
    bool missing = false;
    if (int rc = stream_scratch(dev, stream, (size_t)2 * plan.d.G * kPartialFloats * sizeof(float), (size_t)plan.split_tiles, !capturing, w,
                                &missing, "ll_kv_attention")) return rc;
    if (missing) {
      if (policy == LL_ATTENTION_SPLIT) {
        set_error("ll_kv_attention: the split division needs device memory that cannot be allocated while the stream "
                  "is being captured; call ll_kv_attention_reserve for this shape first, or select another division");
        return LL_ENOSUP;
      }
      plan = plan_attention(p.Lq, p.H, p.n_cached + p.n_new, cus, policy, /*allow_split=*/false);
    }
  }
  p.n_qtiles = plan.n_qtiles;
  p.full_qtiles = plan.full_qtiles;
  p.d = plan.d;
  if (plan.mode == LL_ATTENTION_NARROW) {
    static std::atomic<uint64_t> lds_allowed{0};
    if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(&kv_attention_kernel<false>), smem, lds_allowed, "ll_kv_attention")) return rc;
    hipLaunchKernelGGL(kv_attention_kernel<false>, dim3(p.d.G), dim3(kAttnThreads), smem, stream, p);
  } else {
    if (plan.mode == LL_ATTENTION_SPLIT) {
      p.partials = reinterpret_cast<float*>(w.records);
      p.arrivals = w.counters;
    }
    static std::atomic<uint64_t> lds_allowed_w{0};
    if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(&kv_attention_kernel<true>), smem, lds_allowed_w, "ll_kv_attention")) return rc;
    hipLaunchKernelGGL(kv_attention_kernel<true>, dim3(p.d.G), dim3(kAttnThreads), smem, stream, p);
  }
  LL_CHECK_LAUNCH("kv_attention_kernel");
  return LL_OK;
}

}  // namespace ll

extern "C" int ll_kv_attention_set_policy(int policy) {
  LL_REQUIRE(policy >= LL_ATTENTION_AUTO && policy <= LL_ATTENTION_SPLIT, "ll_kv_attention_set_policy: unknown policy %d", policy);
  ll::g_attention_policy.store(policy);
  return LL_OK;
}

extern "C" int ll_kv_attention_get_policy(void) { return ll::g_attention_policy.load(); }

extern "C" int ll_kv_attention_reserve(int64_t Lq, int num_heads, int64_t n_keys, void* stream) {
  using namespace ll;
  LL_REQUIRE(Lq > 0 && num_heads > 0 && n_keys > 0 && Lq < (1ll << 30) && n_keys < (1ll << 30), "ll_kv_attention_reserve: bad sizes");
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    set_error("ll_kv_attention_reserve: hipGetDevice failed");
    return LL_ELAUNCH;
  }
  if (int rc = compute_units_of(dev, cus, "ll_kv_attention")) return rc;
  const AttentionPlan plan = plan_attention(Lq, num_heads, n_keys, cus, g_attention_policy.load(std::memory_order_relaxed));
  if (plan.mode != LL_ATTENTION_SPLIT) return LL_OK;
  if (stream_is_capturing(static_cast<hipStream_t>(stream))) {
    set_error("ll_kv_attention_reserve: the stream is being captured; reserve before the recording starts");
    return LL_ENOSUP;
  }
  StreamScratch w;
  return stream_scratch(dev, static_cast<hipStream_t>(stream), (size_t)2 * plan.d.G * kPartialFloats * sizeof(float),
                        (size_t)plan.split_tiles, true, w, nullptr, "ll_kv_attention_reserve");
}

extern "C" int ll_kv_attention_release(void* stream) { return ll_release_stream_memory(stream); }

extern "C" int ll_kv_attention_plan(int64_t Lq, int num_heads, int64_t n_keys, int compute_units, int policy,
                                    int* division, uint32_t* workgroups, uint32_t* whole_rounds, int64_t* split_tiles) {
  LL_REQUIRE(Lq > 0 && num_heads > 0 && n_keys > 0 && compute_units > 0 && Lq < (1ll << 30) && n_keys < (1ll << 30),
             "ll_kv_attention_plan: bad sizes");
  LL_REQUIRE(policy >= LL_ATTENTION_AUTO && policy <= LL_ATTENTION_SPLIT, "ll_kv_attention_plan: unknown policy %d", policy);
  const ll::AttentionPlan plan = ll::plan_attention(Lq, num_heads, n_keys, compute_units, policy);
  if (division) *division = plan.mode;
  if (workgroups) *workgroups = plan.d.G;
  if (whole_rounds) *whole_rounds = plan.d.whole_rounds;
  if (split_tiles) *split_tiles = plan.split_tiles;
  return LL_OK;
}

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
  LL_REQUIRE(sink_is_valid(amax_sink), "ll_kv_attention_amax: amax sink needs 8-byte alignment and a non-zero epoch");
  p.sink = make_sink(amax_sink);
  return launch_attention(p, static_cast<hipStream_t>(stream));
}

extern "C" int ll_attention_bf16(const void* q, const void* k, const void* v, int64_t Lq, int64_t Lk, int num_heads,
                                 float softmax_scale, void* out, void* stream) {
  return ll_kv_attention(q, Lq, num_heads, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0, 6.f, 256.f, k,
                         v, Lk, softmax_scale, out, stream);
}
