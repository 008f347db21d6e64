// Chunk attention over an NVFP4 KV cache for gfx950, with the dequantization fused into the K/V tile
// load:  out = softmax(q k^T * scale) v  over  [ cached tokens (FP4 slots) | current chunk (bf16) ].
//
// Replaces "dequantize the whole cache to bf16, copy the chunk in, call flash attention"
// (wan_5b/modules/causal_model.py:557-567, 628-671, 781; utils/quant.py:731-768).
//
// Workgroup = one head x 128 queries, 4 waves.  Wave w owns 64 queries (w & 1) and every second
// 64-key tile (w >> 1); the two halves of the key range are merged at the end.  Per iteration all
// 256 threads decode 128 keys of K and V (e2m1 x e4m3 x amax/(6*256) -> bf16, the values the
// reference's dequantized bf16 cache holds) into LDS: K row-major, V transposed.  The MFMAs compute
// S^T = K Q^T and O^T = V^T P^T (v_mfma_f32_32x32x16_bf16), so every lane owns one query column:
// row max / row sum need no cross-lane traffic beyond one swap between the wave halves, and the
// online-softmax rescale is a per-lane scalar.
#include "ll_common.h"

namespace ll {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef float float2v __attribute__((ext_vector_type(2)));

constexpr int kHeadDim = 128;
constexpr int kTileKeys = 64;                  // keys per wave tile
constexpr int kIterKeys = 2 * kTileKeys;       // keys decoded per iteration (one tile per key-parity)
constexpr int kWgQueries = 128;
constexpr int kKPitch = 272;                   // bytes per key row of K in LDS (256 + 16 pad)
constexpr int kVPitch = 136;                   // bytes per d row of V^T in LDS (128 + 8 pad)
constexpr int kKTileBytes = kTileKeys * kKPitch;
constexpr int kVTileBytes = kHeadDim * kVPitch;
constexpr int kStageBytes = 2 * kKTileBytes + 2 * kVTileBytes;
constexpr int kMaxSlots = 64;
constexpr int kAttnThreads = 256;

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

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  bf16x2 p;
  p[0] = (__bf16)a;
  p[1] = (__bf16)b;
  return __builtin_bit_cast(uint32_t, p);
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

// Swizzled position of the 8-byte chunk (4 keys) `chunk` (0..15) in row `row` of a V^T tile: rows that
// are 16 apart (written by neighbouring lanes) land in different LDS banks.
__device__ __forceinline__ int vt_chunk(int row, int chunk) {
  const int b = (row >> 4) & 7;
  return chunk ^ b ^ ((b & 1) << 3);
}

// Prefetched (one iteration ahead) raw data.  Only FP4 slot data is held in registers across the MFMA
// phase; keys of the current bf16 chunk are read when they are stored (they are a fifth of the keys, and
// keeping 128 bytes per thread live would spill).
struct KFetch {       // K of one key, one half of the head dimension (64 elements)
  uint4 v0, v1;       // 32 packed bytes
  uint32_t scales;    // 4 e4m3 block scales
  float gs;           // amax / (e2m1_max * e4m3_max) of the slot
  const uint4* src;   // bf16 source row (kind 1)
  int kind;           // 0 = fp4 slot, 1 = bf16 chunk, 2 = beyond the end (zeros)
};
struct VFetch {       // V of one key, one 16-element block
  uint2 v;            // 8 packed bytes
  uint32_t scale;     // e4m3 block scale byte
  float gs;
  const uint4* src;
  int kind;
};

// (slot, off) = key / block_token_size and key % block_token_size, tracked incrementally by the caller.
__device__ __forceinline__ void fetch_k(const AttnParams& p, const SlotTable& tab, int key, int slot, int off,
                                        int head, int half, KFetch& f) {
  f.src = nullptr;
  if (key < (int)p.n_cached) {
    const int64_t row = (int64_t)off * p.H + head;
    const uint4* src = reinterpret_cast<const uint4*>(tab.kv[slot] + row * 64 + half * 32);
    f.v0 = src[0];
    f.v1 = src[1];
    f.scales = *reinterpret_cast<const uint32_t*>(tab.ks[slot] + blocked_scale_offset(row, half * 4, 8));
    f.gs = tab.kg[slot];
    f.kind = 0;
  } else if (key < (int)(p.n_cached + p.n_new)) {
    f.src = reinterpret_cast<const uint4*>(p.k_new + ((int64_t)(key - (int)p.n_cached) * p.H + head) * kHeadDim + half * 64);
    f.kind = 1;
  } else {
    f.kind = 2;
  }
}

__device__ __forceinline__ void fetch_v(const AttnParams& p, const SlotTable& tab, int key, int slot, int off,
                                        int head, int blk, VFetch& f) {
  f.src = nullptr;
  if (key < (int)p.n_cached) {
    const int64_t row = (int64_t)off * p.H + head;
    f.v = *reinterpret_cast<const uint2*>(tab.vv[slot] + row * 64 + blk * 8);
    f.scale = tab.vs[slot][blocked_scale_offset(row, blk, 8)];
    f.gs = tab.vg[slot];
    f.kind = 0;
  } else if (key < (int)(p.n_cached + p.n_new)) {
    f.src = reinterpret_cast<const uint4*>(p.v_new + ((int64_t)(key - (int)p.n_cached) * p.H + head) * kHeadDim + blk * 16);
    f.kind = 1;
  } else {
    f.kind = 2;
  }
}

// Decode K (64 elements of one key) to bf16 and store the 128 bytes into the key's LDS row.
__device__ __forceinline__ void store_k(const KFetch& f, uint8_t* dst) {
  uint4* d4 = reinterpret_cast<uint4*>(dst);
  if (f.kind == 0) {
    const uint32_t w[8] = {f.v0.x, f.v0.y, f.v0.z, f.v0.w, f.v1.x, f.v1.y, f.v1.z, f.v1.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {  // block j: dwords 2j, 2j+1
      const float sf = fp8_byte_to_f32(f.scales, j) * f.gs;
      float lo8[8], hi8[8];
      fp4x8_to_f32(w[2 * j], sf, lo8);
      fp4x8_to_f32(w[2 * j + 1], sf, hi8);
      d4[2 * j] = make_uint4(pack_bf16(lo8[0], lo8[1]), pack_bf16(lo8[2], lo8[3]), pack_bf16(lo8[4], lo8[5]),
                             pack_bf16(lo8[6], lo8[7]));
      d4[2 * j + 1] = make_uint4(pack_bf16(hi8[0], hi8[1]), pack_bf16(hi8[2], hi8[3]), pack_bf16(hi8[4], hi8[5]),
                                 pack_bf16(hi8[6], hi8[7]));
    }
  } else if (f.kind == 1) {
#pragma unroll
    for (int i = 0; i < 8; ++i) d4[i] = f.src[i];
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) d4[i] = make_uint4(0, 0, 0, 0);
  }
}

// 16 head-dim elements of 4 consecutive keys -> for every element one 8-byte run of 4 bf16 along the key
// axis, written into the transposed (and swizzled) V tile.  vt_tile points at the tile, row0 = first d row.
__device__ __forceinline__ void store_v4(const VFetch (&f)[4], uint8_t* vt_tile, int row0, int chunk) {
  const bool all_fp4 = (f[0].kind | f[1].kind | f[2].kind | f[3].kind) == 0;
  if (all_fp4) {
    float v[4][16];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      const float sf = fp8_byte_to_f32(f[kk].scale, 0) * f[kk].gs;
      float lo8[8], hi8[8];
      fp4x8_to_f32(f[kk].v.x, sf, lo8);
      fp4x8_to_f32(f[kk].v.y, sf, hi8);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        v[kk][i] = lo8[i];
        v[kk][8 + i] = hi8[i];
      }
    }
#pragma unroll
    for (int dd = 0; dd < 16; ++dd) {
      const int row = row0 + dd;
      *reinterpret_cast<uint2*>(vt_tile + row * kVPitch + vt_chunk(row, chunk) * 8) =
          make_uint2(pack_bf16(v[0][dd], v[1][dd]), pack_bf16(v[2][dd], v[3][dd]));
    }
  } else {
    // generic: bring every key to 8 dwords of bf16, then interleave halves across keys
    uint32_t w[4][8];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      if (f[kk].kind == 0) {
        const float sf = fp8_byte_to_f32(f[kk].scale, 0) * f[kk].gs;
        float lo8[8], hi8[8];
        fp4x8_to_f32(f[kk].v.x, sf, lo8);
        fp4x8_to_f32(f[kk].v.y, sf, hi8);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          w[kk][i] = pack_bf16(lo8[2 * i], lo8[2 * i + 1]);
          w[kk][4 + i] = pack_bf16(hi8[2 * i], hi8[2 * i + 1]);
        }
      } else if (f[kk].kind == 1) {
        const uint4 a = f[kk].src[0], b = f[kk].src[1];
        w[kk][0] = a.x; w[kk][1] = a.y; w[kk][2] = a.z; w[kk][3] = a.w;
        w[kk][4] = b.x; w[kk][5] = b.y; w[kk][6] = b.z; w[kk][7] = b.w;
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) w[kk][i] = 0;
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      // v_perm_b32: bytes 0-3 come from the second operand, 4-7 from the first
      const uint32_t e01 = __builtin_amdgcn_perm(w[1][i], w[0][i], 0x05040100u);
      const uint32_t e23 = __builtin_amdgcn_perm(w[3][i], w[2][i], 0x05040100u);
      const uint32_t o01 = __builtin_amdgcn_perm(w[1][i], w[0][i], 0x07060302u);
      const uint32_t o23 = __builtin_amdgcn_perm(w[3][i], w[2][i], 0x07060302u);
      const int r0 = row0 + 2 * i, r1 = r0 + 1;
      *reinterpret_cast<uint2*>(vt_tile + r0 * kVPitch + vt_chunk(r0, chunk) * 8) = make_uint2(e01, e23);
      *reinterpret_cast<uint2*>(vt_tile + r1 * kVPitch + vt_chunk(r1, chunk) * 8) = make_uint2(o01, o23);
    }
  }
}

__global__ __launch_bounds__(kAttnThreads) void kv_attention_kernel(AttnParams p) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  SlotTable& tab = *reinterpret_cast<SlotTable*>(smem + 2 * kStageBytes);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, lh = lane >> 5;
  const int qh = wave & 1, kp = wave >> 1;

  // workgroup -> (head, query tile); workgroups that share an XCD get the same heads
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
    tab.kg[tid] = *reinterpret_cast<const float*>(p.ka_ptrs[tid]) * p.inv_denom;
    tab.vg[tid] = *reinterpret_cast<const float*>(p.va_ptrs[tid]) * p.inv_denom;
  }

  // Q fragments: B operand, lane = query column, 8 consecutive head-dim elements per k-step
  bf16x8 qf[2][8];
#pragma unroll
  for (int qt = 0; qt < 2; ++qt) {
    int64_t query = (int64_t)qtile * kWgQueries + qh * 64 + qt * 32 + l32;
    if (query >= p.Lq) query = p.Lq - 1;
    const uint16_t* src = p.q + (query * p.H + head) * kHeadDim + 8 * lh;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) qf[qt][ks] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(src + 16 * ks));
  }

  float16v o[4][2];
#pragma unroll
  for (int dt = 0; dt < 4; ++dt)
#pragma unroll
    for (int qt = 0; qt < 2; ++qt)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[dt][qt][i] = 0.0f;
  float m_run[2] = {-INFINITY, -INFINITY}, l_run[2] = {0.0f, 0.0f};

  const int64_t Lk = p.n_cached + p.n_new;
  const int n_iter = (int)((Lk + kIterKeys - 1) / kIterKeys);
  __syncthreads();  // slot table visible

  // ---- decode plan.  K: thread = (key_local = tid / 2, half of the head dim = tid % 2).
  //                    V: thread = (block of 16 head-dim elements = tid % 8, 4 consecutive keys = tid / 8).
  KFetch kf;
  VFetch vf[4];
  // slot / offset of this thread's K key and of its first V key; both advance by kIterKeys per fetch
  int k_key = tid >> 1, v_key = 4 * (tid >> 3);
  int k_slot = k_key / p.bts, k_off = k_key - k_slot * p.bts;
  int v_slot = v_key / p.bts, v_off = v_key - v_slot * p.bts;
  auto fetch_iter = [&]() {
    fetch_k(p, tab, k_key, k_slot, k_off, head, tid & 1, kf);
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      const bool wrap = v_off + kk >= p.bts;
      fetch_v(p, tab, v_key + kk, v_slot + (wrap ? 1 : 0), v_off + kk - (wrap ? p.bts : 0), head, tid & 7, vf[kk]);
    }
    k_key += kIterKeys;
    v_key += kIterKeys;
    k_off += kIterKeys;
    v_off += kIterKeys;
    while (k_off >= p.bts) {
      k_off -= p.bts;
      ++k_slot;
    }
    while (v_off >= p.bts) {
      v_off -= p.bts;
      ++v_slot;
    }
  };
  auto decode_iter = [&](int stage) {
    uint8_t* kbase = smem + stage * kStageBytes;
    uint8_t* vbase = kbase + 2 * kKTileBytes;
    const int key_local = tid >> 1;
    store_k(kf, kbase + (key_local >> 6) * kKTileBytes + (key_local & 63) * kKPitch + (tid & 1) * 128);
    const int vkey = 4 * (tid >> 3);
    store_v4(vf, vbase + (vkey >> 6) * kVTileBytes, (tid & 7) * 16, (vkey & 63) >> 2);
  };

  fetch_iter();
  decode_iter(0);
  __syncthreads();

  for (int it = 0; it < n_iter; ++it) {
    if (it + 1 < n_iter) fetch_iter();
    const int64_t tile_base = (int64_t)it * kIterKeys + kp * kTileKeys;
    if (tile_base < Lk) {
      const uint8_t* kt_base = smem + (it & 1) * kStageBytes + kp * kKTileBytes;
      const uint8_t* vt_base = smem + (it & 1) * kStageBytes + 2 * kKTileBytes + kp * kVTileBytes;
      // ---- S^T = K Q^T  (64 keys x 64 queries)
      float16v s[2][2];
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int qt = 0; qt < 2; ++qt)
#pragma unroll
          for (int i = 0; i < 16; ++i) s[kt][qt][i] = 0.0f;
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
          const bf16x8 a = __builtin_bit_cast(
              bf16x8, *reinterpret_cast<const uint4*>(kt_base + (kt * 32 + l32) * kKPitch + ks * 32 + lh * 16));
#pragma unroll
          for (int qt = 0; qt < 2; ++qt) s[kt][qt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[qt][ks], s[kt][qt], 0, 0, 0);
        }
      }
      // ---- mask keys beyond the end (only the last tile)
      if (tile_base + kTileKeys > Lk) {
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int64_t key = tile_base + kt * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
            if (key >= Lk) {
              s[kt][0][r] = -INFINITY;
              s[kt][1][r] = -INFINITY;
            }
          }
      }
      // ---- online softmax (per lane: one query per qt)
      uint32_t pb[2][2][2][4];  // [qt][kt][half of the 32 keys][4 dwords = 8 bf16]
#pragma unroll
      for (int qt = 0; qt < 2; ++qt) {
        float mx = s[0][qt][0];
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[kt][qt][r]);
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run[qt], mx);
        const float alpha = __builtin_amdgcn_exp2f((m_run[qt] - m_new) * p.scale_log2);
        const float neg = -m_new * p.scale_log2;
        float sum = 0.0f;
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
          float pr[16];
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            pr[r] = __builtin_amdgcn_exp2f(fmaf(s[kt][qt][r], p.scale_log2, neg));
            sum += pr[r];
          }
#pragma unroll
          for (int hf = 0; hf < 2; ++hf)
#pragma unroll
            for (int i = 0; i < 4; ++i) pb[qt][kt][hf][i] = pack_bf16(pr[8 * hf + 2 * i], pr[8 * hf + 2 * i + 1]);
        }
        l_run[qt] = l_run[qt] * alpha + sum;
        m_run[qt] = m_new;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
          for (int i = 0; i < 16; ++i) o[dt][qt][i] *= alpha;
      }
      // ---- O^T += V^T P^T.  k-slot e of wave half lh <-> key 16 step + 8 (e / 4) + 4 lh + e % 4
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
          const int chunk0 = kt * 8 + hf * 4 + lh;  // 8-byte chunk holding keys 4*chunk0 .. +3 of the tile
#pragma unroll
          for (int dt = 0; dt < 4; ++dt) {
            const int row = dt * 32 + l32;
            const uint8_t* src = vt_base + row * kVPitch;
            const uint2 v0 = *reinterpret_cast<const uint2*>(src + vt_chunk(row, chunk0) * 8);
            const uint2 v1 = *reinterpret_cast<const uint2*>(src + vt_chunk(row, chunk0 + 2) * 8);
            const bf16x8 a = __builtin_bit_cast(bf16x8, make_uint4(v0.x, v0.y, v1.x, v1.y));
#pragma unroll
            for (int qt = 0; qt < 2; ++qt) {
              const bf16x8 b = __builtin_bit_cast(
                  bf16x8, make_uint4(pb[qt][kt][hf][0], pb[qt][kt][hf][1], pb[qt][kt][hf][2], pb[qt][kt][hf][3]));
              o[dt][qt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, o[dt][qt], 0, 0, 0);
            }
          }
        }
    }
    if (it + 1 < n_iter) decode_iter((it + 1) & 1);
    __syncthreads();
  }

  // ---- merge the two key-parity halves and write out.  Row sums are per wave half so far.
#pragma unroll
  for (int qt = 0; qt < 2; ++qt) l_run[qt] += __shfl_xor(l_run[qt], 32, 64);
  float* xo = reinterpret_cast<float*>(smem);                 // [qh][128 regs][64 lanes]
  float* xm = xo + 2 * 128 * 64;                               // [qh][2][64]
  float* xl = xm + 2 * 2 * 64;
  if (kp == 1) {
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int qt = 0; qt < 2; ++qt)
#pragma unroll
        for (int i = 0; i < 16; ++i) xo[(qh * 128 + (dt * 2 + qt) * 16 + i) * 64 + lane] = o[dt][qt][i];
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) {
      xm[(qh * 2 + qt) * 64 + lane] = m_run[qt];
      xl[(qh * 2 + qt) * 64 + lane] = l_run[qt];
    }
  }
  __syncthreads();
  if (kp == 0) {
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) {
      const float m1 = xm[(qh * 2 + qt) * 64 + lane], l1 = xl[(qh * 2 + qt) * 64 + lane];
      const float m = fmaxf(m_run[qt], m1);
      const float a0 = __builtin_amdgcn_exp2f((m_run[qt] - m) * p.scale_log2);
      const float a1 = (m1 == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f((m1 - m) * p.scale_log2);
      const float inv_l = 1.0f / (l_run[qt] * a0 + l1 * a1);
      const int64_t query = (int64_t)qtile * kWgQueries + qh * 64 + qt * 32 + l32;
      if (query < p.Lq) {
        uint16_t* dst = p.out + (query * p.H + head) * kHeadDim;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
          for (int rg = 0; rg < 4; ++rg) {
            float v[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const float o1 = xo[(qh * 128 + (dt * 2 + qt) * 16 + 4 * rg + i) * 64 + lane];
              v[i] = (o[dt][qt][4 * rg + i] * a0 + o1 * a1) * inv_l;
            }
            const int d = dt * 32 + 8 * rg + 4 * lh;
            *reinterpret_cast<uint2*>(dst + d) = make_uint2(pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]));
          }
      }
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
    LL_REQUIRE(block_token_size > 0 && e2m1_max > 0.f && e4m3_max > 0.f, "ll_kv_attention: bad slot geometry");
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
  p.bts = block_token_size > 0 ? block_token_size : 1;
  p.n_slots = n_slots;
  p.inv_denom = n_cached > 0 ? 1.0f / (e2m1_max * e4m3_max) : 0.f;
  p.k_new = static_cast<const uint16_t*>(k_new);
  p.v_new = static_cast<const uint16_t*>(v_new);
  p.scale_log2 = softmax_scale * 1.4426950408889634f;
  p.out = static_cast<uint16_t*>(out);
  return launch_attention(p, static_cast<hipStream_t>(stream));
}

extern "C" int ll_attention_bf16(const void* q, const void* k, const void* v, int64_t Lq, int64_t Lk, int num_heads,
                                 float softmax_scale, void* out, void* stream) {
  return ll_kv_attention(q, Lq, num_heads, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0, 6.f, 256.f, k,
                         v, Lk, softmax_scale, out, stream);
}
