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

// Raw data of 16 consecutive head-dim elements of one key, as fetched from HBM.
struct KeyChunk {
  uint4 a, b;  // fp4: a.x,a.y = 8 packed bytes, a.z = scale byte, b.x = global scale bits; bf16: 32 bytes
  int kind;    // 0 = fp4, 1 = bf16, 2 = beyond the end (zeros)
};

__device__ __forceinline__ KeyChunk fetch_chunk(const AttnParams& p, const SlotTable& tab, bool is_v, int64_t key,
                                                int head, int blk) {
  KeyChunk c;
  c.a = make_uint4(0, 0, 0, 0);
  c.b = make_uint4(0, 0, 0, 0);
  if (key < p.n_cached) {
    const int slot = (int)(key / p.bts);
    const int64_t row = (key - (int64_t)slot * p.bts) * p.H + head;
    const uint8_t* vals = is_v ? tab.vv[slot] : tab.kv[slot];
    const uint8_t* scs = is_v ? tab.vs[slot] : tab.ks[slot];
    const uint2 v = *reinterpret_cast<const uint2*>(vals + row * 64 + blk * 8);
    c.a.x = v.x;
    c.a.y = v.y;
    c.a.z = scs[blocked_scale_offset(row, blk, 8)];
    c.b.x = __float_as_uint(is_v ? tab.vg[slot] : tab.kg[slot]);
    c.kind = 0;
  } else if (key < p.n_cached + p.n_new) {
    const uint16_t* src = (is_v ? p.v_new : p.k_new) + ((key - p.n_cached) * p.H + head) * kHeadDim + blk * 16;
    c.a = reinterpret_cast<const uint4*>(src)[0];
    c.b = reinterpret_cast<const uint4*>(src)[1];
    c.kind = 1;
  } else {
    c.kind = 2;
  }
  return c;
}

// 16 bf16 values (as 8 packed dwords) of a chunk.
__device__ __forceinline__ void chunk_to_bf16(const KeyChunk& c, uint32_t (&o)[8]) {
  if (c.kind == 0) {
    const float sf = e4m3_to_f32(c.a.z) * __uint_as_float(c.b.x);
    const uint32_t w[2] = {c.a.x, c.a.y};
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const float2v q0 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[i], 1.0f, 0);
      const float2v q1 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[i], 1.0f, 1);
      const float2v q2 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[i], 1.0f, 2);
      const float2v q3 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[i], 1.0f, 3);
      o[4 * i + 0] = pack_bf16(q0[0] * sf, q0[1] * sf);
      o[4 * i + 1] = pack_bf16(q1[0] * sf, q1[1] * sf);
      o[4 * i + 2] = pack_bf16(q2[0] * sf, q2[1] * sf);
      o[4 * i + 3] = pack_bf16(q3[0] * sf, q3[1] * sf);
    }
  } else {
    o[0] = c.a.x; o[1] = c.a.y; o[2] = c.a.z; o[3] = c.a.w;
    o[4] = c.b.x; o[5] = c.b.y; o[6] = c.b.z; o[7] = c.b.w;
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

  // ---- decode plan.  K: task = (key_local, 16-element block), 4 tasks per thread.
  //                    V: one task per thread = 4 consecutive keys x one 16-element block (transposed store).
  KeyChunk kc[4], vc[4];
  auto fetch_iter = [&](int it) {
    const int64_t base = (int64_t)it * kIterKeys;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int task = tid + i * kAttnThreads;
      kc[i] = fetch_chunk(p, tab, false, base + (task >> 3), head, task & 7);
    }
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) vc[kk] = fetch_chunk(p, tab, true, base + 4 * (tid >> 3) + kk, head, tid & 7);
  };
  auto decode_iter = [&](int stage) {
    uint8_t* kbase = smem + stage * kStageBytes;
    uint8_t* vbase = kbase + 2 * kKTileBytes;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int task = tid + i * kAttnThreads;
      const int key_local = task >> 3, blk = task & 7;
      uint32_t w[8];
      chunk_to_bf16(kc[i], w);
      uint4* dst = reinterpret_cast<uint4*>(kbase + (key_local >> 6) * kKTileBytes + (key_local & 63) * kKPitch + blk * 32);
      dst[0] = make_uint4(w[0], w[1], w[2], w[3]);
      dst[1] = make_uint4(w[4], w[5], w[6], w[7]);
    }
    uint32_t w[4][8];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) chunk_to_bf16(vc[kk], w[kk]);
    const int key_local = 4 * (tid >> 3), blk = tid & 7;
    uint8_t* vt = vbase + (key_local >> 6) * kVTileBytes + (key_local & 63) * 2;
#pragma unroll
    for (int dd = 0; dd < 16; ++dd) {
      // element dd of each of the 4 keys -> 4 consecutive bf16 along the key axis
      const int wi = dd >> 1;
      uint32_t e[4];
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) e[kk] = (dd & 1) ? (w[kk][wi] >> 16) : (w[kk][wi] & 0xFFFFu);
      *reinterpret_cast<uint2*>(vt + (blk * 16 + dd) * kVPitch) = make_uint2(e[0] | (e[1] << 16), e[2] | (e[3] << 16));
    }
  };

  fetch_iter(0);
  decode_iter(0);
  __syncthreads();

  for (int it = 0; it < n_iter; ++it) {
    if (it + 1 < n_iter) fetch_iter(it + 1);
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
          const int key0 = kt * 32 + hf * 16 + 4 * lh;
#pragma unroll
          for (int dt = 0; dt < 4; ++dt) {
            const uint8_t* src = vt_base + (dt * 32 + l32) * kVPitch + key0 * 2;
            const uint2 v0 = *reinterpret_cast<const uint2*>(src);
            const uint2 v1 = *reinterpret_cast<const uint2*>(src + 16);
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
