/*
 * ll_nvfp4.h — C ABI of the MI355X (gfx950) NVFP4 inference hot path.
 *
 * Every entry point takes raw device pointers, sizes and a HIP stream (as void*),
 * launches on that stream and returns 0 on success or a negative LL_E* code;
 * ll_last_error() gives the message for the calling thread.  Nothing is allocated, with
 * one exception that a caller can switch off (ll_kv_attention_set_policy).  All tensors
 * are row-major.  "bf16" means the 16-bit bit pattern.  Pointers must be valid on
 * the current HIP device.
 *
 * NVFP4 tensor format (what the reference's QuantizedTensor carries):
 *   values  u8 [Mp, Kp/2]     byte j of a row = code[2j] | code[2j+1] << 4  (e2m1 codes)
 *   scales  u8 [Mp * Kp/16]   e4m3fn block scales in the 128x4 "blocked" order:
 *                             off(r, c) = ((r/128 * (Kp/64) + c/4) * 32 + r%32) * 16 + (r%128)/32 * 4 + c%4
 *   amax    f32[1]            tensor-wide max |x|
 *   Mp = M rounded up to 128, Kp = K rounded up to 64.
 *
 * Scale-rule ids are the reference's (fouroversix/src/fouroversix/utils.py:113-122).
 */
#ifndef LL_NVFP4_H
#define LL_NVFP4_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
  LL_OK = 0,
  LL_EINVAL = -1,   /* bad shape / pointer / option */
  LL_ELAUNCH = -2,  /* HIP reported an error at launch */
  LL_ENOSUP = -3    /* valid request this build does not implement */
};

enum { LL_RULE_STATIC_6 = 0, LL_RULE_STATIC_4 = 1, LL_RULE_MAE = 2, LL_RULE_MSE = 3, LL_RULE_ABS_MAX = 4 };
enum { LL_ACT_NONE = 0, LL_ACT_GELU_TANH = 1 };
#define LL_AMAX_PARTS 1024 /* partial maxima per tensor: size of the quantizer's scratch and of an amax sink */
enum { LL_DTYPE_BF16 = 0, LL_DTYPE_F16 = 1, LL_DTYPE_F32 = 2 }; /* utils/kernel/kv_dequant.py:18-25 */

const char* ll_last_error(void);
int ll_version(void);

/*
 * Memory of the library's own.  Two kernels let several workgroups compute parts of one output tile and pass the
 * parts through device memory: the attention's split division (ll_kv_attention_set_policy) and the W4A4 GEMM at
 * sizes where whole tiles would leave compute units idle (ll_nvfp4_gemm_reserve).  That memory is allocated per
 * (device, stream) by the first launch that needs it, grown when a later launch needs more (which frees the old
 * set and so waits for the device), shared by both kernels and kept.  ll_release_stream_memory frees the set of
 * (current device, stream), if any, after waiting for the launches that still use it - for callers that create
 * streams as they go.  Launches on a stream that is being captured into a graph never allocate: they use the set a
 * reserve call or an earlier launch left on that stream, or fall back to a division of the work that needs none.
 * A set that a captured launch has used belongs to the recorded graph as well: it is not freed when the stream
 * later needs a larger one (the old set is kept aside), only by ll_release_stream_memory, which must therefore not
 * be called while such a graph may still be replayed.  No counterpart in the reference.
 */
int ll_release_stream_memory(void* stream);

/* Number of floats of scratch ll_nvfp4_quantize needs when it computes amax itself. */
size_t ll_nvfp4_quantize_workspace_floats(void);

/*
 * Replaces torch.ops.fouroversix.quantize_to_fp4 (fouroversix/src/fouroversix/csrc/bindings.cpp:28,
 * csrc/quantize/fp4_quant.cu:99-239) for is_nvfp4, round-to-nearest, no RHT / 2-D / transpose, with
 * the arithmetic of the PyTorch backend (quantize/pytorch/reference.py:242-368, backend.py:36-112).
 *   x        bf16 [M, K], row stride ldx elements
 *   values   u8 [Mp, Kp/2]      every byte written (padding rows/cols quantize zeros)
 *   scales   u8 [Mp*Kp/16]      every byte written
 *   amax     f32[1]             written unless amax_given != 0, in which case it is read: then it must cover the
 *                               tensor (blocks whose maximum exceeds it by more than a fifth would need block
 *                               scales beyond e4m3, NaN in the reference; their bytes are unspecified)
 *   workspace  f32[ll_nvfp4_quantize_workspace_floats()], may be NULL when amax_given != 0
 */
int ll_nvfp4_quantize(const void* x, int64_t M, int64_t K, int64_t ldx, int rule,
                      uint8_t* values, uint8_t* scales, float* amax, int amax_given,
                      float* workspace, void* stream);

/*
 * ll_nvfp4_quantize (amax computed by the call) for callers that cannot allocate device memory: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.
 * The scratch ll_nvfp4_quantize takes as `workspace` lives in a fixed array of LL_AMAX_PARTS floats that every GPU
 * the library runs on holds until the process ends; the call allocates and frees nothing.  Same outputs, bit for
 * bit, as ll_nvfp4_quantize with amax_given == 0.  Limits: M * K <= LL_NOALLOC_MAX_ELEMENTS (larger inputs are
 * refused with LL_EINVAL); all calls on one GPU share the array, so calls that overlap in time on one GPU (two
 * streams, two threads) race -- serialize them, or use ll_nvfp4_quantize with one workspace per stream.
 */
#define LL_NOALLOC_MAX_ELEMENTS (1ll << 32)
int64_t ll_nvfp4_quantize_noalloc_max_elements(void);
int ll_nvfp4_quantize_noalloc(const void* x, int64_t M, int64_t K, int64_t ldx, int rule,
                              uint8_t* values, uint8_t* scales, float* amax, void* stream);

/*
 * Amax sink.  The tensor-wide absolute maximum that NVFP4 quantization starts from
 * (quantize/pytorch/reference.py:242-255, x.abs().max()) costs a pass over the tensor.  A kernel of this
 * library that writes the tensor can leave the maximum behind instead: it raises LL_AMAX_PARTS 64-bit slots,
 * each (epoch << 32) | float bits, with atomic max.  A newer epoch beats every older value, so the buffer is
 * zeroed once when it is allocated and never again; every producer call on a buffer passes an epoch greater
 * than all earlier ones (1, 2, 3, ...; clear the buffer before wrapping around), and
 * ll_nvfp4_quantize_from_sink reads the slots of that epoch.  Calls that share a buffer must be ordered
 * (one stream).
 * Launches recorded into a HIP graph run again with the arguments they were recorded with, the epoch among them,
 * and would meet their own values of the previous replay.  For those, `epoch_offset` names a device word that
 * every kernel adds to `epoch` when it runs; the graph starts with ll_amax_epoch_advance, which raises that word
 * by a step larger than the number of epochs one replay uses, so every replay works with fresh epochs.  A buffer
 * used this way belongs to the graph (eager launches between replays use another buffer).
 */
typedef struct ll_amax_sink {
  uint64_t* parts;              /* device memory, LL_AMAX_PARTS entries, 8-byte aligned */
  uint32_t epoch;               /* > 0 */
  const uint32_t* epoch_offset; /* device word added to epoch at run time, or NULL */
} ll_amax_sink;

/* *epoch_offset += step on the stream (a kernel launch, recordable into a graph); when the sum would come near
 * 2^32 the word restarts from 0 and the LL_AMAX_PARTS slots of `parts` are cleared.  No counterpart in the
 * reference. */
int ll_amax_epoch_advance(uint32_t* epoch_offset, uint32_t step, uint64_t* parts, void* stream);

/* ll_nvfp4_quantize whose tensor amax comes from an amax sink that the producer of x has filled with the
 * same epoch; amax (f32[1]) is written.  The bytes equal those of ll_nvfp4_quantize with amax_given == 0. */
int ll_nvfp4_quantize_from_sink(const void* x, int64_t M, int64_t K, int64_t ldx, int rule,
                                uint8_t* values, uint8_t* scales, float* amax,
                                const ll_amax_sink* amax_sink, void* stream);

/* Two ll_nvfp4_quantize_from_sink calls on tensors of the same shape, leading dimension and rule as one launch: the
 * K and the V of a chunk on their way into the cache (wan_5b/modules/causal_model.py:1420-1429 quantizes one after
 * the other).  Each tensor has its own sink (two buffers: one launch cannot read two epochs of one buffer apart),
 * outputs and amax word; the bytes equal those of the two separate calls. */
int ll_nvfp4_quantize_pair_from_sinks(const void* x0, const void* x1, int64_t M, int64_t K, int64_t ldx, int rule,
                                      uint8_t* values0, uint8_t* values1, uint8_t* scales0, uint8_t* scales1,
                                      float* amax0, float* amax1, const ll_amax_sink* amax_sink0,
                                      const ll_amax_sink* amax_sink1, void* stream);

/*
 * Replaces QuantizedTensor.dequantize (fouroversix/src/fouroversix/quantize/quantized_tensor.py:184-214):
 * out[r, c] = cast(((e2m1 * e4m3) * amax) / (e2m1_max * e4m3_max)) for r < M, c < K; ldo in elements.
 */
int ll_nvfp4_dequantize(const uint8_t* values, const uint8_t* scales, const float* amax, int rule,
                        int64_t Mp, int64_t Kp, int64_t M, int64_t K,
                        void* out, int out_dtype, int64_t ldo, void* stream);

/*
 * Replaces torch.ops.fouroversix.gemm_nvfp4nvfp4_accum_fp32_out_bf16_tnt
 * (fouroversix/src/fouroversix/csrc/bindings.cpp:31, csrc/fp4_gemm.cu:40-186):
 *   D[m, n] = bf16(alpha * sum_k deq(A)[m, k] * deq(B)[n, k])  (+ bias[n], added in bf16 like linear.py:73-74)
 *   A_values u8 [Mp, Kp/2], A_scales blocked [Mp*Kp/16]; B_values u8 [Np, Kp/2], B_scales blocked.
 *   alpha: device f32[1], or NULL to use (*amax_a * *amax_b) / (denom_a * denom_b) as
 *          matmul/cutlass/backend.py:81-90 computes it (denom = e2m1_max * e4m3_max of each rule).
 *   D bf16 [M, N], row stride ldd; only rows < M and columns < N are written (M <= Mp, N <= Np).
 *   bias bf16 [N] or NULL.
 */
int ll_nvfp4_gemm_tnt(const uint8_t* A_values, const uint8_t* A_scales, const uint8_t* B_values,
                      const uint8_t* B_scales, const float* alpha, const float* amax_a, const float* amax_b,
                      float denom_a, float denom_b, int64_t M, int64_t N, int64_t Mp, int64_t Np, int64_t Kp,
                      void* D, int64_t ldd, const void* bias, void* stream);

/*
 * ll_nvfp4_gemm_tnt with an activation applied to the bf16 result (after the bias) in the epilogue, for the
 * Linear -> GELU(tanh) pair of the DiT feed-forward (wan_5b/modules/causal_model.py:822-824):
 *   D = bf16(act(f32(bf16(bf16(alpha * acc) + bias))));  activation: LL_ACT_NONE or LL_ACT_GELU_TANH.
 */
int ll_nvfp4_gemm_tnt_act(const uint8_t* A_values, const uint8_t* A_scales, const uint8_t* B_values,
                          const uint8_t* B_scales, const float* alpha, const float* amax_a, const float* amax_b,
                          float denom_a, float denom_b, int64_t M, int64_t N, int64_t Mp, int64_t Np, int64_t Kp,
                          void* D, int64_t ldd, const void* bias, int activation, void* stream);

/*
 * ll_nvfp4_gemm_tnt with the element-wise operations that follow a projection in the DiT block folded into
 * the epilogue.  With y = bf16(alpha * acc) the steps are, in this order and each optional:
 *   y = bf16(y + bias[n])                                   (model/modules/linear.py:73-74)
 *   y = bf16(act(y))                                         (causal_model.py:822-824, nn.GELU(approximate="tanh"))
 *   y = bf16(y * gate[m / gate_rows, n])   only with residual (causal_model.py:889, 919-920: y * e[2] / e[5])
 *   y = bf16(residual[m, n] + y)                             (causal_model.py:889, 906, 919-920: x + ...)
 *   max |y| goes to amax_sink (see ll_amax_sink) when amax_sink.parts is not NULL.
 * Every rounding is the one the separate bf16 operations of the reference perform.
 *   gate bf16, row stride gate_stride elements; residual bf16 [M, N], row stride ldr; both 16-byte aligned,
 *   strides multiples of 8, and N a multiple of 8 when a residual is given.  residual may alias D.
 */
typedef struct ll_gemm_epilogue {
  const void* bias;       /* bf16 [N] or NULL */
  int activation;         /* LL_ACT_NONE or LL_ACT_GELU_TANH */
  const void* gate;       /* bf16 or NULL (needs residual) */
  int64_t gate_rows;      /* rows of D that share one gate row */
  int64_t gate_stride;
  const void* residual;   /* bf16 [M, N] or NULL */
  int64_t ldr;
  ll_amax_sink amax_sink; /* parts == NULL: none */
} ll_gemm_epilogue;
int ll_nvfp4_gemm_tnt_fused(const uint8_t* A_values, const uint8_t* A_scales, const uint8_t* B_values,
                            const uint8_t* B_scales, const float* alpha, const float* amax_a, const float* amax_b,
                            float denom_a, float denom_b, int64_t M, int64_t N, int64_t Mp, int64_t Np, int64_t Kp,
                            void* D, int64_t ldd, const ll_gemm_epilogue* epilogue, void* stream);

/*
 * Several ll_nvfp4_gemm_tnt products with the same A operand and the same N and Kp in one launch: the q, k and v
 * projections of one activation (wan_5b/modules/causal_model.py:363-365) and the k, v projections of the text
 * (:234-235), three resp. two fp4_matmul calls in the reference.  Each product has its own weight, scales, tensor
 * scale, bias, output and amax sink (bias and sink optional, as in ll_gemm_epilogue); product i computes exactly
 * what ll_nvfp4_gemm_tnt_fused computes for it alone, bit for bit.  1 <= n_products <= 4.
 */
typedef struct ll_gemm_product {
  const uint8_t* B_values;
  const uint8_t* B_scales;
  const float* alpha;     /* f32[1] or NULL: then amax_a * amax_b / (denom_a * denom_b) */
  const float* amax_b;
  float denom_b;
  void* D;                /* bf16 [M, ldd] */
  int64_t ldd;
  const void* bias;       /* bf16 [N] or NULL */
  ll_amax_sink amax_sink; /* parts == NULL: none */
} ll_gemm_product;
int ll_nvfp4_gemm_tnt_grouped(const uint8_t* A_values, const uint8_t* A_scales, const float* amax_a, float denom_a,
                              int64_t M, int64_t N, int64_t Mp, int64_t Np, int64_t Kp, int n_products,
                              const ll_gemm_product* products, void* stream);

/*
 * The GEMM entry points can run one of two kernels.  LL_GEMM_TILES: one workgroup per output tile, two workgroups
 * per compute unit; where Kp is a multiple of 128, the tiles of 256 x 128 and 128 x 256 run their main loop as a
 * hand-scheduled instruction sequence (same arithmetic in the same order as the compiled loop: identical bits), and
 * a shape that gives at most one 128 x 256 tile per compute unit (and fills more than half of them) runs as one
 * workgroup of eight waves per tile, which sums the two halves of every K step of 128 separately and adds them at
 * the end (deterministic; differs from the other kernels by the order of the fp32 additions).
 * LL_GEMM_TILES_COMPILED takes the compiled loop and one workgroup of four waves per tile everywhere, for
 * comparisons.  LL_GEMM_PERSISTENT (wherever Kp is a multiple of 128 and there is at least one K step per
 * compute unit): one workgroup per compute unit, output tiles of 128 x 512, whole rounds of tiles first and the
 * (tile, K step) pairs of the tiles behind them cut into equal shares, so that no compute unit waits for another
 * (the reference's kernel is a persistent tile scheduler too, csrc/fp4_gemm.cu:67-92).  A tile whose K range is
 * shared by several workgroups is summed from their fp32 partial tiles in a fixed order, so results are
 * deterministic; they differ from the other kernel's by the order of the fp32 additions only.  The partial tiles
 * pass through memory of the library's own (see ll_release_stream_memory; 2 x 256 KB per compute unit).
 * ll_nvfp4_gemm_reserve sets that memory up ahead of a launch of the given sizes (n_products = 1 for the plain
 * entry points) and does nothing when such a launch would take the other kernel; on a capturing stream without it,
 * a launch takes the other kernel.  LL_GEMM_AUTO (initial) takes the faster of the two as measured on MI355X,
 * which at the sizes of the DiT block is LL_GEMM_TILES throughout.  ll_nvfp4_gemm_set_schedule is process-wide.
 */
#define LL_GEMM_AUTO (-1)
#define LL_GEMM_TILES 0
#define LL_GEMM_PERSISTENT 1
#define LL_GEMM_TILES_COMPILED 2
int ll_nvfp4_gemm_set_schedule(int schedule);
int ll_nvfp4_gemm_get_schedule(void);
int ll_nvfp4_gemm_reserve(int64_t M, int64_t N, int64_t Kp, int n_products, void* stream);
/* What a launch of these sizes would do on a device with `compute_units` CUs under `schedule` (host arithmetic
 * only): *persistent = 1 and the numbers of workgroups, output tiles and K steps per tile, or *persistent = 0.
 * Output pointers may be NULL. */
int ll_nvfp4_gemm_plan(int64_t M, int64_t N, int64_t Kp, int n_products, int compute_units, int schedule,
                       int* persistent, uint32_t* workgroups, uint32_t* tiles, uint32_t* k_steps);
/* Which kernel a launch of these sizes runs on a device with `compute_units` CUs under `schedule` (host arithmetic
 * only; a persistent launch on a capturing stream without memory falls back to the tile kernels, which this does not
 * see): *kernel = one of the codes below, *hand_scheduled = 1 if its main loop is the generated instruction sequence.
 * The four-wave tile kernels add the K steps in order; LL_GEMM_KERNEL_EIGHT_WAVES and LL_GEMM_KERNEL_PERSISTENT form
 * partial sums over parts of K.  Output pointers may be NULL.  No counterpart in the reference. */
#define LL_GEMM_KERNEL_64X64 0       /* four waves per tile, two workgroups per compute unit */
#define LL_GEMM_KERNEL_128X128 1
#define LL_GEMM_KERNEL_128X256 2
#define LL_GEMM_KERNEL_256X128 3
#define LL_GEMM_KERNEL_EIGHT_WAVES 4 /* 128 x 256 tiles, eight waves per tile, one workgroup per compute unit */
#define LL_GEMM_KERNEL_PERSISTENT 5  /* 128 x 512 tiles, one workgroup per compute unit over several tiles */
int ll_nvfp4_gemm_kernel(int64_t M, int64_t N, int64_t Kp, int n_products, int compute_units, int schedule, int* kernel,
                         int* hand_scheduled);

/*
 * Replaces torch.ops.longlive_kernels.dequantize_kv_cache_fp4 (utils/kernel/kv_dequant.cpp:14,
 * utils/kernel/kv_dequant_cuda.cu:59-239): n_blocks cache slots, each NVFP4 [rows_padded, 128] holding
 * block_token_size*num_heads logical rows, are dequantized to out[1, n_blocks*block_token_size, num_heads, 128]
 * as cast((f32(e2m1) * f32(scale)) * gs) with the slot scale gs = amax * f32(1.0 / (e2m1_max*e4m3_max)), the
 * reciprocal formed in double (kv_dequant_cuda.cu:95-106, 216).  The Triton routine the reference falls back to
 * when its extension is not built (utils/nvfp4_kernel.py:40-176 with utils/quant.py:753-756) divides amax by the
 * denominator instead, which moves gs by at most one fp32 ulp; the fused path is the one followed here, by this
 * entry point and by ll_kv_attention alike.
 *   values_ptrs / scales_ptrs / amax_ptrs: DEVICE arrays of n_blocks device pointers.
 */
int ll_kv_dequantize_blocks(const uint64_t* values_ptrs, const uint64_t* scales_ptrs, const uint64_t* amax_ptrs,
                            int n_blocks, int num_heads, int block_token_size, int out_dtype,
                            float e2m1_max, float e4m3_max, void* out, void* stream);

/*
 * FP4 KV-cache attention for one chunk; replaces dequantize_kv_cache + slice copies + flash attention
 * (wan_5b/modules/causal_model.py:557-567, 628-671, 673-724, 781; wan_5b/modules/attention.py:84-306):
 *   out[t, h, :] = softmax_j(q[t, h, :] . k_j[h, :] * scale) v_j   over the key list
 *       [ n_cached tokens read from the NVFP4 slots (slot = j / block_token_size) | n_new bf16 tokens ]
 *   Cached keys and values enter the products as the bf16 values ll_kv_dequantize_blocks(..., LL_DTYPE_BF16)
 *   returns for the same slots, bit for bit.
 *   q bf16 [Lq, H, 128]; k_new, v_new bf16 [n_new, H, 128] (the caller passes the smoothed K of the
 *   current chunk, utils/quant.py:797-798); out bf16 [Lq, H, 128].  No mask (causal_model.py:781).
 *   k_* / v_* pointer arrays: DEVICE arrays of device pointers, one per slot, slot layout as above
 *   (rows = token*H + head, 128 columns).  Any n_cached >= 0 and n_new >= 0 with n_cached + n_new >= 1.
 */
int ll_kv_attention(const void* q, int64_t Lq, int num_heads,
                    const uint64_t* k_values_ptrs, const uint64_t* k_scales_ptrs, const uint64_t* k_amax_ptrs,
                    const uint64_t* v_values_ptrs, const uint64_t* v_scales_ptrs, const uint64_t* v_amax_ptrs,
                    int64_t n_cached, int block_token_size, float e2m1_max, float e4m3_max,
                    const void* k_new, const void* v_new, int64_t n_new,
                    float softmax_scale, void* out, void* stream);

/* ll_kv_attention that also leaves max |out| in amax_sink (may be NULL), for the quantization in front of the
 * output projection (causal_model.py:783-785 feeds FourOverSixLinear.forward, model/modules/linear.py:243-270). */
int ll_kv_attention_amax(const void* q, int64_t Lq, int num_heads,
                         const uint64_t* k_values_ptrs, const uint64_t* k_scales_ptrs, const uint64_t* k_amax_ptrs,
                         const uint64_t* v_values_ptrs, const uint64_t* v_scales_ptrs, const uint64_t* v_amax_ptrs,
                         int64_t n_cached, int block_token_size, float e2m1_max, float e4m3_max,
                         const void* k_new, const void* v_new, int64_t n_new,
                         float softmax_scale, void* out, const ll_amax_sink* amax_sink, void* stream);

/*
 * How ll_kv_attention / ll_kv_attention_amax / ll_attention_bf16 divide a launch between workgroups.  No
 * counterpart in the reference (it calls flash attention).  LL_ATTENTION_AUTO, the initial setting, picks per
 * launch the cheapest of the three by a cost estimate:
 *   LL_ATTENTION_NARROW  one workgroup per (head, 128 queries);
 *   LL_ATTENTION_WIDE    one workgroup per (head, 256 queries): every decoded K/V tile serves twice as many MFMAs;
 *   LL_ATTENTION_SPLIT   256-query tiles; what does not fill whole rounds of one tile per compute unit is cut
 *                        along the key range into shares of equal cost (a head's last, partly filled group of
 *                        queries counts for less), so that no compute unit waits for another.  Tiles shared by two
 *                        workgroups pass through device memory that the library allocates on the first such
 *                        launch on a (device, stream) pair and keeps (69 MB on a 256-CU device); launches that
 *                        use it must not overlap on one stream's memory, which same-stream order guarantees.
 * The three give the same result up to the order of fp32 additions (each is deterministic).  The setting is
 * process-wide.  A launch on a stream that is being captured into a graph never allocates: it uses the memory an
 * earlier launch or ll_kv_attention_reserve left on that stream, and without such memory the automatic choice
 * takes the cheaper of NARROW and WIDE while an explicit LL_ATTENTION_SPLIT returns LL_ENOSUP.
 */
#define LL_ATTENTION_AUTO (-1)
#define LL_ATTENTION_NARROW 0
#define LL_ATTENTION_WIDE 1
#define LL_ATTENTION_SPLIT 2
int ll_kv_attention_set_policy(int policy); /* LL_OK, or LL_EINVAL for an unknown policy */
int ll_kv_attention_get_policy(void);
/* Sets up, on (current device, stream), the memory that a launch of Lq queries x num_heads heads over n_keys keys
 * would need under the current policy (nothing when that launch would not take the split division), so that the
 * launch itself allocates nothing: call it ahead of a graph recording or a latency-critical loop.  May allocate,
 * and may free a smaller set (which waits for the device).  LL_ENOSUP while the stream is being captured.  No
 * counterpart in the reference. */
int ll_kv_attention_reserve(int64_t Lq, int num_heads, int64_t n_keys, void* stream);
/* ll_release_stream_memory under its first name. */
int ll_kv_attention_release(void* stream);
/* What a launch of Lq queries x num_heads heads over n_keys keys would do on a device with `compute_units` CUs
 * under `policy` (pure host arithmetic, no GPU needed): the division taken (an LL_ATTENTION_SPLIT request falls
 * back to WIDE when there is nothing to split), the number of workgroups, the whole rounds of tiles all of them
 * run first and the number of tiles cut into shares (tiles behind the whole rounds that are not counted here run
 * whole on workgroups that take no share).  Lets a caller know ahead of a launch whether it will
 * take the allocating division.  Output pointers may be NULL. */
int ll_kv_attention_plan(int64_t Lq, int num_heads, int64_t n_keys, int compute_units, int policy,
                         int* division, uint32_t* workgroups, uint32_t* whole_rounds, int64_t* split_tiles);

/* Plain bf16 attention (cross-attention to the text context; wan_5b/modules/causal_model.py:197-262):
 * q [Lq,H,128], k/v [Lk,H,128], out [Lq,H,128], no mask. */
int ll_attention_bf16(const void* q, const void* k, const void* v, int64_t Lq, int64_t Lk, int num_heads,
                      float softmax_scale, void* out, void* stream);

/*
 * Replaces rope_apply_triton (utils/rope_triton.py:36-135): x bf16 [S, N, D] (strides in elements, last
 * dim contiguous), cos/sin f32 [seq_len, D/2]; rows < seq_len are rotated in fp32, the rest copied.
 */
int ll_rope_apply(const void* x, int64_t S, int N, int D, int64_t x_stride_s, int64_t x_stride_n,
                  const float* cos, const float* sin, int64_t seq_len, void* out, void* stream);

/*
 * Replaces adaln_modulate_triton (utils/adaln_triton.py:36-126): x bf16 [B, L, C] contiguous,
 * scale/shift bf16 indexed [b, l / frame_seqlen, :] with the given strides (elements);
 * y = bf16(bf16(LN(x)) * bf16(1 + scale)) + shift.
 */
int ll_adaln_modulate(const void* x, int64_t B, int64_t L, int C, const void* scale, const void* shift,
                      int64_t scale_stride_b, int64_t scale_stride_f, int64_t shift_stride_b, int64_t shift_stride_f,
                      int64_t frame_seqlen, float eps, int add_one_to_scale, void* out, void* stream);

/* ll_adaln_modulate that also leaves max |y| in amax_sink (may be NULL), for the quantization that follows
 * (causal_model.py:869-878, 909-918). */
int ll_adaln_modulate_amax(const void* x, int64_t B, int64_t L, int C, const void* scale, const void* shift,
                           int64_t scale_stride_b, int64_t scale_stride_f, int64_t shift_stride_b,
                           int64_t shift_stride_f, int64_t frame_seqlen, float eps, int add_one_to_scale, void* out,
                           const ll_amax_sink* amax_sink, void* stream);

/*
 * Gated residual of the DiT block (wan_5b/modules/causal_model.py:889, 919-920):
 *   out = bf16(x + bf16(y * gate[b, l / frame_seqlen, :]));  x, y, out bf16 [B, L, C] contiguous, gate bf16 with
 *   the given strides (elements).  out may alias x.
 */
int ll_gate_residual(const void* x, const void* y, int64_t B, int64_t L, int C, const void* gate,
                     int64_t gate_stride_b, int64_t gate_stride_f, int64_t frame_seqlen, void* out, void* stream);

/* WanLayerNorm with elementwise affine (wan_5b/modules/model.py:101-111, used as norm3 ahead of cross-attention,
 * wan_5b/modules/causal_model.py:892-906): y = bf16(((x - mean) * rsqrt(var + eps)) * w + b) over the last dim C of
 * x bf16 [rows, C], statistics and affine map in fp32; weight / bias bf16 [C], either may be NULL (1 / 0).
 * amax_sink (may be NULL) receives the absolute maximum of y, see ll_amax_sink. */
int ll_layer_norm(const void* x, int64_t rows, int C, const void* weight, const void* bias, float eps, void* out,
                  const ll_amax_sink* amax_sink, void* stream);

/*
 * ll_adaln_modulate_amax followed by ll_nvfp4_quantize_from_sink of its result (the pairs at
 * wan_5b/modules/causal_model.py:869-878 and :909-918 with a quantized linear layer behind them) as one launch that
 * never writes the modulated tensor: values [Mp, C/2], scales [Mp * C / 16] in the blocked layout and amax [1] are
 * byte for byte what the two calls give (M = B * L rows, Mp = M rounded up to 128).  The launch is one resident
 * grid whose workgroups exchange their maxima through amax_sink (required: a buffer of LL_AMAX_PARTS slots and a
 * fresh epoch, as for ll_adaln_modulate_amax; nothing has to read it afterwards).  A workgroup waits for the others
 * at most spin_limit + 1 looks at the slots (one to two microseconds each; with the device to itself a launch's
 * workgroups arrive within ~10 us of each other, and 64 is plenty) and then computes the maxima of the rows of the
 * workgroups it has not seen itself, so the launch ends whatever else occupies the device (another stream may hold
 * compute units for milliseconds) and costs at most one extra pass over the rows; spin_limit < 0 makes every
 * workgroup do that (tests of that path).  LL_ENOSUP when C is not a multiple of 64 or exceeds 3072, or when the
 * device does not hold one wave per row of Mp at once (3072 rows on 256 compute units; with more rows per wave the
 * launch was measured no faster than the two kernels): call the two separate entry points then.  No allocation, safe
 * under stream capture.
 */
int ll_adaln_quantize(const void* x, int64_t B, int64_t L, int C, const void* scale, const void* shift,
                      int64_t scale_stride_b, int64_t scale_stride_f, int64_t shift_stride_b, int64_t shift_stride_f,
                      int64_t frame_seqlen, float eps, int add_one_to_scale, int rule, uint8_t* values,
                      uint8_t* scales, float* amax, const ll_amax_sink* amax_sink, int64_t spin_limit, void* stream);

/* ll_layer_norm followed by ll_nvfp4_quantize_from_sink of its result (norm3 ahead of the cross-attention query
 * projection, wan_5b/modules/causal_model.py:892-906) as one launch; everything else as ll_adaln_quantize. */
int ll_layer_norm_quantize(const void* x, int64_t rows, int C, const void* weight, const void* bias, float eps,
                           int rule, uint8_t* values, uint8_t* scales, float* amax, const ll_amax_sink* amax_sink,
                           int64_t spin_limit, void* stream);

/* WanRMSNorm (wan_5b/modules/model.py:82-98): y = bf16(bf16(x * rsqrt(mean(x^2) + eps)) * w) over the
 * last dim C of x bf16 [rows, C]; w bf16 [C]. */
int ll_rms_norm(const void* x, int64_t rows, int C, const void* weight, float eps, void* out, void* stream);

/*
 * q / k path between the projections and attention in one pass (wan_5b/modules/causal_model.py:362-368,
 * 477-487; utils/quant.py:797-798): WanRMSNorm over rows of num_heads*128 channels, then the rotary embedding
 * per head (rows < seq_len; cos/sin f32 [seq_len, 64]), with the roundings of ll_rms_norm followed by
 * ll_rope_apply.  out bf16 [rows, num_heads, 128]; out_smooth (may be NULL) receives
 * bf16(out - bf16(mean of out over the 128 channels of the head)), the K handed to attention for the current chunk.
 */
int ll_qk_norm_rope(const void* x, int64_t rows, int num_heads, const void* weight, float eps, const float* cos,
                    const float* sin, int64_t seq_len, void* out, void* out_smooth, void* stream);

/* ll_qk_norm_rope for q and k of one attention layer in a single launch (same rows, heads, eps and angles;
 * one weight each); k_out_smooth may be NULL. */
int ll_qk_norm_rope_pair(const void* q, const void* k, int64_t rows, int num_heads, const void* q_weight,
                         const void* k_weight, float eps, const float* cos, const float* sin, int64_t seq_len,
                         void* q_out, void* k_out, void* k_out_smooth, void* stream);

/* ll_qk_norm_rope_pair that also leaves max |k_out| in k_amax_sink (may be NULL): k_out is what the cache
 * quantizes when the chunk is written (wan_5b/modules/causal_model.py:1406-1429), and with the maximum at hand
 * that quantization needs no pass of its own over the tensor to find it. */
int ll_qk_norm_rope_pair_amax(const void* q, const void* k, int64_t rows, int num_heads, const void* q_weight,
                              const void* k_weight, float eps, const float* cos, const float* sin, int64_t seq_len,
                              void* q_out, void* k_out, void* k_out_smooth, const ll_amax_sink* k_amax_sink,
                              void* stream);

#ifdef __cplusplus
}
#endif
#endif /* LL_NVFP4_H */
