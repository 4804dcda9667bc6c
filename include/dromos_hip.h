/*
 * libdromos_hip.so: the decode matrix-product path of Dromos on MI355X (gfx950), as a drop-in backend
 * library. Every symbol below keeps the name, signature, argument meaning and status codes of the
 * reference's backend ABI, so the engine's dispatch layer (engine/dispatch/dispatch.cpp:43-56,162-235,
 * which already knows "libdromos_hip.so") binds it with dlsym and calls it unchanged. A symbol of the
 * reference ABI that is not declared here is simply absent from the library: the dispatch stubs answer
 * LX_ERR_NOT_SUPPORTED (801) for it (tools/gen_dispatch.py:168-184).
 *
 * Conventions (engine/cuda/kernels.h:1-4,27-38,294-302):
 *   - return value: 0 ok, 1 invalid value, 2 out of memory, 801 not supported; checked before any launch
 *   - tensor pointers are device pointers to row-major buffers owned by the caller; an lx_weight* is a
 *     host pointer to a struct whose fields are device pointers
 *   - `stream` is a hipStream_t (null = the default stream); calls are asynchronous, and the decode
 *     calls neither allocate nor synchronise, so they can be captured in a graph
 */
#ifndef DROMOS_HIP_H_
#define DROMOS_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#ifndef LX_API
#define LX_API __attribute__((visibility("default")))
#endif

/* engine/cuda/kernels.h:27 */
typedef enum { LX_F32 = 0, LX_BF16 = 1 } lx_dtype;
/* engine/cuda/kernels.h:243 (LX_W_BF16X: the lossless form of bf16 below; lx_gemm_w and the grouped experts answer 801 for it) */
typedef enum { LX_W_BF16 = 0, LX_W_INT8 = 1, LX_W_FP8 = 2, LX_W_NVFP4 = 3, LX_W_BF16X = 4 } lx_wtype;
/* engine/cuda/kernels.h:431 */
typedef enum { LX_MATH_BF16 = 0, LX_MATH_INT8 = 1, LX_MATH_FP8 = 2, LX_MATH_FP4 = 3 } lx_math;
/* engine/cuda/kernels.h:302-306 */
#define LX_ERR_NOT_SUPPORTED 801
typedef enum { LX_BACKEND_CUDA = 0, LX_BACKEND_HIP = 1, LX_BACKEND_METAL = 2, LX_BACKEND_CPU = 3 } lx_backend;
typedef enum { LX_COPY_H2D = 0, LX_COPY_D2H = 1, LX_COPY_D2D = 2, LX_COPY_DEFAULT = 3 } lx_copy_kind;
/* engine/cuda/tunable.h:27-32 */
#define LX_ERR_TUNE_REJECTED 802
#define LX_ERR_TUNE_VARIANT 803

/*
 * One weight in one format, row-major [N, K], K contiguous (engine/cuda/kernels.h:383-417):
 *   LX_W_BF16   data bf16 [N, K]
 *   LX_W_INT8   data int8 [N, K], scale f32 [N]            w = q * scale[n]
 *   LX_W_FP8    data e4m3fn [N, K], scale f32 [N]          w = fp8 * scale[n]
 *   LX_W_NVFP4  data u8 [N, K/2] (low nibble = even k), scale e4m3 [N, K/16], global f32
 *                                                          w = e2m1 * scale[n, k/16] * global
 *   LX_W_BF16X  data the encoding lx_bf16x_encode writes of bf16 [N, K] (8-byte aligned); no scale
 * A stack of experts is [E, N, K] laid out expert after expert (scales likewise); an NVFP4 stack may
 * carry one global per expert in expert_global (f32 [E] on the device, null = `global` for all).
 */
typedef struct {
  lx_wtype type;
  const void* data;
  const void* scale;
  float global;
  const float* expert_global;
} lx_weight;

/* ---- decode GEMV, M <= 8 (replaces engine/cuda/kernels.h:235-246, 433-438, 594-596) ---------------
 *   y[m, n] = alpha * (rowfactor[n] * sum_k x[m, k] * w[n, k] + bias[n]) + beta * y[m, n]
 * x [M, K] f32 or bf16 (row stride ld_x elements); bias [N] f32 / bf16 or null; y [M, N] f32 / bf16
 * (row stride ld_y), read only when beta != 0. Weight-only: weights are expanded exactly in registers,
 * sums are f32, deterministic, and a row's bits do not depend on M or on the other rows.
 * M > 8 or bad arguments -> 1; M == 0 or N == 0 -> 0 with nothing touched. */
LX_API int lx_gemv(const void* x, lx_dtype x_dtype, int ld_x, const void* w, lx_wtype w_type, const float* w_scale,
                   const void* bias, lx_dtype bias_dtype, void* y, lx_dtype y_dtype, int ld_y, int M, int N, int K,
                   float alpha, float beta, void* stream);
LX_API int lx_gemv_w(const void* x, lx_dtype x_dtype, int ld_x, const lx_weight* w, const void* bias,
                     lx_dtype bias_dtype, void* y, lx_dtype y_dtype, int ld_y, int M, int N, int K, float alpha,
                     float beta, void* stream);
LX_API int lx_gemv_decode_bf16(const void* x, lx_dtype x_dtype, int ld_x, const void* w, const void* bias,
                               lx_dtype bias_dtype, void* y, lx_dtype y_dtype, int ld_y, int M, int N, int K,
                               float alpha, float beta, void* stream);

/* ---- batched decode products (replaces engine/cuda/kernels.h:440-451 and 453-477) ----------------
 * lx_gemm_w: any M, the same product with `math` (engine/cpu/gemm.cpp:189-296):
 *   LX_MATH_BF16  any weight format: activations rounded to bf16, weights expanded exactly to bf16, f32 sums on
 *                 the matrix cores; the workspace is not used (may be null)
 *   LX_MATH_INT8  int8 weights: activations quantised per token to int8 inside the call (lx_quantize_act's rule),
 *                 exact int32 sums; other weight formats answer 801
 *   LX_MATH_FP8   fp8 or NVFP4 weights: activations quantised per token to e4m3, exact products, f32 sums
 *   LX_MATH_FP4   NVFP4 weights (K % 16 == 0): activations quantised per token to e2m1 with e4m3 block scales,
 *                 exact products, f32 sums
 * Any other pair of math and weight format answers 801 (engine/cpu/gemm.cpp:195-212).
 * The quantised maths keep the activations' scales and bytes in the workspace (lx_gemm_workspace_bytes); with a
 * null workspace they take scratch from the stream's memory pool instead (hipMallocAsync / hipFreeAsync, as the
 * reference's kernels do: such a call allocates and cannot be captured in a graph).
 * For some shapes (17 .. 64 rows, few weight tiles) the product is split over K between workgroups and a second
 * kernel adds the partial sums in the fixed order: their memory is a buffer of 64 MiB that the library makes once
 * per (device, stream), on the first such call outside a graph capture, and keeps until the process ends. Calls on
 * one stream share it (they run one after the other); a graph captured with such a call must be launched on the
 * stream it was captured on, or not at the same time as other lx_gemm_w calls there.
 * lx_gemm_skinny: bf16 x, up to 64 rows per pass, every format, with the reduction-order contract of
 * engine/cuda/kernels.h:457-474: the K split depends on (N, K) only, never on M, so a row's bits do not
 * depend on the batch. With the environment variable LX_BATCH_INVARIANT set (non-empty, not starting
 * with '0'; read on every call, engine/cuda/common.cuh:66-73) lx_gemv_w with bf16 x and lx_gemm_w run
 * this same kernel, so a row's bits are the same for every row count from 1 up. */
LX_API int lx_gemm_w(const void* x, lx_dtype x_dtype, int ld_x, const lx_weight* w, lx_math math, const void* bias,
                     lx_dtype bias_dtype, void* y, lx_dtype y_dtype, int ld_y, int M, int N, int K, float alpha,
                     float beta, void* workspace, void* stream);
LX_API int64_t lx_gemm_workspace_bytes(int M, int K, lx_math math);
LX_API int lx_gemm_skinny(const void* x, lx_dtype x_dtype, int ld_x, const lx_weight* w, const void* bias,
                          lx_dtype bias_dtype, void* y, lx_dtype y_dtype, int ld_y, int M, int N, int K, float alpha,
                          float beta, void* stream);

/* ---- weight quantisers (replaces engine/cuda/kernels.h:248-251, 513-523) -------------------------
 * Round-to-nearest-even, IEEE f32 divisions, bytes identical to the reference's CPU quantisers
 * (engine/cpu/quant.cpp:66-140). NVFP4 writes the tensor's global back to out->global (synchronises
 * the stream once: load time only). lx_dequantize_weight: out[n, k] = bf16(element * row factor). */
LX_API int lx_quantize_w8(const void* w, int8_t* q, float* scale, int64_t rows, int cols, void* stream);
LX_API int lx_quantize_weight(const void* w, lx_weight* out, int64_t rows, int cols, void* stream);
LX_API int lx_dequantize_weight(const lx_weight* w, void* out, int64_t rows, int cols, void* stream);

/* ---- per-token activation quantiser (replaces engine/cuda/kernels.h:479-493) ---------------------------
 * x [M, K] (x_dtype, row stride ld_x). Per row, a = max |x|: INT8 q = rne(x * (127 / a)) clamped to +-127,
 * scale[m] = a / 127; FP8 q = e4m3(x * (448 / a)), scale[m] = a / 448; FP4 (K % 16 == 0) two e2m1 per byte,
 * block_scale e4m3 [M, ld_bs] one per 16 k, scale[m] = g = a / 2688, s_b = e4m3(a_b / (6 g)),
 * q = e2m1(x * (1 / (s_b g))), 0 where s_b = 0. A zero row: scale 1, q = 0. ld_q and ld_bs are in bytes.
 * Bytes identical to engine/cpu/quant.cpp:159-203. lx_gemm_w's INT8 and FP8 maths quantise their activations by
 * these rules. */
LX_API int lx_quantize_act(const void* x, lx_dtype x_dtype, int ld_x, lx_math math, void* q, int ld_q, float* scale,
                           void* block_scale, int ld_bs, int M, int K, void* stream);

/* ---- routing and routed experts (replaces engine/cuda/kernels.h:203-209, 220-225, 495-511, 606-611)
 * lx_moe_route: per row of f32 logits [T, E]: entropy and confidence of the softmax, ids = top_k by
 * logit + selection_bias (ties to the lower index), weights = softmax of the picked unbiased logits.
 * Experts: out[t, :] = sum_k weights[t, k] * down[e] @ bf16(silu(gate[e] @ x) * (up[e] @ x)), e =
 * ids[t, k]; latent bf16 [T, L]; gate_up [E, 2I, L] (gate rows first); down [E, L, I]; out f32 [T, L],
 * written once; the k terms are added in slot order. The pairs are grouped by expert on the device
 * (counting sort + prefix-summed offset table in the workspace): no host round trip.
 *   lx_moe_experts_decode   T <= 8, top_k <= 8, weight-only f32 math
 *   lx_moe_experts_grouped  any T, on the matrix cores, E <= 1024; LX_MATH_BF16 on any stacks, LX_MATH_INT8 on int8
 *                           stacks, LX_MATH_FP8 on fp8 or NVFP4 stacks, LX_MATH_FP4 on NVFP4 stacks (the latent rows are
 *                           quantised per token and the intermediate rows per pair by lx_quantize_act's rule; other
 *                           pairs answer 801, engine/cpu/moe.cpp:555-569)
 *   lx_moe_experts / lx_moe_experts_decode_bf16   the bf16-stack forms of the two (lx_moe_experts takes the decode
 *                           kernels for T <= 8, top_k <= 8 and is then lx_moe_experts_decode_bf16 to the bit, the
 *                           grouped kernels otherwise; its workspace comes from hipMallocAsync on the stream) */
LX_API int lx_moe_route(const float* logits, const float* selection_bias, int32_t* ids, float* weights,
                        float* entropy, float* confidence, int T, int E, int top_k, void* stream);
LX_API int lx_moe_experts(const void* latent, const int32_t* ids, const float* weights, const void* gate_up,
                          const void* down, float* out, int T, int L, int I, int top_k, void* stream);
LX_API int lx_moe_experts_decode(const void* latent, const int32_t* ids, const float* weights,
                                 const lx_weight* gate_up, const lx_weight* down, float* out, void* workspace, int T,
                                 int L, int I, int top_k, void* stream);
LX_API int64_t lx_moe_decode_workspace_bytes(int T, int I, int top_k);
LX_API int lx_moe_experts_decode_bf16(const void* latent, const int32_t* ids, const float* weights,
                                      const void* gate_up, const void* down, float* out, void* workspace, int T,
                                      int L, int I, int top_k, void* stream);
LX_API int64_t lx_moe_bf16x_workspace_bytes(int T, int I, int top_k);

/* ---- lossless bf16, LX_W_BF16X (replaces engine/cuda/kernels.h:567-611; CPU behaviour: engine/cpu/bf16x.cpp,
 * engine/cpu/gemm.cpp:364-371, engine/cpu/moe.cpp:480-494) --------------------------------------------
 * bf16 weights in about 12.2 bits a value, every bit kept: a value is one sign|mantissa byte and a 4-bit exponent
 * code below the largest exponent of its span of 128 values; the rare value out of that range is listed in the
 * row's header. The encoder writes the reference's bytes exactly, so encoded checkpoints are interchangeable.
 *   lx_bf16x_row_bytes   bytes of one encoded row of K values (-1 unless 0 < K < 2^23)
 *   lx_bf16x_bytes       bytes the encoding of w (bf16 [rows, K] on the device) needs: rows * row bytes plus the spill
 *                        records of rows with more exceptions than header slots; -1 on bad arguments. Synchronizes.
 *   lx_bf16x_encode      w -> out (8-byte aligned, out_bytes >= lx_bf16x_bytes); deterministic; synchronizes once,
 *                        scratch from hipMallocAsync: load time, not graph capture
 *   lx_bf16x_decode      the encoding back to bf16 [rows, K]
 *   lx_gemv_bf16x        lx_gemv's contract on encoded rows; y is lx_gemv_decode_bf16's on the original weights to
 *                        the bit (same lanes, steps, split and summation order), so a row's bits do not depend on M
 *   lx_moe_experts_bf16x lx_moe_experts_decode_bf16's contract (any T, top_k <= 8, workspace of
 *                        lx_moe_bf16x_workspace_bytes) on encoded stacks [E, 2I, L] and [E, L, I]; out equals
 *                        lx_moe_experts_decode_bf16's on the original stacks to the bit. Nothing is allocated. */
LX_API int64_t lx_bf16x_row_bytes(int K);
LX_API int64_t lx_bf16x_bytes(const void* w, int64_t rows, int K, void* stream);
LX_API int lx_bf16x_encode(const void* w, int64_t rows, int K, void* out, int64_t out_bytes, void* stream);
LX_API int lx_bf16x_decode(const void* data, int64_t rows, int K, void* w, void* stream);
LX_API int lx_gemv_bf16x(const void* x, lx_dtype x_dtype, int ld_x, const void* w, const void* bias,
                         lx_dtype bias_dtype, void* y, lx_dtype y_dtype, int ld_y, int M, int N, int K, float alpha,
                         float beta, void* stream);
LX_API int lx_moe_experts_bf16x(const void* latent, const int32_t* ids, const float* weights, const void* gate_up,
                                const void* down, float* out, void* workspace, int T, int L, int I, int top_k,
                                void* stream);
LX_API int lx_moe_experts_grouped(const void* latent, const int32_t* ids, const float* weights,
                                  const lx_weight* gate_up, const lx_weight* down, lx_math math, float* out,
                                  void* workspace, int T, int L, int I, int E, int top_k, void* stream);
LX_API int64_t lx_moe_grouped_workspace_bytes(int T, int L, int I, int E, int top_k, lx_math math);
/* ---- the calls either side of the experts in a decode layer (replaces engine/cuda/kernels.h:211-233, 253-261,
 * 814-819; the model calls them at engine/model/metis.cpp:2086-2096) and the legacy product forms (:66-70) ------
 *   lx_spec_gemv_f32        y[M, N] = x[M, K] @ w[N, K]^T + bias[N], all f32, M <= 8, a row's bits independent of M
 *   lx_gemm_f32             the same product for any M (engine/cuda/kernels.h:72-76: the routers and the depth head,
 *                           engine/model/metis.cpp:1314-1319,2095); a row's bits are lx_spec_gemv_f32's
 *   lx_router_route         that product on the router's weights w [E, K] into logits [M, E], then lx_moe_route on
 *                           them: every output has the bits of the two calls (it is the two calls, in two launches);
 *                           M <= 8, E <= 1024, K <= 2048, top_k <= 32; `ticket` (one zeroed int32 the fused CUDA
 *                           kernel counts in) must be given and is left untouched
 *   lx_moe_summary          summary[t, :] = sum_k weights[t, k] * expert_emb[ids[t, k], :], expert_emb bf16 [E, R],
 *                           summary f32 [T, R]; _history also history = a * history + b * summary in place
 *   lx_moe_experts_w8       lx_moe_experts on int8 stacks with per-row scales (gate_up_scale [E, 2I], down_scale
 *                           [E, L]), any T and top_k (more than 8 picks take element-wise kernels), workspace of
 *                           lx_moe_workspace_bytes(T, I, top_k)
 *   lx_gemm_bf16            y = alpha * (x @ w^T + bias) + beta * y, x and w bf16, bias bf16 or null, any M */
LX_API int lx_spec_gemv_f32(const float* x, int ld_x, const float* w, const float* bias, float* y, int ld_y, int M, int N,
                            int K, void* stream);
LX_API int lx_gemm_f32(const float* x, int ld_x, const float* w, const float* bias, float* y, int ld_y, int M, int N, int K,
                       void* stream);
LX_API int lx_router_route(const float* x, int ld_x, const float* w, const float* bias, float* logits,
                           const float* selection_bias, int32_t* ids, float* weights, float* entropy, float* confidence,
                           int32_t* ticket, int M, int E, int K, int top_k, void* stream);
LX_API int lx_moe_summary(const int32_t* ids, const float* weights, const void* expert_emb, float* summary, int T, int R,
                          int top_k, void* stream);
LX_API int lx_moe_summary_history(const int32_t* ids, const float* weights, const void* expert_emb, float* summary,
                                  float* history, float a, float b, int T, int R, int top_k, void* stream);
LX_API int lx_moe_experts_w8(const void* latent, const int32_t* ids, const float* weights, const int8_t* gate_up,
                             const float* gate_up_scale, const int8_t* down, const float* down_scale, float* out,
                             void* workspace, int T, int L, int I, int top_k, void* stream);
LX_API int64_t lx_moe_workspace_bytes(int T, int I, int top_k);
LX_API int lx_gemm_bf16(const void* x, int ld_x, const void* w, const void* bias, void* y, lx_dtype y_dtype, int ld_y,
                        int M, int N, int K, float alpha, float beta, void* stream);

/* lx_moe_experts for callers that cannot allocate: code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc. It has no counterpart in the reference (whose lx_moe_experts takes its scratch from the
 * stream's memory pool, as lx_moe_experts here does). Same arguments, same kernels, same bits; the workspace is a
 * fixed 8 MiB array in device memory that each device the library runs on holds until the process ends. A call
 * whose lx_moe_grouped_workspace_bytes(T, L, I, 1024, top_k, LX_MATH_BF16) exceeds 8 MiB answers 1 (and says so on
 * stderr) with nothing launched. Every call on a device shares that device's array: calls that overlap on one
 * device (two streams, two threads) race; calls in stream order do not. The array's address is looked up on the
 * first call on a device (no allocation; make that call outside a capture). */
LX_API int lx_moe_experts_noalloc(const void* latent, const int32_t* ids, const float* weights, const void* gate_up,
                                  const void* down, float* out, int T, int L, int I, int top_k, void* stream);

/* ---- runtime (replaces engine/cuda/kernels.h:308-381 on the HIP runtime) --------------------------- */
typedef struct {
  char name[256];
  int cc_major, cc_minor;
  int sms;
  int64_t l2_bytes;
  int64_t mem_clock_khz;
  int bus_bits;
  int driver_version, runtime_version;
  int64_t l1_bytes, l3_bytes;
  int64_t read_bandwidth;
  char isa[192];
  int native_math;
} lx_device_props;

LX_API int lx_rt_backend(void); /* LX_BACKEND_HIP */
LX_API int lx_rt_device_count(void);
LX_API int lx_rt_set_device(int ordinal);
LX_API int lx_rt_alloc(void** ptr, int64_t bytes); /* zeroed */
LX_API int lx_rt_free(void* ptr);
LX_API int lx_rt_host_alloc(void** ptr, int64_t bytes);
LX_API int lx_rt_host_free(void* ptr);
LX_API int lx_rt_memset(void* ptr, int value, int64_t bytes, void* stream);
LX_API int lx_rt_copy(void* dst, const void* src, int64_t bytes, lx_copy_kind kind, void* stream);
LX_API int lx_rt_stream_create(void** stream);
LX_API int lx_rt_stream_destroy(void* stream);
LX_API int lx_rt_stream_sync(void* stream);
/* No counterpart in the reference. A stream made by lx_rt_stream_create owns 64 MiB of device memory that some products
 * of lx_gemm_w / lx_gemm_skinny (9 .. 64 rows on matrices of few tiles or long rows) keep their partial sums in; no product ever
 * allocates. A host that brings streams of its own (or uses the null stream) calls lx_rt_stream_reserve once per stream
 * (and device) to give it the same, and lx_rt_stream_release before it destroys the stream; without it those products
 * take another kernel with the same results. */
LX_API int lx_rt_stream_reserve(void* stream);
LX_API int lx_rt_stream_release(void* stream);
LX_API int lx_rt_event_create(void** event);
LX_API int lx_rt_event_create_timed(void** event);
LX_API int lx_rt_event_destroy(void* event);
LX_API int lx_rt_event_record(void* event, void* stream);
LX_API int lx_rt_event_sync(void* event);
LX_API int lx_rt_event_elapsed(void* start, void* stop, float* ms);
LX_API int lx_rt_capture_begin(void* stream);
LX_API int lx_rt_capture_end(void* stream, void** graph);
LX_API int lx_rt_graph_launch(void* graph, void* stream);
LX_API int lx_rt_graph_destroy(void* graph);
LX_API int lx_rt_device_sync(void);
LX_API int lx_rt_last_error(void); /* and clears it */
LX_API const char* lx_rt_error_string(int status);
LX_API int lx_rt_is_host_memory(const void* ptr);
LX_API int lx_rt_device_props(int ordinal, lx_device_props* props);
LX_API int lx_rt_mem_info(int64_t* free_bytes, int64_t* total_bytes);
LX_API int lx_bandwidth_probe(int64_t bytes, int reps, double* read_gbps, double* spec_gbps, void* stream);

/* ---- a model folder -> the weights on the device (the C form of the loader interface of engine/core/checkpoint.h:24-101;
 * behaviour: engine/core/checkpoint.cpp). Host code, load time: these calls read files, allocate and synchronise. ---------
 * A folder is safetensors (model.safetensors, or the shards model.safetensors.index.json names). A tensor's dtype names
 * its format: BF16; F8_E4M3 with an F32 weight_scale per row (compressed-tensors FP8); U8 nibble pairs with an e4m3
 * weight_scale per 16 values and an F32 weight_scale_2 per expert (GPTQ NVFP4). With the target equal to the folder's
 * own format every projection is held exactly as the file stores it; otherwise the target's recipe decides per
 * projection, and a projection whose file format differs is converted on the device (bf16 values, copied or
 * dequantised, rounded by lx_quantize_weight; lx_bf16x_encode for LX_W_BF16X) one expert at a time. LX_W_NVFP4 loads
 * only from an NVFP4 folder (round-to-nearest to NVFP4 is refused, as in the reference). The tied head "lm_head" comes
 * from embedding.weight, whose bf16 gather table is a plain tensor. The model's config is not read here: shapes are
 * taken from the file and checked against the formats' layouts, not against a config.
 *   lx_ckpt_projection_format  the recipe: the format `projection` ("layers.4.mixer.qkv", "embedding") is held in under
 *                              `target` (checkpoint.h: projection_format)
 *   lx_ckpt_stored_format      LX_W_BF16 / LX_W_FP8 / LX_W_NVFP4: what the folder holds; -1 and lx_ckpt_error() on failure
 *   lx_ckpt_load               0 and a handle, or 1 with the reason in lx_ckpt_error(); skip_experts leaves the routed
 *                              expert stacks off the device (their shapes, formats and sizes stay readable)
 *   lx_ckpt_projection         the lx_weight of a loaded projection ([N, K] or a stack [E, N, K]); null when absent or skipped
 *   lx_ckpt_expert             expert e of a projection as its own lx_weight (its rows, scales and global)
 *   lx_ckpt_expert_bytes       bytes of one expert's data and scales in the format it is (or would be) held in
 *   lx_ckpt_tensor             a plain tensor (norms, embeddings, routers, biases): device pointer, dtype, shape */
typedef struct lx_ckpt lx_ckpt;
LX_API const char* lx_ckpt_error(void);
LX_API int lx_ckpt_projection_format(lx_wtype target, const char* projection);
LX_API int lx_ckpt_stored_format(const char* dir);
LX_API int lx_ckpt_load(const char* dir, lx_wtype target, int skip_experts, lx_ckpt** out);
LX_API void lx_ckpt_free(lx_ckpt* c);
LX_API const lx_weight* lx_ckpt_projection(const lx_ckpt* c, const char* name);
LX_API int lx_ckpt_count(const lx_ckpt* c);
LX_API const char* lx_ckpt_name(const lx_ckpt* c, int i);
LX_API int lx_ckpt_shape(const lx_ckpt* c, const char* name, int64_t* E, int64_t* N, int64_t* K, int* stack);
LX_API int lx_ckpt_format_of(const lx_ckpt* c, const char* name);
LX_API int lx_ckpt_expert(const lx_ckpt* c, const char* name, int64_t e, lx_weight* out);
LX_API int lx_ckpt_expert_bytes(const lx_ckpt* c, const char* name, int64_t* data, int64_t* scale);
LX_API const void* lx_ckpt_tensor(const lx_ckpt* c, const char* name, lx_dtype* dtype, int* rank, int64_t* shape, int capacity);
LX_API int lx_ckpt_target(const lx_ckpt* c);
LX_API int64_t lx_ckpt_device_bytes(const lx_ckpt* c);
LX_API int64_t lx_ckpt_peak_device_bytes(const lx_ckpt* c);

/* ---- measurement floors (no counterpart in the reference: for benches that state how far a product is from a
 * plain read of the same bytes). Both are asynchronous and capturable.
 *   lx_probe_read   reads `bytes` bytes at `data` (16-byte aligned) once, as the decode GEMV streams a weight: 16-byte
 *                   non-temporal loads, 1 KB contiguous per wavefront instruction, eight in flight per lane, nothing
 *                   computed or written
 *   lx_probe_empty  one empty kernel launch */
LX_API int lx_probe_read(const void* data, int64_t bytes, void* stream);
LX_API int lx_probe_empty(void* stream);

/* ---- architecture and kernel variants (replaces engine/cuda/tunable.h:37-55) -----------------------
 * lx_arch is 95 on gfx950. The GEMV registers its variants under gemv_w_<format>; a variant's name starts
 * with s<S>, its K split, and lx_tune_set admits a variant for a shape only when its split is the
 * shape's own (so the rows' bits never depend on the table). The matrix-core products (lx_gemm_w, lx_gemm_skinny)
 * register theirs under gemm_w_<format>: which kernel family runs ("tiles", "walk1", "walk2", "walk4", "window",
 * "slab", "walkparts", "walksplit"); none changes a sum, so every one is admitted. */
LX_API int lx_arch(void);
LX_API int lx_set_arch_override(int arch);
LX_API int lx_tune_get(const char* kernel, int M, int N, int K);
LX_API int lx_tune_set(const char* kernel, int M, int N, int K, int variant);
LX_API int lx_tune_force(const char* kernel, int M, int N, int K, int variant);
LX_API void lx_tune_clear(void);
LX_API int lx_tune_kernels(const char** names, int capacity);
LX_API int lx_tune_variants(const char* kernel);
LX_API const char* lx_tune_variant_name(const char* kernel, int variant);
/* The autotuner's entry points (engine/cuda/tunable.h:57-75). A problem is one timed case: M rows against an N x K
 * weight in format `weight` and math `math` (0 for both: the kernel's own), `experts` such weights (1 here).
 *   lx_tune_run       runs variant `variant` of a registered kernel on inputs of its own making (seeded, kept per
 *                     problem) and writes the result as f32 [M, N] to `out` (device memory); 801 when the kernel has no
 *                     runner or the variant / problem cannot run (the tuner skips those)
 *   lx_tune_runnable  1 when lx_tune_run can run the kernel's variants (gemv_w_<format>, gemm_w_<format>), else 0
 *   lx_tune_key       the table key of a kernel's problem: the name, then "@w<weight>m<math>" when either is not 0,
 *                     then "@e<experts>" when it is not 1 (engine/cuda/tunable.cu:180-185); writes it NUL-terminated
 *                     into `out` (at most `capacity` bytes) and returns its length */
typedef struct {
  int M, N, K;
  int experts;
  int weight;
  int math;
} lx_tune_problem;
LX_API int lx_tune_run(const char* kernel, int variant, const lx_tune_problem* problem, float* out, void* stream);
LX_API int lx_tune_runnable(const char* kernel);
LX_API int lx_tune_key(const char* kernel, const lx_tune_problem* problem, char* out, int capacity);

#ifdef __cplusplus
}
#endif
#endif /* DROMOS_HIP_H_ */
