// The calls either side of the routed experts in a decode layer, and the legacy forms of the products:
// lx_spec_gemv_f32, lx_gemm_f32, lx_router_route, lx_moe_summary, lx_moe_summary_history, lx_moe_experts_w8, lx_gemm_bf16
// (contracts: engine/cuda/kernels.h:66-76,211-233,253-261,814-819; CPU behaviour: engine/cpu/gemm.cpp:304-337,
// engine/cpu/spec.cpp:21-28, engine/cpu/moe.cpp:399-442,460-476,512-517).
#include "common.h"
#include "moe_common.h"

namespace dro {

int gemm_bf16_math(const void* x, int x_dtype, int64_t ld_x, const lx_weight& w, const void* bias, int bias_dtype, void* y,
                   int y_dtype, int64_t ld_y, int M, int N, int K, float alpha, float beta, void* stream);

namespace {

constexpr int kThreads = 256;
constexpr int kSpecRows = 8;  // engine/cpu/spec.cpp:12

// y[m, n] = sum_k x[m, k] * w[n, k] + bias[n] on f32 weights: one wavefront per output column n and block of eight rows
// (blockIdx.y; the last block may hold fewer), a lane taking four consecutive k of every 256 (a 16-byte load where the
// rows allow it), f32 FMAs in ascending k, the lane sums combined by one fixed tree. Nothing in a row's sums depends on
// the other rows.
template <bool VEC>
__global__ void __launch_bounds__(kThreads) spec_gemv_f32_kernel(const float* __restrict__ x, int64_t ld_x, const float* __restrict__ w,
                                                                 const float* __restrict__ bias, float* __restrict__ y, int64_t ld_y,
                                                                 int rows, int N, int K) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t n = static_cast<int64_t>(blockIdx.x) * (kThreads / kWave) + threadIdx.x / kWave;
  if (n >= N) return;
  const int m0 = blockIdx.y * kSpecRows, M = min(kSpecRows, rows - m0);
  x += m0 * ld_x;
  y += m0 * ld_y;
  const float* wrow = w + n * K;
  float acc[kSpecRows];
#pragma unroll
  for (int m = 0; m < kSpecRows; ++m) acc[m] = 0.0f;
  if constexpr (VEC) {
    for (int k = lane * 4; k < K; k += kWave * 4) {
      const f32x4 wv = *reinterpret_cast<const f32x4*>(wrow + k);
#pragma unroll
      for (int m = 0; m < kSpecRows; ++m) {
        if (m < M) {
          const f32x4 xv = *reinterpret_cast<const f32x4*>(x + m * ld_x + k);
          acc[m] = __builtin_fmaf(xv.x, wv.x, acc[m]);
          acc[m] = __builtin_fmaf(xv.y, wv.y, acc[m]);
          acc[m] = __builtin_fmaf(xv.z, wv.z, acc[m]);
          acc[m] = __builtin_fmaf(xv.w, wv.w, acc[m]);
        }
      }
    }
  } else {
    // The same assignment of k to lanes and the same order, element by element.
    for (int k0 = lane * 4; k0 < K; k0 += kWave * 4) {
      for (int k = k0; k < min(k0 + 4, K); ++k) {
        const float wv = wrow[k];
#pragma unroll
        for (int m = 0; m < kSpecRows; ++m)
          if (m < M) acc[m] = __builtin_fmaf(x[m * ld_x + k], wv, acc[m]);
      }
    }
  }
#pragma unroll
  for (int m = 0; m < kSpecRows; ++m) {
    const float s = wave_sum(acc[m]);
    if (lane == 0 && m < M) y[m * ld_y + n] = bias ? s + bias[n] : s;
  }
}

int spec_gemv(const float* x, int ld_x, const float* w, const float* bias, float* y, int ld_y, int M, int N, int K, hipStream_t s) {
  const bool vec = K % 4 == 0 && ld_x % 4 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0;
  const dim3 grid((N + kThreads / kWave - 1) / (kThreads / kWave), (M + kSpecRows - 1) / kSpecRows);
  if (vec) hipLaunchKernelGGL(spec_gemv_f32_kernel<true>, grid, dim3(kThreads), 0, s, x, ld_x, w, bias, y, ld_y, M, N, K);
  else hipLaunchKernelGGL(spec_gemv_f32_kernel<false>, grid, dim3(kThreads), 0, s, x, ld_x, w, bias, y, ld_y, M, N, K);
  return status_of(hipGetLastError());
}

// summary[t, r] = sum_k weights[t, k] * emb[ids[t, k], r], from zero, a separate multiply and add per slot in slot
// order (engine/cpu/moe.cpp:405-416); with HISTORY also history = a * history + b * summary (:436-437).
template <bool HISTORY>
__global__ void __launch_bounds__(kThreads) summary_kernel(const int32_t* __restrict__ ids, const float* __restrict__ weights,
                                                           const uint16_t* __restrict__ emb, float* __restrict__ summary,
                                                           float* __restrict__ history, float a, float b, int64_t n, int R, int top_k) {
  const int64_t at = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (at >= n) return;
  const int64_t t = at / R;
  const int r = static_cast<int>(at - t * R);
  float s = 0.0f;
  for (int k = 0; k < top_k; ++k) {
    const float p = weights[t * top_k + k] * bf16_bits_to_f32(emb[static_cast<int64_t>(ids[t * top_k + k]) * R + r]);
    s = s + p;
  }
  summary[at] = s;
  if constexpr (HISTORY) {
    const float u = a * history[at], v = b * s;
    history[at] = u + v;
  }
}

int64_t round256(int64_t b) { return (b + 255) / 256 * 256; }

}  // namespace
}  // namespace dro

using namespace dro;

extern "C" {

int64_t lx_moe_decode_workspace_bytes(int T, int I, int top_k);

// engine/cuda/kernels.h:72-76, engine/cpu/gemm.cpp:316-337: the same product for any number of rows (the routers and
// the depth head at more than eight rows); a row's bits are those of lx_spec_gemv_f32.
int lx_gemm_f32(const float* x, int ld_x, const float* w, const float* bias, float* y, int ld_y, int M, int N, int K, void* stream) {
  if (M < 0 || N < 0 || K <= 0 || ld_x < K || ld_y < N) return fail(kInvalid);
  if (M == 0 || N == 0) return kOk;
  if (!x || !w || !y) return fail(kInvalid);
  if (M > 65535 * kSpecRows) return fail(kInvalid);
  return spec_gemv(x, ld_x, w, bias, y, ld_y, M, N, K, as_stream(stream));
}

int lx_spec_gemv_f32(const float* x, int ld_x, const float* w, const float* bias, float* y, int ld_y, int M, int N, int K,
                     void* stream) {
  if (M == 0 || N == 0) return kOk;
  if (M < 0 || M > kSpecRows || N < 0 || K <= 0 || ld_x < K || ld_y < N || !x || !w || !y) return fail(kInvalid);
  return spec_gemv(x, ld_x, w, bias, y, ld_y, M, N, K, as_stream(stream));
}

// Two launches (the product, then the routing of its logits): every output has the bits of the two calls because it
// is the two calls. The ticket word is the fused CUDA kernel's; it is neither read nor written here and stays zero.
int lx_router_route(const float* x, int ld_x, const float* w, const float* bias, float* logits, const float* selection_bias,
                    int32_t* ids, float* weights, float* entropy, float* confidence, int32_t* ticket, int M, int E, int K, int top_k,
                    void* stream) {
  if (M <= 0) return kOk;
  if (M > kSpecRows || E <= 0 || E > 1024 || K <= 0 || K > 2048 || ld_x < K || top_k < 1 || top_k > 32 || top_k > E || !x || !w ||
      !logits || !ids || !weights || !entropy || !confidence || !ticket)
    return fail(kInvalid);
  hipStream_t s = as_stream(stream);
  if (int st = spec_gemv(x, ld_x, w, bias, logits, E, M, E, K, s)) return st;
  return route(logits, selection_bias, ids, weights, entropy, confidence, M, E, top_k, s);
}

int lx_moe_summary(const int32_t* ids, const float* weights, const void* expert_emb, float* summary, int T, int R, int top_k,
                   void* stream) {
  if (T <= 0 || R <= 0) return kOk;
  if (!ids || !weights || !expert_emb || !summary || top_k < 1) return fail(kInvalid);
  const int64_t n = static_cast<int64_t>(T) * R;
  hipLaunchKernelGGL(summary_kernel<false>, dim3(static_cast<unsigned>((n + kThreads - 1) / kThreads)), dim3(kThreads), 0,
                     as_stream(stream), ids, weights, static_cast<const uint16_t*>(expert_emb), summary, static_cast<float*>(nullptr), 0.0f,
                     0.0f, n, R, top_k);
  return status_of(hipGetLastError());
}

int lx_moe_summary_history(const int32_t* ids, const float* weights, const void* expert_emb, float* summary, float* history, float a,
                           float b, int T, int R, int top_k, void* stream) {
  if (T <= 0 || R <= 0) return kOk;
  if (!ids || !weights || !expert_emb || !summary || !history || top_k < 1) return fail(kInvalid);
  const int64_t n = static_cast<int64_t>(T) * R;
  hipLaunchKernelGGL(summary_kernel<true>, dim3(static_cast<unsigned>((n + kThreads - 1) / kThreads)), dim3(kThreads), 0,
                     as_stream(stream), ids, weights, static_cast<const uint16_t*>(expert_emb), summary, history, a, b, n, R, top_k);
  return status_of(hipGetLastError());
}

// The int8 experts of the legacy entry (weight-only, any T): the decode experts' kernels, eight tokens at a time (a
// token's bits do not depend on the tokens beside it). The workspace holds the intermediate rows of one such
// step.
int lx_moe_experts_w8(const void* latent, const int32_t* ids, const float* weights, const int8_t* gate_up, const float* gate_up_scale,
                      const int8_t* down, const float* down_scale, float* out, void* workspace, int T, int L, int I, int top_k,
                      void* stream) {
  if (T <= 0) return kOk;
  if (!latent || !ids || !weights || !out || L <= 0 || I <= 0 || top_k < 1) return fail(kInvalid);
  if (!gate_up || !gate_up_scale || !down || !down_scale || !workspace) return fail(kInvalid);
  const lx_weight gu{LX_W_INT8, gate_up, gate_up_scale, 1.0f, nullptr}, dn{LX_W_INT8, down, down_scale, 1.0f, nullptr};
  hipStream_t s = as_stream(stream);
  if (top_k > 8) {
    // More picks than the decode kernels take, and no expert count to group pairs by: the element-wise experts, every
    // pair on its own, the intermediate rows [T * top_k, I] in the workspace (the reference takes any top_k here,
    // engine/cpu/moe.cpp:460-476).
    DecodeArgs d{};
    d.latent = static_cast<const uint16_t*>(latent);
    d.ids = ids;
    d.weights = weights;
    d.gu = as_stack(gu);
    d.dn = as_stack(dn);
    d.inter = static_cast<uint16_t*>(workspace);
    d.out = out;
    d.T = T, d.L = L, d.I = I, d.top_k = top_k;
    return experts_plain(d, LX_W_INT8, LX_W_INT8, s);
  }
  for (int t0 = 0; t0 < T; t0 += 8) {
    const int n = T - t0 < 8 ? T - t0 : 8;
    const int st = experts_decode(static_cast<const uint16_t*>(latent) + static_cast<int64_t>(t0) * L, ids + static_cast<int64_t>(t0) * top_k,
                                  weights + static_cast<int64_t>(t0) * top_k, gu, dn, out + static_cast<int64_t>(t0) * L, workspace, n, L, I,
                                  top_k, s);
    if (st) return st;
  }
  return kOk;
}

// At least the reference's size (engine/cpu/moe.cpp:512-517), and room for one eight-token step of the decode experts.
int64_t lx_moe_workspace_bytes(int T, int I, int top_k) {
  if (T <= 0 || I <= 0 || top_k <= 0) return 0;
  const int64_t pairs = static_cast<int64_t>(T) * top_k;
  const int64_t theirs = round256((2 * pairs * I + 15) / 16 * 16 + 8 * pairs);
  const int64_t ours = lx_moe_decode_workspace_bytes(T < 8 ? T : 8, I, top_k);
  return theirs > ours ? theirs : ours;
}

// engine/cpu/gemm.cpp:304-314: bf16 x and weights, f32 sums on the matrix cores, bias bf16 or null, any M.
int lx_gemm_bf16(const void* x, int ld_x, const void* w, const void* bias, void* y, lx_dtype y_dtype, int ld_y, int M, int N, int K,
                 float alpha, float beta, void* stream) {
  if (y_dtype != LX_F32 && y_dtype != LX_BF16) return fail(kInvalid);
  if (M < 0 || N < 0 || K <= 0 || ld_x < K || ld_y < N) return fail(kInvalid);
  if (M == 0 || N == 0) return kOk;
  if (!x || !w || !y) return fail(kInvalid);
  const lx_weight wt{LX_W_BF16, w, nullptr, 1.0f, nullptr};
  return gemm_bf16_math(x, LX_BF16, ld_x, wt, bias, LX_BF16, y, y_dtype, ld_y, M, N, K, alpha, beta, stream);
}

}  // extern "C"
