// Decode GEMV for M <= 8 on every weight format: lx_gemv, lx_gemv_w, lx_gemv_decode_bf16
// (contract: engine/cuda/kernels.h:235-246,433-438; CPU behaviour: engine/cpu/gemm.cpp:160-183,339-381).
//
//   y[m, n] = alpha * (rowfactor[n] * sum_k x[m, k] * w[n, k] + bias[n]) + beta * y[m, n]
//
// One pass over the weights at HBM speed is the whole cost, so the kernels (gemv_kernels.h, one source per format)
// are built around the stream (stream_dot.h): many short workgroups, every wavefront asking for its whole share of
// R rows before anything else; x staged once per workgroup in LDS. When N is too small to give every compute unit
// rows, S wavefronts of a workgroup share a row's steps and their partial sums are added in wavefront order
// through LDS. S depends on (format, N, K) only, never on M, so a row's bits are the same for every M.
#include "gemv_kernels.h"

namespace dro {

// Whether variant `v` (split 1 << v) is the order class of (format, N, K): the tuner's admission rule.
bool gemv_admits(int wtype, int variant, int N, int K) {
  int S = 1;
  switch (wtype) {
    case LX_W_BF16:
    case LX_W_BF16X: S = order_class<LX_W_BF16>(N, K, 2); break;
    case LX_W_INT8: S = order_class<LX_W_INT8>(N, K, 2); break;
    case LX_W_FP8: S = order_class<LX_W_FP8>(N, K, 2); break;
    default: S = order_class<LX_W_NVFP4>(N, K, 2); break;
  }
  return (1 << variant) == S;
}

// The GEMV of every format behind the three entry points. Validation follows engine/cpu/gemm.cpp:160-168.
int gemv_any(const void* x, int x_dtype, int ld_x, const lx_weight& w, const void* bias, int bias_dtype, void* y,
             int y_dtype, int ld_y, int M, int N, int K, float alpha, float beta, void* stream) {
  if (M == 0 || N == 0) return kOk;
  if (M < 0 || M > 8 || N < 0 || K <= 0 || ld_x < K || ld_y < N) return fail(kInvalid);
  if (!valid_dtype(x_dtype) || !valid_dtype(y_dtype) || !valid_dtype(bias_dtype)) return fail(kInvalid);
  if (!x || !y || !w.data) return fail(kInvalid);
  if (w.type == LX_W_BF16X) {
    if (K >= bf16x::kMaxK) return fail(kInvalid);
  } else {
    if (w.type != LX_W_BF16 && w.type != LX_W_INT8 && w.type != LX_W_FP8 && w.type != LX_W_NVFP4) return fail(kInvalid);
    if (w.type != LX_W_BF16 && !w.scale) return fail(kInvalid);
  }
  if (w.type == LX_W_NVFP4 && K % 16 != 0) return fail(kInvalid);
  GemvArgs a{};
  a.x = x;
  a.x_dtype = x_dtype;
  a.ld_x = ld_x;
  a.w = static_cast<const uint8_t*>(w.data);
  a.scale = static_cast<const uint8_t*>(w.scale);
  a.global = w.type == LX_W_NVFP4 ? w.global : 1.0f;
  a.bias = bias;
  a.bias_dtype = bias_dtype;
  a.y = y;
  a.y_dtype = y_dtype;
  a.ld_y = ld_y;
  a.M = M;
  a.N = N;
  a.K = K;
  a.alpha = alpha;
  a.beta = beta;
  a.split = 1;
  hipStream_t s = as_stream(stream);
  switch (w.type) {
    case LX_W_BF16: return gemv_launch_bf16(a, s);
    case LX_W_INT8: return gemv_launch_int8(a, s);
    case LX_W_FP8: return gemv_launch_fp8(a, s);
    case LX_W_BF16X: return gemv_launch_bf16x(a, s);
    default: return gemv_launch_nvfp4(a, s);
  }
}

}  // namespace dro

using namespace dro;

extern "C" {

// engine/cpu/gemm.cpp:339-348
int lx_gemv(const void* x, lx_dtype x_dtype, int ld_x, const void* w, lx_wtype w_type, const float* w_scale, const void* bias,
            lx_dtype bias_dtype, void* y, lx_dtype y_dtype, int ld_y, int M, int N, int K, float alpha, float beta,
            void* stream) {
  if (w_type != LX_W_BF16 && w_type != LX_W_INT8) return fail(kInvalid);
  if (w_type == LX_W_INT8 && !w_scale && M > 0 && N > 0) return fail(kInvalid);
  const lx_weight wt{w_type, w, w_scale, 1.0f, nullptr};
  return gemv_any(x, x_dtype, ld_x, wt, bias, bias_dtype, y, y_dtype, ld_y, M, N, K, alpha, beta, stream);
}

// engine/cpu/gemm.cpp:364-371: the bf16 product on the encoded rows; the kernel decodes a lane's eight values to the
// bf16 bits the bf16 kernel loads, in the same lanes and steps, so y is lx_gemv's on the original weights to the bit.
int lx_gemv_bf16x(const void* x, lx_dtype x_dtype, int ld_x, const void* w, const void* bias, lx_dtype bias_dtype, void* y,
                  lx_dtype y_dtype, int ld_y, int M, int N, int K, float alpha, float beta, void* stream) {
  if (M != 0 && N != 0 && (reinterpret_cast<uintptr_t>(w) & 7) != 0) return fail(kInvalid);
  const lx_weight wt{LX_W_BF16X, w, nullptr, 1.0f, nullptr};
  return gemv_any(x, x_dtype, ld_x, wt, bias, bias_dtype, y, y_dtype, ld_y, M, N, K, alpha, beta, stream);
}

int lx_gemv_decode_bf16(const void* x, lx_dtype x_dtype, int ld_x, const void* w, const void* bias, lx_dtype bias_dtype,
                        void* y, lx_dtype y_dtype, int ld_y, int M, int N, int K, float alpha, float beta, void* stream) {
  const lx_weight wt{LX_W_BF16, w, nullptr, 1.0f, nullptr};
  return gemv_any(x, x_dtype, ld_x, wt, bias, bias_dtype, y, y_dtype, ld_y, M, N, K, alpha, beta, stream);
}

}  // extern "C"
