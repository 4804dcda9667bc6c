// Batched decode products on the matrix cores: lx_gemm_w, lx_gemm_skinny, and lx_gemv_w's entry (which
// routes to the streaming GEMV, or to the skinny kernel in batch-invariant mode).
#include "common.h"

namespace dro {
int gemv_any(const void* x, int x_dtype, int ld_x, const lx_weight& w, const void* bias, int bias_dtype, void* y,
             int y_dtype, int ld_y, int M, int N, int K, float alpha, float beta, void* stream);
}

using namespace dro;

extern "C" {

int lx_gemv_w(const void* x, lx_dtype x_dtype, int ld_x, const lx_weight* w, const void* bias, lx_dtype bias_dtype, void* y,
              lx_dtype y_dtype, int ld_y, int M, int N, int K, float alpha, float beta, void* stream) {
  if (!w) return fail(kInvalid);
  return gemv_any(x, x_dtype, ld_x, *w, bias, bias_dtype, y, y_dtype, ld_y, M, N, K, alpha, beta, stream);
}

int64_t lx_gemm_workspace_bytes(int M, int K, lx_math math) {
  if (M <= 0 || K <= 0) return 0;
  const int64_t elem = math == LX_MATH_INT8 ? 1 : 4;
  const int64_t bytes = (static_cast<int64_t>(M) * 4 + 63) / 64 * 64 + static_cast<int64_t>(M) * K * elem;
  return (bytes + 255) / 256 * 256;
}

}  // extern "C"

// TEMPORARY until the matrix-core kernels land.
extern "C" {
int lx_gemm_w(const void*, lx_dtype, int, const lx_weight*, lx_math, const void*, lx_dtype, void*, lx_dtype, int, int, int, int,
              float, float, void*, void*) {
  return fail(kNotSupported);
}
int lx_gemm_skinny(const void*, lx_dtype, int, const lx_weight*, const void*, lx_dtype, void*, lx_dtype, int, int, int, int,
                   float, float, void*) {
  return fail(kNotSupported);
}
int lx_moe_experts(const void*, const int32_t*, const float*, const void*, const void*, float*, int, int, int, int, void*) {
  return fail(kNotSupported);
}
int lx_moe_experts_grouped(const void*, const int32_t*, const float*, const lx_weight*, const lx_weight*, lx_math, float*, void*,
                           int, int, int, int, int, void*) {
  return fail(kNotSupported);
}
int64_t lx_moe_grouped_workspace_bytes(int, int, int, int, int, lx_math) { return 0; }
}
