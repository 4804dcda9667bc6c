// Decode GEMV for M <= 8 on every weight format: lx_gemv, lx_gemv_w, lx_gemv_decode_bf16
// (contract: engine/cuda/kernels.h:235-246,433-438; CPU behaviour: engine/cpu/gemm.cpp:160-183,339-381).
//
//   y[m, n] = alpha * (rowfactor[n] * sum_k x[m, k] * w[n, k] + bias[n]) + beta * y[m, n]
//
// One pass over the weights at HBM speed is the whole cost, so the kernel is built around the stream
// (stream_dot.h): a persistent grid of at most two workgroups per compute unit, four wavefronts each, every
// wavefront streaming R whole rows at a time with U 128-bit loads per row in flight; x staged once per
// workgroup in LDS as f32. When N is too small to give every compute unit rows, S wavefronts of a
// workgroup share a row's steps (interleaved) and their partial sums are added in wavefront order through
// LDS. S depends on (format, N, K) only, never on M, so a row's bits are the same for every M.
#include "common.h"
#include "stream_dot.h"

namespace dro {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;
constexpr int kLdsFloats = 32 * 1024;  // 128 KB of x at most: one workgroup per compute unit then

struct GemvArgs {
  const void* x;
  int x_dtype;
  int64_t ld_x;
  const uint8_t* w;
  const uint8_t* scale;  // f32 [N] (INT8 / FP8) or e4m3 [N, K / 16] (NVFP4)
  float global;
  const void* bias;
  int bias_dtype;
  void* y;
  int y_dtype;
  int64_t ld_y;
  int M, N;
  int64_t K;
  float alpha, beta;
  int split;  // S: wavefronts sharing a row
};

// The epilogue's operation order (engine/cpu/gemm.cpp:21-34).
__device__ __forceinline__ void write_out(const GemvArgs& a, int wtype, int m, int64_t n, float sum) {
  float t = row_factor(wtype, a.scale, a.global, n) * sum;
  if (a.bias) t += load_as_f32(a.bias, a.bias_dtype, n);
  float v = a.alpha * t;
  const int64_t at = m * a.ld_y + n;
  if (a.beta != 0.0f) v = a.beta * load_as_f32(a.y, a.y_dtype, at) + v;
  store_from_f32(a.y, a.y_dtype, at, v);
}

// Row sets are handed to workgroups round-robin; a set is kWaves / S groups of R rows.
template <int F, int MT, int R, int U>
__global__ void __launch_bounds__(kThreads) gemv_stream_kernel(const GemvArgs a) {
  extern __shared__ __align__(16) float lds[];
  const int steps = steps_for<F>(a.K);
  const int per_row = x_row_floats<F>(steps);
  float* xs = lds;
  float* partial = lds + MT * per_row;  // [kWaves][MT * R] when S > 1
  stage_x<F, MT>(xs, a.x, a.x_dtype, a.ld_x, nullptr, a.M, a.K, steps);
  __syncthreads();

  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int S = a.split;
  const int groups_per_set = kWaves / S;
  const int part = wave % S;  // which share of the steps
  const int group_in_set = wave / S;
  const int64_t rb = row_bytes<F>(a.K);
  const int chunks = static_cast<int>(rb / 16);
  const int64_t n_groups = (a.N + R - 1) / R;
  const int64_t n_sets = (n_groups + groups_per_set - 1) / groups_per_set;
  const int64_t scale_row = F == LX_W_NVFP4 ? a.K / 16 : 0;

  for (int64_t set = blockIdx.x; set < n_sets; set += gridDim.x) {
    const int64_t group = set * groups_per_set + group_in_set;
    const int64_t n0 = group * R;
    const uint8_t* rows[R];
    const uint8_t* scales[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      int64_t n = n0 + r;
      if (n > a.N - 1) n = a.N - 1;  // past the end: stream a valid row, write nothing
      rows[r] = a.w + n * rb;
      scales[r] = a.scale + n * scale_row;
    }
    float acc[MT][R];
    {
      // Part p of S takes the contiguous steps [p * per, (p + 1) * per).
      const int per = (steps + S - 1) / S;
      const int s_begin = min(steps, part * per), s_end = min(steps, s_begin + per);
      stream_rows<F, MT, R, U>(rows, scales, chunks, s_begin, s_end, xs, per_row, acc);
    }
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int r = 0; r < R; ++r) acc[m][r] = wave_sum(acc[m][r]);
    if (S > 1) {
      if (lane == 0) {
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
          for (int r = 0; r < R; ++r) partial[wave * (MT * R) + m * R + r] = acc[m][r];
      }
      __syncthreads();
      if (part == 0) {
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
          for (int r = 0; r < R; ++r) {
            float s = acc[m][r];
            for (int p = 1; p < S; ++p) s += partial[(wave + p) * (MT * R) + m * R + r];
            acc[m][r] = s;
          }
      }
      __syncthreads();
    }
    if (lane == 0 && part == 0) {
#pragma unroll
      for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int r = 0; r < R; ++r)
          if (m < a.M && n0 + r < a.N) write_out(a, F, m, n0 + r, acc[m][r]);
    }
  }
}

// Any K, any alignment, x read where it lies: one wavefront per output row, lanes striding over k, the
// lane sums combined by the same tree. Rows whose bytes cannot be read 16 at a time take this kernel
// (the choice depends on K and the weight's address only, never on M).
__global__ void __launch_bounds__(kThreads) gemv_plain_kernel(const GemvArgs a, int wtype) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t n = static_cast<int64_t>(blockIdx.x) * kWaves + threadIdx.x / kWave;
  if (n >= a.N) return;
  float acc[8];
#pragma unroll
  for (int m = 0; m < 8; ++m) acc[m] = 0.0f;
  for (int64_t k = lane; k < a.K; k += kWave) {
    const float w = weight_element(wtype, a.w, a.scale, n, k, a.K);
#pragma unroll
    for (int m = 0; m < 8; ++m)
      if (m < a.M) acc[m] = __builtin_fmaf(load_as_f32(a.x, a.x_dtype, m * a.ld_x + k), w, acc[m]);
  }
#pragma unroll
  for (int m = 0; m < 8; ++m) {
    const float s = wave_sum(acc[m]);
    if (lane == 0 && m < a.M) write_out(a, wtype, m, n, s);
  }
}

// The K split of a shape: its order class. A function of (format, N, K) only.
template <int F>
int order_class(int N, int64_t K, int R) {
  const int steps = steps_for<F>(K);
  const int cus = compute_units();
  int S = 1;
  // Fewer row groups than wavefront slots the device wants busy: let wavefronts share rows.
  while (S < kWaves && (static_cast<int64_t>(N) + R - 1) / R * S < 2LL * cus && steps >= 2 * S) S *= 2;
  return S;
}

template <int F>
constexpr int rows_per_wave() {
  return 2;
}
template <int F>
constexpr int loads_in_flight() {
  return F == LX_W_NVFP4 ? 2 : 4;
}

template <int F, int MT>
int launch_stream(const GemvArgs& a, hipStream_t stream) {
  constexpr int R = rows_per_wave<F>(), U = loads_in_flight<F>();
  const int steps = steps_for<F>(a.K);
  const size_t lds = sizeof(float) * (static_cast<size_t>(MT) * x_row_floats<F>(steps) + kWaves * MT * R);
  const int groups_per_set = kWaves / a.split;
  const int64_t n_groups = (a.N + R - 1) / R;
  const int64_t n_sets = (n_groups + groups_per_set - 1) / groups_per_set;
  const int per_cu = lds <= 64 * 1024 ? 2 : 1;
  const int64_t cap = static_cast<int64_t>(compute_units()) * per_cu;
  const unsigned grid = static_cast<unsigned>(n_sets < cap ? n_sets : cap);
  auto kernel = gemv_stream_kernel<F, MT, R, U>;
  if (lds > 48 * 1024) {
    static thread_local bool raised = false;
    if (!raised) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                              160 * 1024 - 256) != hipSuccess)
        (void)hipGetLastError();
      raised = true;
    }
  }
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(kThreads), lds, stream, a);
  return status_of(hipGetLastError());
}

template <int F>
int launch_format(GemvArgs& a, const char* kernel_name, hipStream_t stream) {
  constexpr int R = rows_per_wave<F>();
  const int64_t rb = row_bytes<F>(a.K);
  const int steps = steps_for<F>(a.K);
  const bool vector_rows = rb % 16 == 0 && reinterpret_cast<uintptr_t>(a.w) % 16 == 0 &&
                           (F != LX_W_NVFP4 || reinterpret_cast<uintptr_t>(a.scale) % 2 == 0);
  // Activation rows a pass can hold in LDS: a function of K only. More rows than that run as several
  // passes over the weights; each row's arithmetic is the same in any pass, so its bits do not change.
  int fit = 8;
  while (fit >= 1 && static_cast<int64_t>(fit) * x_row_floats<F>(steps) + kWaves * fit * R > kLdsFloats) fit /= 2;
  if (!vector_rows || fit < 1) {
    const unsigned grid = static_cast<unsigned>((a.N + kWaves - 1) / kWaves);
    hipLaunchKernelGGL(gemv_plain_kernel, dim3(grid), dim3(kThreads), 0, stream, a, F);
    return status_of(hipGetLastError());
  }
  a.split = order_class<F>(a.N, a.K, R);
  const int tuned = tuned_variant(kernel_name, a.M, a.N, static_cast<int>(a.K));
  if (tuned >= 0 && tuned <= 2) a.split = 1 << tuned;
  const int M = a.M;
  const char* x0 = static_cast<const char*>(a.x);
  char* y0 = static_cast<char*>(a.y);
  const int64_t x_row = a.ld_x * (a.x_dtype == LX_BF16 ? 2 : 4), y_row = a.ld_y * (a.y_dtype == LX_BF16 ? 2 : 4);
  for (int m0 = 0; m0 < M; m0 += fit) {
    a.M = M - m0 < fit ? M - m0 : fit;
    a.x = x0 + m0 * x_row;
    a.y = y0 + m0 * y_row;
    const int mt = a.M <= 1 ? 1 : a.M <= 2 ? 2 : a.M <= 4 ? 4 : 8;
    int st;
    switch (mt) {
      case 1: st = launch_stream<F, 1>(a, stream); break;
      case 2: st = launch_stream<F, 2>(a, stream); break;
      case 4: st = launch_stream<F, 4>(a, stream); break;
      default: st = launch_stream<F, 8>(a, stream); break;
    }
    if (st) return st;
  }
  return kOk;
}

bool valid_dtype(int d) { return d == LX_F32 || d == LX_BF16; }

}  // namespace

// Whether variant `v` (split 1 << v) is the order class of (format, N, K): the tuner's admission rule.
bool gemv_admits(int wtype, int variant, int N, int K) {
  int S = 1;
  switch (wtype) {
    case LX_W_BF16: S = order_class<LX_W_BF16>(N, K, rows_per_wave<LX_W_BF16>()); break;
    case LX_W_INT8: S = order_class<LX_W_INT8>(N, K, rows_per_wave<LX_W_INT8>()); break;
    case LX_W_FP8: S = order_class<LX_W_FP8>(N, K, rows_per_wave<LX_W_FP8>()); break;
    default: S = order_class<LX_W_NVFP4>(N, K, rows_per_wave<LX_W_NVFP4>()); break;
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
  if (w.type == LX_W_BF16X) return fail(kNotSupported);
  if (w.type != LX_W_BF16 && w.type != LX_W_INT8 && w.type != LX_W_FP8 && w.type != LX_W_NVFP4) return fail(kInvalid);
  if (w.type != LX_W_BF16 && !w.scale) return fail(kInvalid);
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
    case LX_W_BF16: return launch_format<LX_W_BF16>(a, "gemv_w_bf16", s);
    case LX_W_INT8: return launch_format<LX_W_INT8>(a, "gemv_w_int8", s);
    case LX_W_FP8: return launch_format<LX_W_FP8>(a, "gemv_w_fp8", s);
    default: return launch_format<LX_W_NVFP4>(a, "gemv_w_nvfp4", s);
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

int lx_gemv_decode_bf16(const void* x, lx_dtype x_dtype, int ld_x, const void* w, const void* bias, lx_dtype bias_dtype,
                        void* y, lx_dtype y_dtype, int ld_y, int M, int N, int K, float alpha, float beta, void* stream) {
  const lx_weight wt{LX_W_BF16, w, nullptr, 1.0f, nullptr};
  return gemv_any(x, x_dtype, ld_x, wt, bias, bias_dtype, y, y_dtype, ld_y, M, N, K, alpha, beta, stream);
}

}  // extern "C"
