// The decode GEMV kernels and their launchers (templates on the weight format). Included by gemv.hip, which holds
// the entry points, and by one small source per format, so the formats compile side by side.
#pragma once

#include <stdlib.h>

#include "common.h"
#include "stream_dot.h"

namespace dro {

constexpr int kThreads = 256;  // the plain kernel's workgroup
constexpr int kMaxThreads = 512;  // the streaming kernel's workgroup is chosen per launch, up to this
constexpr int kMaxWaves = kMaxThreads / kWave;
constexpr int kLdsFloats = 38 * 1024;  // 152 KB of x at most: one workgroup per compute unit then

struct GemvArgs {
  const void* x;
  int x_dtype;
  int64_t ld_x;
  const uint8_t* w;
  const uint8_t* scale;  // f32 [N] (INT8 / FP8) or e4m3 [N, K / 16] (NVFP4); BF16X streamed: the first row's span tops
  float global;
  const void* bias;
  int bias_dtype;
  void* y;
  int y_dtype;
  int64_t ld_y;
  int M, N;
  int64_t K;
  float alpha, beta;
  int split;  // S: wavefronts sharing a row (1, 2 or 4)
  // Launch geometry, computed once on the host so a wavefront's first load is a few instructions away.
  int split_log2;
  int steps;           // wave steps covering K
  int steps_per_part;  // ceil(steps / S)
  int chunks;          // 16-byte chunks in a row (BF16X: groups of eight values)
  int64_t row_bytes;
  int64_t scale_row_bytes;  // NVFP4: bytes of block scales per row; BF16X: a whole record
  int phase_steps;  // > 0: the activation image holds this many steps at a time (two images in turn), else all
  int rounds;       // ROLL kernels: the consecutive row groups a workgroup takes (at least one per wavefront)
};

namespace {

// The epilogue's operation order (engine/cpu/gemm.cpp:21-34); rf is the row factor, b the bias (unused without one).
__device__ __forceinline__ void write_out(const GemvArgs& a, int m, int64_t n, float sum, float rf, float b) {
  float t = rf * sum;
  if (a.bias) t += b;
  float v = a.alpha * t;
  const int64_t at = m * a.ld_y + n;
  if (a.beta != 0.0f) v = a.beta * load_as_f32(a.y, a.y_dtype, at) + v;
  store_from_f32(a.y, a.y_dtype, at, v);
}

__device__ __forceinline__ void write_out(const GemvArgs& a, int wtype, int m, int64_t n, float sum) {
  write_out(a, m, n, sum, row_factor(wtype, a.scale, a.global, n), a.bias ? load_as_f32(a.bias, a.bias_dtype, n) : 0.0f);
}

// One workgroup takes blockDim / 64 / S groups of R rows, one group per wavefront (S wavefronts share a
// group's steps when S > 1), and every wavefront asks for its whole share of the weights (up to two batches of
// U steps) before anything else: many short-lived wavefronts, each with all its loads in flight, keep the
// memory system busier than a few long-lived ones.
// XB: the activations are bf16 and go into the packed image (two products per instruction); otherwise the f32 image.
// ONE: a wavefront's share of a row's steps fits one batch of U (the usual case at decode sizes).
// ROLL (several bf16 activation rows, one-batch rows, no K split): the products of several rows cost about as many
// vector instructions as the weights take to arrive, and with a workgroup per set of rows the device holds only part of
// the workgroups at a time: all ask, all wait, all multiply, and only then do the others ask. Here the grid is what the
// device holds at once and a wavefront streams `rounds` groups through its one batch of registers (run_rolling), so the
// memory and the vector units work at the same time; the image is staged once per workgroup.
template <int F, int MT, int R, int U, bool XB, bool ONE, bool ROLL = false>
__global__ void __launch_bounds__(kMaxThreads) gemv_stream_kernel(const GemvArgs a) {
  static_assert(!ROLL || (ONE && XB && MT > 1 && F != LX_W_BF16X), "rolling: one batch, the packed image, several activation rows");
  extern __shared__ __align__(16) float lds[];
  const int steps = a.steps;
  const int per_row = x_row_words<F, XB>(a.phase_steps > 0 ? a.phase_steps : steps);
  float* xs = lds;
  float* partial = lds + MT * per_row;  // [waves][MT * R] when S > 1

  const int lane = threadIdx.x & (kWave - 1), wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int S = a.split;
  const int part = wave & (S - 1);  // which share of the steps
  const int group = blockIdx.x * ((blockDim.x / kWave) >> a.split_log2) + (wave >> a.split_log2);
  const int64_t rb = a.row_bytes;
  // Part p of S takes the contiguous steps [p * per, (p + 1) * per).
  const int s_begin = min(steps, part * a.steps_per_part), s_end = min(steps, s_begin + a.steps_per_part);

  auto rows_fn = [&](int g, const uint8_t* (&rows)[R], const uint8_t* (&scales)[R], const float* (&x_image)[R]) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int64_t n = min(g * R + r, a.N - 1);  // past the end: stream a valid row, write nothing
      rows[r] = a.w + n * rb;
      scales[r] = a.scale + n * a.scale_row_bytes;
      x_image[r] = xs;
    }
  };
  // A group's MT * R lane sums become wave sums sixteen at a time: lane j of a round ends with the sum of output j
  // (activation row j / R, weight row j % R of the group), so the S > 1 exchange and the epilogue run once across the
  // lanes instead of once per output.
  constexpr int NO = MT * R, PER = NO < 16 ? NO : 16;
  // What lane j's outputs of group g need besides their sums: the weight row's factor and bias (the same weight row in
  // every round of sixteen when there are several, as 16 is a multiple of R).
  struct Epilogue {
    float rf, bias;
  };
  auto pre_fn = [&](int g) {
    const int64_t n = min(static_cast<int64_t>(g) * R + (lane & (PER - 1)) % R, static_cast<int64_t>(a.N) - 1);
    Epilogue e;
    e.rf = row_factor(F, a.scale, a.global, n);
    e.bias = a.bias ? load_as_f32(a.bias, a.bias_dtype, n) : 0.0f;
    return e;
  };
  auto finish = [&](int g, float (&acc)[MT][R], const Epilogue& e) {
#pragma unroll
    for (int o0 = 0; o0 < NO; o0 += PER) {
      float sum;
      if constexpr (PER == 1) {
        sum = wave_sum(acc[0][0]);
      } else {
        float v[PER];
#pragma unroll
        for (int j = 0; j < PER; ++j) v[j] = acc[(o0 + j) / R][(o0 + j) % R];
        sum = wave_sum_many<PER>(v);
      }
      const int o = o0 + (lane & (PER - 1)), m = o / R, r = o % R;
      if (S > 1) {
        if (lane < PER) partial[wave * NO + o] = sum;
        __syncthreads();
        if (part == 0 && lane < PER)
          for (int p = 1; p < S; ++p) sum += partial[(wave + p) * NO + o];
      }
      if (lane < PER && part == 0 && m < a.M && g * R + r < a.N) write_out(a, m, static_cast<int64_t>(g) * R + r, sum, e.rf, e.bias);
    }
  };
  auto done_fn = [&](int g, float (&acc)[MT][R]) { finish(g, acc, pre_fn(g)); };

  RowStreamer<F, MT, R, U, XB, ONE> st(a.chunks, s_begin, s_end, per_row);
  if constexpr (F == LX_W_BF16X) st.set_bf16x(static_cast<int>(a.K));
  if constexpr (ROLL) {
    // The workgroup's a.rounds consecutive groups go round its wavefronts (the first ones take one more when they do not
    // divide: the device's share of groups per SIMD is then the same everywhere). A group past the last streams the last
    // rows again and writes nothing.
    const int waves_per_wg = blockDim.x / kWave;
    const int group = blockIdx.x * a.rounds + wave;
    // Ask for the activation rows, then for the first group's weights, and only then wait for the rows.
    XRowRegsN<MT> xr;
    stage_rows_load<F>(xr, static_cast<const uint16_t*>(a.x), a.ld_x, nullptr, a.M, a.K, steps);
    st.prefetch(rows_fn, group, 0, 1);
    if (xr.ready) stage_rows_store<F, MT>(xr, reinterpret_cast<uint32_t*>(xs), a.M, a.K, steps);
    else stage_x_pairs<F, MT>(reinterpret_cast<uint32_t*>(xs), static_cast<const uint16_t*>(a.x), a.ld_x, nullptr, a.M, a.K, steps);
    __syncthreads();
    st.run_rolling(rows_fn, pre_fn, finish, group, waves_per_wg, (a.rounds - wave + waves_per_wg - 1) / waves_per_wg);
    return;
  }
  auto stage_all = [&] {
    if constexpr (XB) stage_x_pairs<F, MT>(reinterpret_cast<uint32_t*>(xs), static_cast<const uint16_t*>(a.x), a.ld_x, nullptr, a.M, a.K, steps);
    else stage_x<F, MT>(xs, a.x, a.x_dtype, a.ld_x, nullptr, a.M, a.K, steps);
  };
  if constexpr (MT == 1) {
    // Ask for x, then for the weights, and only then wait for x: loads return in order.
    // Vectors of x a thread holds: a one-batch row of U steps is U * kElems / 8 * 64 values / 8 per vector, over at
    // least 256 threads (a longer row, or f32 activations, may need all four).
    constexpr int XV = ONE && XB ? (U * Fmt<F>::kElems / 32 < 1 ? 1 : U * Fmt<F>::kElems / 32 > 4 ? 4 : U * Fmt<F>::kElems / 32) : 4;
    XRegs<XV> xr;
    stage_x_load<F>(xr, a.x, a.x_dtype, a.ld_x, a.K, steps);
    st.prefetch(rows_fn, group, 0, 1);
    if (xr.ready) {
      if constexpr (XB) stage_x_store_pairs<F>(xr, reinterpret_cast<uint32_t*>(xs), steps);
      else stage_x_store<F>(xr, xs, a.x_dtype, steps);
    } else {
      stage_all();
    }
  } else {
    if constexpr (XB) {
      if (a.phase_steps == 0) {
        // Several bf16 rows: ask for them, then for the weights, and only then wait for the rows (loads return in
        // order): the image is in place while the weights are still on their way, and each chunk is multiplied as it
        // arrives instead of after everything has.
        XRowRegsN<MT> xr;
        stage_rows_load<F>(xr, static_cast<const uint16_t*>(a.x), a.ld_x, nullptr, a.M, a.K, steps);
        st.prefetch(rows_fn, group, 0, 1);
        if (xr.ready) stage_rows_store<F, MT>(xr, reinterpret_cast<uint32_t*>(xs), a.M, a.K, steps);
        else stage_all();
        __syncthreads();
        st.run(rows_fn, done_fn, group, 0, 1);
        return;
      }
    }
    st.prefetch(rows_fn, group, 0, 1);
    if constexpr (XB && ONE) {
      if (a.phase_steps > 0) {
        // Long rows and several activation rows: the image holds half of K at a time.
        const int64_t phase_k = static_cast<int64_t>(a.phase_steps) * kWave * Fmt<F>::kElems;
        const uint16_t* x16 = static_cast<const uint16_t*>(a.x);
        uint32_t* image = reinterpret_cast<uint32_t*>(xs);
        stage_x_pairs<F, MT>(image, x16, a.ld_x, nullptr, a.M, a.K < phase_k ? a.K : phase_k, a.phase_steps);
        __syncthreads();
        st.run_two_images(rows_fn, done_fn, group, a.phase_steps, [&] {
          __syncthreads();
          stage_x_pairs<F, MT>(image, x16 + phase_k, a.ld_x, nullptr, a.M, a.K > phase_k ? a.K - phase_k : 0, a.phase_steps);
          __syncthreads();
        });
        return;
      }
    }
    stage_all();
  }
  __syncthreads();
  st.run(rows_fn, done_fn, group, 0, 1);
}

// Any K, any alignment, x read where it lies: one wavefront per output row, lanes striding over k, the
// lane sums combined by the same tree. Rows whose bytes cannot be read 16 at a time take this kernel
// (the choice depends on K and the weight's address only, never on M).
__global__ void __launch_bounds__(kThreads) gemv_plain_kernel(const GemvArgs a, int wtype) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t n = static_cast<int64_t>(blockIdx.x) * (kThreads / kWave) + threadIdx.x / kWave;
  if (n >= a.N) return;
  float acc[8];
#pragma unroll
  for (int m = 0; m < 8; ++m) acc[m] = 0.0f;
  for (int64_t k = lane; k < a.K; k += kWave) {
    const float w = weight_element_any(wtype, a.w, a.scale, n, k, a.K);
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
  while (S < 4 && (static_cast<int64_t>(N) + R - 1) / R * S < 2LL * cus && steps >= 2 * S) S *= 2;
  return S;
}

// How a launch is shaped. None of it changes an output's bits (only S does).
struct Shape {
  int threads;  // workgroup size
  int depth;    // U: steps asked for at once; a wavefront holds R = 8 / U rows (4 at most)
};

// Measured on MI355X at the decode shapes: a wavefront should own about 8 KB of weights, all requested at once,
// so rows of few steps are taken several at a time.
Shape shape_for(int wtype, int steps) {
  Shape s{wtype == LX_W_NVFP4 ? 512 : 256, batch_depth(steps, 8)};
  return s;
}

template <int F, int MT, int R, int U, bool XB>
int launch_stream(GemvArgs a, const Shape& shape, hipStream_t stream) {
  const int waves = shape.threads / kWave;
  const size_t lds = sizeof(float) * (static_cast<size_t>(MT) * x_row_words<F, XB>(a.phase_steps > 0 ? a.phase_steps : a.steps) + waves * MT * R);
  const int groups_per_wg = waves / a.split;
  const int64_t n_groups = (a.N + R - 1) / R;
  int64_t grid = (n_groups + groups_per_wg - 1) / groups_per_wg;
  auto launch = [&](auto kernel) {
    if (lds > 48 * 1024) {
      static thread_local bool raised = false;  // one per kernel: the lambda is instantiated per kernel type
      if (!raised) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                160 * 1024 - 256) != hipSuccess)
          (void)hipGetLastError();
        raised = true;
      }
    }
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(grid)), dim3(shape.threads), lds, stream, a);
    return status_of(hipGetLastError());
  };
  a.rounds = 1;
  if constexpr (MT > 1 && XB && F != LX_W_BF16X) {
    if (a.phase_steps == 0 && a.split == 1 && a.steps_per_part <= U) {
      // The workgroups the device holds at once (asked once per kernel and workgroup shape).
      static thread_local int held_for_lds = -1, held = 0;
      if (held_for_lds != static_cast<int>(lds)) {
        int per_cu = 0;
        if (lds > 48 * 1024) (void)hipFuncSetAttribute(reinterpret_cast<const void*>(gemv_stream_kernel<F, MT, R, U, XB, true, true>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 256);
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, gemv_stream_kernel<F, MT, R, U, XB, true, true>, shape.threads, lds) != hipSuccess) {
          (void)hipGetLastError();
          per_cu = 0;
        }
        held = per_cu * compute_units();
        held_for_lds = static_cast<int>(lds);
      }
      if (held > 0 && grid > held) {
        a.rounds = static_cast<int>((n_groups + held - 1) / held);  // groups per workgroup
        if (a.rounds < waves) a.rounds = waves;
        grid = (n_groups + a.rounds - 1) / a.rounds;
        return launch(gemv_stream_kernel<F, MT, R, U, XB, true, true>);
      }
    }
  }
  return a.steps_per_part <= U ? launch(gemv_stream_kernel<F, MT, R, U, XB, true>) : launch(gemv_stream_kernel<F, MT, R, U, XB, false>);
}

// A wavefront asks for about 8 KB (one activation row) or 16 KB (several: the rows' products share the
// activation reads) of weights at once: rows of few steps are taken several at a time.
template <int F, int MT, bool XB>
int launch_rows(const GemvArgs& a, const Shape& shape, hipStream_t stream) {
  if constexpr (MT == 1) {
    // Rows of five or six steps (K = 5120, 6144 of one-byte weights) are asked for whole, like those of seven below: as
    // batches of two steps they would be three round trips, as a batch of eight a third of the loads would be repeats.
    if (a.split == 1 && a.steps == 5) return launch_stream<F, MT, 1, 5, XB>(a, shape, stream);
    if (a.split == 1 && a.steps == 6) return launch_stream<F, MT, 1, 6, XB>(a, shape, stream);
    // Rows of 9 .. 14 steps in two even batches of one row (they were 4 + 4 + x of two rows, or 8 + x): 4096 rows of 9216 ..
    // 14336 one-byte values 8.7 .. 11.6 -> 8.2 .. 11.3 us, bf16 11008 x 4608 .. 7168 18.4 .. 25.0 -> 16.3 .. 24.4 (one-byte
    // 11008 x 9216 / 10240 lose 4 - 6 %).
    if (a.split == 1 && a.steps >= 9 && a.steps <= 14) {
      switch ((a.steps + 1) / 2) {
        case 5: return launch_stream<F, MT, 1, 5, XB>(a, shape, stream);
        case 6: return launch_stream<F, MT, 1, 6, XB>(a, shape, stream);
        default: return launch_stream<F, MT, 1, 7, XB>(a, shape, stream);
      }
    }
    switch (shape.depth) {
      case 8:
        // Rows of exactly seven steps (K = 14336 in NVFP4) are asked for whole, without an eighth, repeated load.
        if (a.split == 1 && a.steps == 7) return launch_stream<F, MT, 1, 7, XB>(a, shape, stream);
        return launch_stream<F, MT, 1, 8, XB>(a, shape, stream);
      case 4: return launch_stream<F, MT, 2, 4, XB>(a, shape, stream);
      case 2: return launch_stream<F, MT, 4, 2, XB>(a, shape, stream);
      default: return launch_stream<F, MT, 4, 1, XB>(a, shape, stream);
    }
  } else {
    switch (shape.depth) {
      case 8: return launch_stream<F, MT, 2, 8, XB>(a, shape, stream);
      case 4: return launch_stream<F, MT, 2, 4, XB>(a, shape, stream);
      case 2: return launch_stream<F, MT, 4, 2, XB>(a, shape, stream);
      default: return launch_stream<F, MT, 4, 1, XB>(a, shape, stream);
    }
  }
}

template <int F>
int launch_format(GemvArgs& a, const char* kernel_name, hipStream_t stream) {
  constexpr int R = 2;  // the order class counts row groups of two
  const int64_t rb = row_bytes<F>(a.K);
  const int steps = steps_for<F>(a.K);
  // BF16X: a lane's loads are 8 and 4 bytes within 8-byte aligned records, eight values at a time.
  const bool vector_rows = F == LX_W_BF16X ? a.K % 8 == 0 && reinterpret_cast<uintptr_t>(a.w) % 8 == 0
                                           : rb % 16 == 0 && reinterpret_cast<uintptr_t>(a.w) % 16 == 0 &&
                                                 (F != LX_W_NVFP4 || reinterpret_cast<uintptr_t>(a.scale) % 2 == 0);
  // Activation rows a pass can hold in LDS: a function of K only. More rows than that run as several
  // passes over the weights; each row's arithmetic is the same in any pass, so its bits do not change.
  const bool xb = a.x_dtype == LX_BF16;
  const int64_t row_words = xb ? x_row_words<F, true>(steps) : x_row_words<F, false>(steps);
  int fit = 8;
  while (fit >= 1 && fit * row_words + kMaxWaves * fit * 4 > kLdsFloats) fit /= 2;
  // Rows too long for the call's activation rows to share one image: two images in turn, each half of K (bf16
  // activations, a row's steps in one batch, no K split), rather than a second pass over the weights.
  a.phase_steps = 0;
  if (xb && vector_rows && fit >= 1 && fit < (a.M <= 8 ? a.M : 8) && steps >= 2 && steps <= 8 && batch_depth(steps, 8) >= steps &&
      (a.K * 2) % 16 == 0 && reinterpret_cast<uintptr_t>(a.x) % 16 == 0 && (a.ld_x * 2) % 16 == 0) {
    const int half = (steps + 1) / 2;
    int fit_half = 8;
    while (fit_half >= 1 && fit_half * static_cast<int64_t>(x_row_words<F, true>(half)) + kMaxWaves * fit_half * 4 > kLdsFloats) fit_half /= 2;
    if (fit_half > fit && order_class<F>(a.N, a.K, R) == 1) {
      fit = fit_half;
      a.phase_steps = half;
    }
  }
  if (!vector_rows || fit < 1) {
    const int waves = kThreads / kWave;
    const unsigned grid = static_cast<unsigned>((a.N + waves - 1) / waves);
    hipLaunchKernelGGL(gemv_plain_kernel, dim3(grid), dim3(kThreads), 0, stream, a, F);
    return status_of(hipGetLastError());
  }
  a.split = order_class<F>(a.N, a.K, R);
  const int tuned = tuned_variant(kernel_name, a.M, a.N, static_cast<int>(a.K));
  if (tuned >= 0 && tuned <= 2 && a.phase_steps == 0) a.split = 1 << tuned;
  a.split_log2 = a.split == 4 ? 2 : a.split == 2 ? 1 : 0;
  a.steps = steps;
  a.steps_per_part = (steps + a.split - 1) / a.split;
  const RowBase<F> base(a.w, a.scale, a.K);
  a.w = base.data;
  a.scale = base.scale;
  a.chunks = base.chunks;
  a.row_bytes = rb;
  a.scale_row_bytes = base.scale_row;
  const int M = a.M, phase_steps = a.phase_steps;
  const char* x0 = static_cast<const char*>(a.x);
  char* y0 = static_cast<char*>(a.y);
  const int64_t x_row = a.ld_x * (a.x_dtype == LX_BF16 ? 2 : 4), y_row = a.ld_y * (a.y_dtype == LX_BF16 ? 2 : 4);
  for (int m0 = 0; m0 < M; m0 += fit) {
    a.M = M - m0 < fit ? M - m0 : fit;
    a.x = x0 + m0 * x_row;
    a.y = y0 + m0 * y_row;
    const int mt = a.M <= 1 ? 1 : a.M <= 2 ? 2 : a.M <= 4 ? 4 : 8;
    // A pass of one row stages its whole row (the single-row kernel has no phases; one row of any streamed K fits).
    a.phase_steps = mt >= 2 ? phase_steps : 0;
    Shape shape = shape_for(F, steps);
    // Several activation rows, or one of more than 8192 values: more wavefronts behind one image, which every workgroup
    // stages for itself (4096 x 14336 fp8 at one row 13.8 -> 11.7 us, 11008 x 11008 25.0 -> 22.5, bf16 4096 x 14336 20.6 -> 19.6).
    if (mt >= 2 || a.K > 8192) shape.threads = 512;
    int st;
    switch (mt) {
      case 1: st = xb ? launch_rows<F, 1, true>(a, shape, stream) : launch_rows<F, 1, false>(a, shape, stream); break;
      case 2: st = xb ? launch_rows<F, 2, true>(a, shape, stream) : launch_rows<F, 2, false>(a, shape, stream); break;
      case 4: st = xb ? launch_rows<F, 4, true>(a, shape, stream) : launch_rows<F, 4, false>(a, shape, stream); break;
      default: st = xb ? launch_rows<F, 8, true>(a, shape, stream) : launch_rows<F, 8, false>(a, shape, stream); break;
    }
    if (st) return st;
  }
  return kOk;
}

bool valid_dtype(int d) { return d == LX_F32 || d == LX_BF16; }

}  // namespace

// One format's GEMV, defined in gemv_<format>.hip.
int gemv_launch_bf16(GemvArgs& a, hipStream_t stream);
int gemv_launch_int8(GemvArgs& a, hipStream_t stream);
int gemv_launch_fp8(GemvArgs& a, hipStream_t stream);
int gemv_launch_nvfp4(GemvArgs& a, hipStream_t stream);
int gemv_launch_bf16x(GemvArgs& a, hipStream_t stream);

}  // namespace dro
