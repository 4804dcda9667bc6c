// What the matrix-core products' kernels take: the call's operands and the launch geometry the host worked out,
// and the epilogue they share (engine/cpu/gemm.cpp:21-34).
#pragma once

#include "common.h"

namespace dro {

constexpr size_t kLdsMax = 160 * 1024;  // LDS a workgroup may take

struct XRows {
  const void* x;
  int dtype;
  int64_t ld;  // elements between rows
};

struct GemmArgs {
  XRows xs;
  const uint8_t* w;
  const uint8_t* scale;
  float global;
  const void* bias;
  int bias_dtype;
  void* y;
  int y_dtype;
  int64_t ld_y;
  int M, N, K;
  float alpha, beta;
  int chunks, steps, steps_per_wave, S;
  int64_t row_bytes, scale_row_bytes;
  int tiles_per_wg, x_vecs, x_row_vecs, x_pitch, x_iters;  // the LDS activation image (XL kernels)
  int x_phased;  // lean kernel with two slices a wavefront: the image holds half of K at a time
  int win;       // windowed kernel: load steps of every slice the image holds at a time (2, 4 or 8)
  int win_steps_shift, win_shift, row_shift;  // log2 of win, of the 16-byte pieces in a window, and in an image row
  const int8_t* xq;     // the INT8 math: quantised activations [M, K], rows K bytes apart
  const float* xscale;  // and their per-row scales
  const float* act_scale;  // BF16-math kernels on a quantised math's activation images: the rows' scales (else null)
  int pass_begin, pass_steps, pass_continues;  // slab kernel: the part of every slice this launch takes, and whether it goes on from `partial`
  void* partial;  // slab kernel with S > 1: the slices' partial tiles, [S][tile][16 rows][lane] x 4 words (f32, or i32 for the INT8 math)
  int walk_slices;  // walk kernel with partial tiles: the slices a workgroup walks; split over a workgroup's wavefronts: the slices a wavefront walks
  int walk_split;   // walk kernel: the wavefronts of a workgroup take one tile between them (two or four of them)
};

// The epilogue's operation order (engine/cpu/gemm.cpp:21-34); rf is the row factor, b the bias (0 without one).
__device__ __forceinline__ void write_out(const GemmArgs& a, int m, int n, float sum, float rf, float b) {
  float t = (a.act_scale ? rf * a.act_scale[m] : rf) * sum;
  if (a.bias) t += b;
  float v = a.alpha * t;
  const int64_t at = m * a.ld_y + n;
  if (a.beta != 0.0f) v = a.beta * load_as_f32(a.y, a.y_dtype, at) + v;
  store_from_f32(a.y, a.y_dtype, at, v);
}

__device__ __forceinline__ void write_out(const GemmArgs& a, int wtype, int m, int n, float sum) {
  write_out(a, m, n, sum, row_factor(wtype, a.scale, a.global, n), a.bias ? load_as_f32(a.bias, a.bias_dtype, n) : 0.0f);
}

// gemm_walk_<format>.hip: the walk kernel (gemm_walk.h) for up to 64 bf16 activation rows with W tiles a workgroup
// (1, 2 or 4; with a.partial set, 4 or 8, and a workgroup walks a.walk_slices slices and leaves their sums there; with a.walk_split
// set, W = 2 or 4 wavefronts on one tile); false when it does not apply to the call (the caller then takes another kernel), otherwise *status holds
// the launch's status.
bool launch_walk_bf16(const GemmArgs& a, int W, int* status, hipStream_t stream);
bool launch_walk_int8(const GemmArgs& a, int W, int* status, hipStream_t stream);
bool launch_walk_fp8(const GemmArgs& a, int W, int* status, hipStream_t stream);
bool launch_walk_nvfp4(const GemmArgs& a, int W, int* status, hipStream_t stream);

}  // namespace dro
