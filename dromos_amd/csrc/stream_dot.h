// The weight-streaming dot product shared by the decode GEMV and the decode experts.
//
// A wavefront owns R weight rows at a time and streams them whole: at step s, lane l reads the 16 bytes
// at chunk s * 64 + l of each row (one 128-bit non-temporal load, 1 KB contiguous per row per wave), so a
// row's bytes are read exactly once, in order. The activations sit in LDS as f32, laid out so that the
// 16 bytes a lane reads next are always 16 bytes after its neighbour's (no bank conflicts): the k values
// of chunk (s, l) are stored as kElems / 4 groups of four, group q at float index
//   s * 64 * kElems + q * 256 + l * 4.
// Every (activation row, weight row) pair keeps one f32 accumulator per lane, fed in ascending step
// order, and the 64 lane sums are combined by one fixed tree (wave_sum). The order never depends on how
// many activation rows share the pass (MT) or how many weight rows the wave holds (R), so an output's
// bits depend only on its own x row, its weight row and the K split.
#pragma once

#include "common.h"

namespace dro {

// Float index in the LDS image of x of element j of chunk (s, l); see the layout above.
template <int F>
__device__ __forceinline__ int x_slot(int s, int l, int j) {
  constexpr int E = Fmt<F>::kElems;
  return s * (kWave * E) + (j >> 2) * 256 + l * 4 + (j & 3);
}

// Floats the LDS image of one x row takes for a K of `steps` wave steps.
template <int F>
__host__ __device__ constexpr int x_row_floats(int steps) {
  return steps * kWave * Fmt<F>::kElems;
}

// Wave steps that cover K values of format F.
template <int F>
__host__ __device__ inline int steps_for(int64_t K) {
  const int64_t per_step = static_cast<int64_t>(kWave) * Fmt<F>::kElems;
  return static_cast<int>((K + per_step - 1) / per_step);
}

// Stages rows [0, M) of x (f32 or bf16, row stride ld_x, optionally gathered through row_of[m]) into the
// LDS image `xs` for MT rows of `steps` steps each; everything past K, and rows M .. MT - 1, are zero.
// Called by the whole workgroup; the caller synchronises afterwards.
template <int F, int MT>
__device__ __forceinline__ void stage_x(float* xs, const void* x, int x_dtype, int64_t ld_x, const int* row_of, int M,
                                        int64_t K, int steps) {
  constexpr int E = Fmt<F>::kElems;
  const int per_row = steps * kWave * E;
  for (int m = 0; m < MT; ++m) {
    float* dst = xs + m * per_row;
    if (m >= M) {
      for (int i = threadIdx.x; i < per_row; i += blockDim.x) dst[i] = 0.0f;
      continue;
    }
    const int64_t base = static_cast<int64_t>(row_of ? row_of[m] : m) * ld_x;
    for (int k = threadIdx.x; k < per_row; k += blockDim.x) {
      const float v = k < K ? load_as_f32(x, x_dtype, base + k) : 0.0f;
      const int s = k / (kWave * E), within = k % (kWave * E);
      dst[x_slot<F>(s, within / E, within % E)] = v;
    }
  }
}

// What a lane holds of one weight row for one step: its 16 bytes, and for NVFP4 the two block scales.
template <int F>
struct Chunk {
  u32x4 w;
  uint32_t scales;  // NVFP4: two e4m3 bytes (block of dwords 0-1, block of dwords 2-3)
};

template <int F>
__device__ __forceinline__ Chunk<F> load_chunk(const uint8_t* row, const uint8_t* row_scales, int chunk, bool valid) {
  Chunk<F> c;
  c.w = u32x4{0u, 0u, 0u, 0u};
  c.scales = 0u;
  if (valid) {
    c.w = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(row) + chunk);
    if constexpr (F == LX_W_NVFP4)
      c.scales = __builtin_nontemporal_load(reinterpret_cast<const uint16_t*>(row_scales) + chunk);
  }
  return c;
}

// acc[m] += sum over the chunk's k of x[m, k] * w[k], for MT activation rows; xs points at the LDS image of
// row 0 for this lane's chunk (x_slot(s, lane, 0)), per_row floats separate the rows.
template <int F, int MT>
__device__ __forceinline__ void chunk_fma(const Chunk<F>& c, const float* xs, int per_row, float (&acc)[MT]) {
  constexpr int DV = DwordVals<F>::kCount;  // values per dword
  if constexpr (F == LX_W_NVFP4) {
    // Two blocks of 16 codes: each block's products are summed from zero and take the block scale once.
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const float scale = b == 0 ? e4m3_byte_to_f32<0>(c.scales) : e4m3_byte_to_f32<1>(c.scales);
      float part[MT];
#pragma unroll
      for (int m = 0; m < MT; ++m) part[m] = 0.0f;
#pragma unroll
      for (int d = 0; d < 2; ++d) {
        float w[8];
        decode_dword<F>(c.w[2 * b + d], w);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int q = (2 * b + d) * 2 + h;  // group of four k
#pragma unroll
          for (int m = 0; m < MT; ++m) {
            const f32x4 xv = *reinterpret_cast<const f32x4*>(xs + m * per_row + q * 256);
            part[m] = __builtin_fmaf(xv.x, w[4 * h + 0], part[m]);
            part[m] = __builtin_fmaf(xv.y, w[4 * h + 1], part[m]);
            part[m] = __builtin_fmaf(xv.z, w[4 * h + 2], part[m]);
            part[m] = __builtin_fmaf(xv.w, w[4 * h + 3], part[m]);
          }
        }
      }
#pragma unroll
      for (int m = 0; m < MT; ++m) acc[m] = __builtin_fmaf(part[m], scale, acc[m]);
    }
  } else {
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      float w[DV];
      decode_dword<F>(c.w[d], w);
      if constexpr (DV == 2) {
        // bf16: a dword is half a group of four
        const int q = d >> 1, off = (d & 1) * 2;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          const f32x2 xv = *reinterpret_cast<const f32x2*>(xs + m * per_row + q * 256 + off);
          acc[m] = __builtin_fmaf(xv.x, w[0], acc[m]);
          acc[m] = __builtin_fmaf(xv.y, w[1], acc[m]);
        }
      } else {
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          const f32x4 xv = *reinterpret_cast<const f32x4*>(xs + m * per_row + d * 256);
          acc[m] = __builtin_fmaf(xv.x, w[0], acc[m]);
          acc[m] = __builtin_fmaf(xv.y, w[1], acc[m]);
          acc[m] = __builtin_fmaf(xv.z, w[2], acc[m]);
          acc[m] = __builtin_fmaf(xv.w, w[3], acc[m]);
        }
      }
    }
  }
}

// acc[m][r] = sum_k x[m, k] * row_r[k] over steps [s_begin, s_end) of R rows, U steps of loads in flight.
// rows[r] / scales[r] point at the rows' first bytes; a row has `chunks` 16-byte chunks. Lane sums only:
// the caller reduces across the wave.
template <int F, int MT, int R, int U>
__device__ __forceinline__ void stream_rows(const uint8_t* const (&rows)[R], const uint8_t* const (&scales)[R],
                                            int chunks, int s_begin, int s_end, const float* xs, int per_row,
                                            float (&acc)[MT][R]) {
  const int lane = threadIdx.x & (kWave - 1);
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int r = 0; r < R; ++r) acc[m][r] = 0.0f;
  for (int s0 = s_begin; s0 < s_end; s0 += U) {
    Chunk<F> c[U][R];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int chunk = (s0 + u) * kWave + lane;
      const bool valid = s0 + u < s_end && chunk < chunks;
#pragma unroll
      for (int r = 0; r < R; ++r) c[u][r] = load_chunk<F>(rows[r], scales[r], chunk, valid);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (s0 + u < s_end) {
        const float* xl = xs + x_slot<F>(s0 + u, lane, 0);
#pragma unroll
        for (int r = 0; r < R; ++r) {
          float a[MT];
#pragma unroll
          for (int m = 0; m < MT; ++m) a[m] = acc[m][r];
          chunk_fma<F, MT>(c[u][r], xl, per_row, a);
#pragma unroll
          for (int m = 0; m < MT; ++m) acc[m][r] = a[m];
        }
      }
    }
  }
}

}  // namespace dro
