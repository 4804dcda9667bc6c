// The matrix-core product shared by the skinny GEMM and the grouped experts.
//
// One wavefront multiplies NT tiles of 16 weight rows by up to 64 activation rows (MT tiles of 16) over a slice
// of K with v_mfma_f32_16x16x32_bf16. The weights are the A operand, so a lane ends up holding four
// consecutive output columns n of one activation row m (D[i = 4 * (lane / 16) + r][j = lane % 16], i the
// weight row, j the activation row): a 16-byte store per lane.
//
// Weights are read where they lie, 16 bytes per lane per load: lane (g = lane / 16, i = lane % 16) reads chunk
// 4 * t + g of row i at load step t, which is kElems consecutive k, i.e. kElems / 8 matrix instructions' worth.
// The instruction sums over k in whatever order the operands present it, so instruction j of a load step simply
// takes each lane's elements [8j, 8j + 8) on both sides: the activation fragment of lane (g, m) for that
// instruction is x[m, (4t + g) * kElems + 8j .. + 8]. Quantised weights are expanded to bf16 exactly in
// registers (int8 and e4m3 fit bf16's 8 significant bits; an e2m1 code times its e4m3 block scale has at most
// six), activations are bf16 (f32 activations are rounded to bf16 first: the BF16 math), sums are f32.
//
// S wavefronts of a workgroup split the load steps of one tile into contiguous slices; each slice is an
// ascending f32 chain from zero and the slices are added in ascending order through LDS. S depends on K and
// the format only, so an output's bits depend on its activation row, its weight row and nothing else.
#pragma once

#include "common.h"

namespace dro {

constexpr int kTileRows = 16;     // weight rows per tile
constexpr int kMaxSplit = 16;     // wavefronts per workgroup at most
constexpr int kLoadsInFlight = 8; // load steps a wavefront asks for at once

// Load steps (4 chunks of 16 bytes per row each) that cover a row of K values.
template <int F>
__host__ __device__ inline int load_steps_for(int64_t K) {
  const int64_t chunks = row_bytes<F>(K) / 16;
  return static_cast<int>((chunks + 3) / 4);
}

// The K split for rows of K values in format F when a wavefront holds NT tiles: enough wavefronts that each
// asks for its whole slice at once, at most kMaxSplit. A function of (F, K, NT) only.
template <int F>
inline int split_for(int64_t K, int NT) {
  const int steps = load_steps_for<F>(K);
  const int per_wave = kLoadsInFlight / NT;
  int S = (steps + per_wave - 1) / per_wave;
  if (S > kMaxSplit) S = kMaxSplit;
  if (S < 1) S = 1;
  return S;
}

// Eight consecutive values of a lane's 16 bytes as the A operand: instruction j of the load step.
template <int F>
__device__ __forceinline__ bf16x8 weight_fragment(const u32x4& w, uint32_t scales, int j);

template <>
__device__ __forceinline__ bf16x8 weight_fragment<LX_W_BF16>(const u32x4& w, uint32_t, int) {
  return __builtin_bit_cast(bf16x8, w);
}

__device__ __forceinline__ bf16x2 pack_bf16(float a, float b) {
  const f32x2 v = {a, b};
  return __builtin_convertvector(v, bf16x2);  // v_cvt_pk_bf16_f32, nearest even; exact for the values here
}

template <>
__device__ __forceinline__ bf16x8 weight_fragment<LX_W_INT8>(const u32x4& w, uint32_t, int j) {
  const uint32_t d0 = j == 0 ? w.x : w.z, d1 = j == 0 ? w.y : w.w;
  float v[8];
  decode_dword<LX_W_INT8>(d0, v);
  decode_dword<LX_W_INT8>(d1, v + 4);
  bf16x2 p[4] = {pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]), pack_bf16(v[4], v[5]), pack_bf16(v[6], v[7])};
  return __builtin_bit_cast(bf16x8, p);
}

template <>
__device__ __forceinline__ bf16x8 weight_fragment<LX_W_FP8>(const u32x4& w, uint32_t, int j) {
  const uint32_t d0 = j == 0 ? w.x : w.z, d1 = j == 0 ? w.y : w.w;
  bf16x2 p[4] = {__builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(d0, 1.0f, false), __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(d0, 1.0f, true),
                 __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(d1, 1.0f, false), __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(d1, 1.0f, true)};
  return __builtin_bit_cast(bf16x8, p);
}

template <>
__device__ __forceinline__ bf16x8 weight_fragment<LX_W_NVFP4>(const u32x4& w, uint32_t scales, int j) {
  // Dword j holds eight codes of block j / 2 of the lane's two blocks; the block scale is applied here, where
  // the product is still exact (the matrix instruction mixes blocks of different lanes).
  const uint32_t d = j == 0 ? w.x : j == 1 ? w.y : j == 2 ? w.z : w.w;
  const float s = j < 2 ? e4m3_byte_to_f32<0>(scales) : e4m3_byte_to_f32<1>(scales);
  float v[8];
  decode_dword<LX_W_NVFP4>(d, v);
  bf16x2 p[4] = {pack_bf16(v[0] * s, v[1] * s), pack_bf16(v[2] * s, v[3] * s), pack_bf16(v[4] * s, v[5] * s),
                 pack_bf16(v[6] * s, v[7] * s)};
  return __builtin_bit_cast(bf16x8, p);
}

// Where a wavefront's activation fragments come from: rows of bf16 or f32 in global memory whose addresses and
// strides are multiples of 16 bytes. XF32 says which; the caller resolves each lane's row pointers (one per
// activation tile, clamped into the matrix: the columns of a clamped row are computed and never written).
template <bool XF32>
struct XFrag {
  u32x4 raw[XF32 ? 2 : 1];
};

// x[row, k .. k + 8) as loaded; k is clamped into the row (a fragment past K is zeroed when it is used).
template <bool XF32>
__device__ __forceinline__ void load_x_fragment(XFrag<XF32>& f, const void* row, int k, int K) {
  const int kc = min(k, K - 8);
  if constexpr (XF32) {
    const u32x4* p = reinterpret_cast<const u32x4*>(static_cast<const float*>(row) + kc);
    f.raw[0] = p[0];
    f.raw[1] = p[1];
  } else {
    f.raw[0] = *reinterpret_cast<const u32x4*>(static_cast<const uint16_t*>(row) + kc);
  }
}

// The fragment as the B operand: bf16 as it is, f32 rounded to bf16 (nearest even); zero past K.
template <bool XF32>
__device__ __forceinline__ bf16x8 x_operand(const XFrag<XF32>& f, int k, int K) {
  u32x4 v;
  if constexpr (XF32) {
    bf16x2 q[4] = {pack_bf16(__uint_as_float(f.raw[0].x), __uint_as_float(f.raw[0].y)),
                   pack_bf16(__uint_as_float(f.raw[0].z), __uint_as_float(f.raw[0].w)),
                   pack_bf16(__uint_as_float(f.raw[1].x), __uint_as_float(f.raw[1].y)),
                   pack_bf16(__uint_as_float(f.raw[1].z), __uint_as_float(f.raw[1].w))};
    v = __builtin_bit_cast(u32x4, q);
  } else {
    v = f.raw[0];
  }
  if (k >= K) v = u32x4{0u, 0u, 0u, 0u};
  return __builtin_bit_cast(bf16x8, v);
}

// Load steps asked for at once: bounded by the registers the activation fragments of a batch take
// (steps x instructions per step x activation tiles x 4 or 8 registers), at most kLoadsInFlight / NT.
template <int F, int NT, int MT, bool XF32>
constexpr int batch_steps() {
  constexpr int J = Fmt<F>::kElems / 8;
  int u = 16 / (J * MT * (XF32 ? 2 : 1));
  const int cap = kLoadsInFlight / NT;
  u = u > cap ? cap : u;
  return u < 1 ? 1 : u;
}

// acc[t][mt] += tile t's rows times activation tile mt over load steps [t_begin, t_end).
// rows[t] / scales[t] point at this lane's weight row of tile t (row i = lane % 16 of the tile, clamped into the
// matrix by the caller); xrow[mt] at this lane's activation row of tile mt. `chunks` is the number of 16-byte
// chunks in a weight row. Every load of a batch, weights and activations, is asked for before the first use.
template <int F, int NT, int MT, bool XF32>
__device__ __forceinline__ void mfma_slice(const uint8_t* const (&rows)[NT], const uint8_t* const (&scales)[NT], int chunks,
                                           int t_begin, int t_end, const void* const (&xrow)[MT], int K, f32x4 (&acc)[NT][MT]) {
  constexpr int E = Fmt<F>::kElems;
  constexpr int J = E / 8;  // matrix instructions per load step
  constexpr int U = batch_steps<F, NT, MT, XF32>();
  const int lane = threadIdx.x & (kWave - 1);
  const int g = lane >> 4;
  for (int tb = t_begin; tb < t_end; tb += U) {
    u32x4 wv[U][NT];
    uint32_t sc[U][NT];
    XFrag<XF32> xf[U][J][MT];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      // A step past the slice, or a chunk past the row's end, re-reads a valid chunk of the same row; its
      // activation fragment is zero (past K) or the step is skipped.
      const int t = min(tb + u, t_end - 1);
      const int c = min(4 * t + g, chunks - 1);
#pragma unroll
      for (int n = 0; n < NT; ++n) {
        wv[u][n] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(rows[n]) + c);
        sc[u][n] = 0;
        if constexpr (F == LX_W_NVFP4) sc[u][n] = __builtin_nontemporal_load(reinterpret_cast<const uint16_t*>(scales[n]) + c);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k0 = (4 * min(tb + u, t_end - 1) + g) * E;
#pragma unroll
      for (int j = 0; j < J; ++j)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) load_x_fragment<XF32>(xf[u][j][mt], xrow[mt], k0 + 8 * j, K);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (tb + u < t_end) {
        const int k0 = (4 * (tb + u) + g) * E;
#pragma unroll
        for (int j = 0; j < J; ++j) {
#pragma unroll
          for (int n = 0; n < NT; ++n) {
            const bf16x8 wf = weight_fragment<F>(wv[u][n], sc[u][n], j);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
              acc[n][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, x_operand<XF32>(xf[u][j][mt], k0 + 8 * j, K), acc[n][mt], 0, 0, 0);
          }
        }
      }
    }
  }
}

// The whole workgroup: wavefront w of S takes load steps [w * per, (w + 1) * per), the partial tiles are added
// in ascending w through `lds` (S * NT * MT * 64 f32x4), and epi(mt, q, sums) is called once for every
// (activation tile mt, lane slot q) with the NT finished sums: sums[t][r] belongs to weight row 4 * (q / 16) + r
// of tile t and activation row mt * 16 + q % 16.
template <int F, int NT, int MT, bool XF32, class Epi>
__device__ __forceinline__ void mfma_tile(const uint8_t* const (&rows)[NT], const uint8_t* const (&scales)[NT], int chunks,
                                          int steps, int steps_per_wave, const void* const (&xrow)[MT], int K, f32x4* lds,
                                          Epi&& epi) {
  const int lane = threadIdx.x & (kWave - 1), wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int S = blockDim.x / kWave;
  f32x4 acc[NT][MT];
#pragma unroll
  for (int n = 0; n < NT; ++n)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[n][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int t_begin = min(steps, wave * steps_per_wave), t_end = min(steps, t_begin + steps_per_wave);
  mfma_slice<F, NT, MT, XF32>(rows, scales, chunks, t_begin, t_end, xrow, K, acc);
  if (S == 1) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      f32x4 sums[NT];
#pragma unroll
      for (int n = 0; n < NT; ++n) sums[n] = acc[n][mt];
      epi(mt, lane, sums);
    }
    return;
  }
#pragma unroll
  for (int n = 0; n < NT; ++n)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) lds[((wave * NT + n) * MT + mt) * kWave + lane] = acc[n][mt];
  __syncthreads();
  for (int item = threadIdx.x; item < MT * kWave; item += blockDim.x) {
    const int mt = item / kWave, q = item % kWave;
    f32x4 sums[NT];
#pragma unroll
    for (int n = 0; n < NT; ++n) {
      f32x4 s = lds[((0 * NT + n) * MT + mt) * kWave + q];
      for (int w = 1; w < S; ++w) s += lds[((w * NT + n) * MT + mt) * kWave + q];
      sums[n] = s;
    }
    epi(mt, q, sums);
  }
}

}  // namespace dro
