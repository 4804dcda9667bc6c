// Batched decode products on the matrix cores: lx_gemm_skinny, lx_gemm_w (LX_MATH_BF16), and lx_gemv_w's entry
// (contracts: engine/cuda/kernels.h:433-477; CPU behaviour of the BF16 math: engine/cpu/gemm.cpp:189-296).
//
//   y[m, n] = alpha * (rowfactor[n] * sum_k bf16(x[m, k]) * w[n, k] + bias[n]) + beta * y[m, n]
//
// One workgroup per tile of 16 weight rows; its S wavefronts split K (tile_mfma.h) and each asks for its whole
// slice of the weights at once. Up to 64 activation rows ride along in one pass (more rows are further passes).
// Neither S nor anything else that shapes a sum depends on M, so a row's bits are the same in any batch: the
// reduction-order contract of the skinny GEMM, for every weight format.
#include <stdlib.h>

#include <map>
#include <mutex>
#include <type_traits>
#include <utility>

#include "common.h"
#include "gemm_args.h"
#include "tile_mfma.h"

namespace dro {

int gemv_any(const void* x, int x_dtype, int ld_x, const lx_weight& w, const void* bias, int bias_dtype, void* y,
             int y_dtype, int ld_y, int M, int N, int K, float alpha, float beta, void* stream);

namespace {

// XL: the activation rows (at most 16, MT == 1) are staged once per workgroup into LDS as bf16, behind the
// wavefronts' regions: rows of x_row_vecs * 8 values (K rounded up to whole weight batches, zero from K on),
// x_pitch = that + 8 elements apart (16 bytes off a multiple of the banks' span, so the 16 rows of a fragment read
// fall into different banks). A workgroup then holds `tiles_per_wg` tiles of S wavefronts each, which share the
// image. Otherwise (any M up to 64) the fragments are read from global memory and a workgroup is one tile.
// LEAN (NVFP4, whose nibble decode does not fit the 128 registers a wavefront has in a workgroup of sixteen: 90 to 256
// registers spilled with two to four activation tiles): the same kernel compiled for the workgroups of at most LEAN = 4
// or 8 wavefronts that most shapes ask for (at 4, three wavefronts a SIMD, what measured best in the grouped experts,
// which are this code), with the block scales read eight bytes at a time (the launcher checks that they can be).
template <int F, int MT, bool XF32, bool XL, int LEAN = 0>
__global__ void __launch_bounds__((LEAN ? LEAN : kMaxSplit) * kWave) __attribute__((amdgpu_waves_per_eu(LEAN == 4 ? 3 : 1)))
skinny_kernel(const GemmArgs a) {
  extern __shared__ __align__(16) f32x4 lds4[];
  static_assert(!XL || MT == 1, "only one activation tile is staged in LDS");
  constexpr int kRegion = wave_region_bytes<1, MT>();
  const int lane = threadIdx.x & (kWave - 1), wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int S = a.S, tile_in_wg = XL ? wave / S : 0, slice = XL ? wave - tile_in_wg * S : wave;
  // A tile past the last one (an odd count of tiles and two to a workgroup) repeats the last tile; its outputs are
  // not written.
  const int tile_raw = blockIdx.x * (XL ? a.tiles_per_wg : 1) + tile_in_wg;
  const int n_tiles = (a.N + kTileRows - 1) / kTileRows;
  const bool tile_live = tile_raw < n_tiles;
  const int n0 = min(tile_raw, n_tiles - 1) * kTileRows;
  // Rows past the end of the matrix stand for its last row: read, and never written.
  const TileRows tiles[1] = {{a.w + n0 * a.row_bytes, a.scale + n0 * a.scale_row_bytes, min(kTileRows, a.N - n0)}};
  uint8_t* const lds_bytes = reinterpret_cast<uint8_t*>(lds4);
  uint16_t* const ximg = reinterpret_cast<uint16_t*>(lds_bytes + (blockDim.x / kWave) * kRegion);
  const void* xrow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = min(mt * 16 + (lane & 15), a.M - 1);
    if constexpr (XL) xrow[mt] = ximg + m * a.x_pitch;
    else xrow[mt] = static_cast<const char*>(a.xs.x) + static_cast<int64_t>(m) * a.xs.ld * (XF32 ? 4 : 2);
  }
  // Staging slots: (row m, pass j) in row-major order; a thread's piece of a slot is vector j * blockDim + thread
  // of row m. The first four slots are asked for before the weights (a wait for them then leaves the weights
  // in flight), with clamped addresses: what lies past K is replaced by zeros when it is stored.
  u32x4 xr[4][XF32 ? 2 : 1];
  auto x_piece = [&](int m, int j, u32x4 (&r)[XF32 ? 2 : 1]) {
    const int v = min(static_cast<int>(threadIdx.x) + j * static_cast<int>(blockDim.x), a.x_vecs - 1);
    const char* src = static_cast<const char*>(a.xs.x) + (static_cast<int64_t>(min(m, a.M - 1)) * a.xs.ld + v * 8) * (XF32 ? 4 : 2);
    r[0] = *reinterpret_cast<const u32x4*>(src);
    if constexpr (XF32) r[1] = *reinterpret_cast<const u32x4*>(src + 16);
  };
  auto x_store = [&](int m, int j, const u32x4 (&r)[XF32 ? 2 : 1]) {
    const int v = threadIdx.x + j * blockDim.x;
    u32x4 val = r[0];
    if constexpr (XF32) {
      bf16x2 q[4] = {pack_bf16(__uint_as_float(r[0].x), __uint_as_float(r[0].y)), pack_bf16(__uint_as_float(r[0].z), __uint_as_float(r[0].w)),
                     pack_bf16(__uint_as_float(r[1].x), __uint_as_float(r[1].y)), pack_bf16(__uint_as_float(r[1].z), __uint_as_float(r[1].w))};
      val = __builtin_bit_cast(u32x4, q);
    }
    if (v >= a.x_vecs) val = u32x4{0u, 0u, 0u, 0u};
    if (v < a.x_row_vecs) *reinterpret_cast<u32x4*>(ximg + m * a.x_pitch + v * 8) = val;
  };
  if constexpr (XL) {
    int m = 0, j = 0;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      x_piece(m, j, xr[u]);
      if (++j == a.x_iters) j = 0, ++m;
    }
  }
  const bool bias_f32 = a.bias && a.bias_dtype == LX_F32;
  float rf[4], bs[4];
  auto between = [&] {
    // The epilogue's row factors and f32 biases: a lane always finishes the same four weight rows.
    const int nq = n0 + 4 * (lane >> 4);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int n = min(nq + r, a.N - 1);
      rf[r] = row_factor(F, a.scale, a.global, n);
      bs[r] = bias_f32 ? static_cast<const float*>(a.bias)[n] : 0.0f;
    }
    if constexpr (XL) {
      int m = 0, j = 0;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (m < a.M) x_store(m, j, xr[u]);
        if (++j == a.x_iters) j = 0, ++m;
      }
      while (m < a.M) {
        u32x4 r[XF32 ? 2 : 1];
        x_piece(m, j, r);
        x_store(m, j, r);
        if (++j == a.x_iters) j = 0, ++m;
      }
      __syncthreads();
    }
  };
  constexpr int XS = XL ? kXLds : XF32 ? kXGlobalF32 : kXGlobalBf16;
  mfma_tile<F, 1, MT, XS, LEAN != 0>(tiles, a.row_bytes, a.scale_row_bytes, a.chunks, a.steps, a.steps_per_wave, xrow, a.K,
                                     reinterpret_cast<f32x4*>(lds_bytes + tile_in_wg * S * kRegion), S, slice, between,
                          [&](int mt, int q, f32x4(&sums)[1]) {
    const int m = mt * 16 + (q & 15), nq = n0 + 4 * (q >> 4);  // q % 64 == lane: rf and bs are this slot's
    if (m < a.M && tile_live) {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (nq + r < a.N)
          write_out(a, m, nq + r, sums[0][r], rf[r], bias_f32 || !a.bias ? bs[r] : load_as_f32(a.bias, a.bias_dtype, nq + r));
    }
  });
}

// ---- up to 16 activation rows: the lean tile kernel ------------------------------------------------------
//
// The same arithmetic as skinny_kernel (one 16 x 16 tile per S wavefronts, contiguous K slices of
// steps_per_wave steps, each an ascending chain from zero, slices added in ascending order through LDS), written
// for the registers: a wavefront keeps its eight weight loads, one staging group's fragments, one step's
// activation fragments and one accumulator, so eight wavefronts fit a SIMD and two 1024-thread workgroups a
// compute unit. The activation rows sit in LDS behind the wavefronts' staging regions: bf16 (BF16 math: f32
// activations are rounded on the way in) or the per-token int8 (INT8 math), rows x_pitch bytes apart, zero from K
// to the end of the last weight batch. MATH: LX_MATH_BF16 (any weight format) or LX_MATH_INT8 (int8 weights).
// VS: K slices a wavefront takes (1, or 2: slice w of the first half of K, then slice w of the second half; the tile
// then needs half the wavefronts and the image only half of K at a time, so a workgroup holds more tiles behind one
// image and a compute unit's whole share is in flight at once; both slices' first loads are asked for up front and
// each slice keeps its own sum, so the order of the sums does not change).
template <int F, int MATH, bool XF32, int VS>
__global__ void __launch_bounds__(kMaxSplit* kWave) __attribute__((amdgpu_waves_per_eu(VS == 2 ? 4 : F == LX_W_NVFP4 ? 6 : 8, 8))) tile16_kernel(const GemmArgs a) {
  extern __shared__ __align__(16) f32x4 lds4[];
  constexpr bool I8 = MATH != LX_MATH_BF16;  // byte activations: the INT8 and FP8 maths
  constexpr int E = Fmt<F>::kElems, J = I8 ? 1 : E / 8;
  using Acc = typename std::conditional<MATH == LX_MATH_INT8, i32x4, f32x4>::type;
  const int lane = threadIdx.x & (kWave - 1), wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int S = a.S, waves_per_tile = S / VS, tile_in_wg = wave / waves_per_tile, wave_in_tile = wave - tile_in_wg * waves_per_tile;
  const int n_tiles = (a.N + kTileRows - 1) / kTileRows;
  const int tile_raw = blockIdx.x * a.tiles_per_wg + tile_in_wg;
  const int n0 = min(tile_raw, n_tiles - 1) * kTileRows;  // a tile past the last repeats it and writes nothing
  const int valid = min(kTileRows, a.N - n0);
  const int g = lane >> 4, i = lane & 15;
  uint8_t* const lds_bytes = reinterpret_cast<uint8_t*>(lds4);
  uint8_t* const tile_lds = lds_bytes + tile_in_wg * waves_per_tile * kStageBytes;
  uint8_t* const stage = tile_lds + wave_in_tile * kStageBytes;
  uint8_t* const ximg = lds_bytes + (blockDim.x / kWave) * kStageBytes;

  // One 16-byte piece of the image per thread is asked for before the weights; the rest after them.
  const char* const xsrc = I8 ? reinterpret_cast<const char*>(a.xq) : static_cast<const char*>(a.xs.x);
  const int64_t x_ld_bytes = I8 ? a.K : a.xs.ld * (XF32 ? 4 : 2);
  // The image holds the k range of one phase (VS == 2: the first half of the slices, then the second); `base` is the
  // phase's first 16-byte piece within a row.
  auto x_piece = [&](int m, int v, int base, u32x4 (&r)[XF32 ? 2 : 1]) {
    const char* src = xsrc + min(m, a.M - 1) * x_ld_bytes + min(base + v, a.x_vecs - 1) * (XF32 ? 32 : 16);
    r[0] = *reinterpret_cast<const u32x4*>(src);
    if constexpr (XF32) r[1] = *reinterpret_cast<const u32x4*>(src + 16);
  };
  auto x_store = [&](int m, int v, int base, const u32x4 (&r)[XF32 ? 2 : 1]) {
    u32x4 val = r[0];
    if constexpr (XF32) {
      bf16x2 q[4] = {pack_bf16(__uint_as_float(r[0].x), __uint_as_float(r[0].y)), pack_bf16(__uint_as_float(r[0].z), __uint_as_float(r[0].w)),
                     pack_bf16(__uint_as_float(r[1].x), __uint_as_float(r[1].y)), pack_bf16(__uint_as_float(r[1].z), __uint_as_float(r[1].w))};
      val = __builtin_bit_cast(u32x4, q);
    }
    if (base + v >= a.x_vecs) val = u32x4{0u, 0u, 0u, 0u};
    // No branch around the store (a piece that belongs nowhere goes to a spare slot behind the image): a branch here
    // makes the wait for x a wait for every load, the weights included.
    const bool placed = m < a.M && v < a.x_row_vecs;
    *reinterpret_cast<u32x4*>(placed ? ximg + m * a.x_pitch + v * 16 : ximg + a.M * a.x_pitch) = val;
  };
  // Pieces are numbered row by row: piece p is vector p % x_row_vecs of row p / x_row_vecs.
  u32x4 xr[XF32 ? 2 : 1];
  const int first_m = threadIdx.x / a.x_row_vecs, first_v = threadIdx.x - first_m * a.x_row_vecs;
  x_piece(first_m, first_v, 0, xr);

  // This lane's loads: rows 4 q + g of the tile, chunk i of each 4-step group (256 contiguous bytes per 16 lanes).
  const uint8_t* const tile_w = a.w + static_cast<int64_t>(n0) * a.row_bytes;
  uint32_t row_off[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) row_off[q] = static_cast<uint32_t>(min(4 * q + g, valid - 1)) * static_cast<uint32_t>(a.row_bytes);
  const uint8_t* const own_scale = a.scale + (static_cast<int64_t>(n0) + min(i, valid - 1)) * a.scale_row_bytes;  // NVFP4 only
  int t_begin[VS], t_end[VS];
#pragma unroll
  for (int v = 0; v < VS; ++v) {
    // Phased: slice w of each half of K; otherwise two neighbouring slices.
    const int slice = a.x_phased ? wave_in_tile + v * waves_per_tile : wave_in_tile * VS + v;
    t_begin[v] = min(a.steps, slice * a.steps_per_wave);
    t_end[v] = min(a.steps, t_begin[v] + a.steps_per_wave);
  }
  u32x4 raw[VS][2][4];
  uint32_t sc[VS][8];
  // Asks for one 4-step group of a batch (grp 0 or 1 of the batch at step tb) of slice v.
  auto issue_group = [&](int v, int tb, int grp) {
    const uint32_t c = static_cast<uint32_t>(min(4 * (tb + 4 * grp) + i, a.chunks - 1)) * 16u;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const uint32_t off = row_off[q] + c;  // one 32-bit offset from the tile's (uniform) base
      raw[v][grp][q] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(tile_w + off));
    }
    if constexpr (F == LX_W_NVFP4) {
#pragma unroll
      for (int u = 0; u < 4; ++u)
        sc[v][4 * grp + u] = __builtin_nontemporal_load(reinterpret_cast<const uint16_t*>(own_scale) + min(4 * (tb + 4 * grp + u) + g, a.chunks - 1));
    }
  };
  auto issue = [&](int v, int tb) {
    issue_group(v, tb, 0);
    issue_group(v, tb, 1);
  };
  // Unconditionally (an empty slice reads clamped addresses): the wait for x can then count past these loads.
#pragma unroll
  for (int v = 0; v < VS; ++v) issue(v, t_begin[v]);

  x_store(first_m, first_v, 0, xr);
  auto stage_image = [&](int base, int first_piece) {
    for (int v = first_piece; v < a.M * a.x_row_vecs; v += blockDim.x) {
      const int m = v / a.x_row_vecs, vv = v - m * a.x_row_vecs;
      u32x4 r[XF32 ? 2 : 1];
      x_piece(m, vv, base, r);
      x_store(m, vv, base, r);
    }
    __syncthreads();
  };
  stage_image(0, threadIdx.x + blockDim.x);  // the other pieces, if any

  u32x4* const put = reinterpret_cast<u32x4*>(stage + g * kStagePitch + i * 16);
  const u32x4* const get = reinterpret_cast<const u32x4*>(stage + i * kStagePitch + g * 16);
  const uint8_t* const xrow = ximg + min(i, a.M - 1) * a.x_pitch + g * (I8 ? 16 : E * 2);  // + step * 4 chunks
  Acc acc[VS];
#pragma unroll
  for (int v = 0; v < VS; ++v) {
    acc[v] = Acc{0, 0, 0, 0};
    const int phase_t0 = a.x_phased ? v * waves_per_tile * a.steps_per_wave : 0;  // the image starts at this step's k
    if (v > 0 && a.x_phased) {
      __syncthreads();  // every wavefront is done with the first phase's image
      stage_image(v * a.x_row_vecs, threadIdx.x);
    }
    for (int tb = t_begin[v]; tb < t_end[v]; tb += 8) {
#pragma unroll
      for (int grp = 0; grp < 2; ++grp) {
        uint32_t scales[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) scales[u] = F == LX_W_NVFP4 ? sc[v][4 * grp + u] : 0u;
#pragma unroll
        for (int q = 0; q < 4; ++q) put[q * (4 * kStagePitch / 16)] = raw[v][grp][q];
        // The group's registers are free: ask for the same group of the slice's next batch, so a wavefront that
        // walks a long slice always has a batch in flight.
        if (tb + 8 < t_end[v]) issue_group(v, tb + 8, grp);
        wave_lds_order();
        // Two steps' fragments at a time keep the registers of eight wavefronts a SIMD.
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          u32x4 wv[2];
#pragma unroll
          for (int st = 0; st < 2; ++st) wv[st] = get[(2 * half + st) * 4];
#pragma unroll
          for (int st = 0; st < 2; ++st) {
            const int step = 4 * grp + 2 * half + st;
            const uint8_t* xs = xrow + (tb + step - phase_t0) * 4 * (I8 ? 16 : E * 2);
            if constexpr (I8) {
              acc[v] = byte_mfma<MATH>(__builtin_bit_cast(i32x4, wv[st]), *reinterpret_cast<const i32x4*>(xs), acc[v]);
            } else {
#pragma unroll
              for (int j = 0; j < J; ++j)
                acc[v] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(weight_fragment<F>(wv[st], scales[2 * half + st], j),
                                                                 *reinterpret_cast<const bf16x8*>(xs + 16 * j), acc[v], 0, 0, 0);
            }
          }
        }
        wave_lds_order();
      }
    }
  }

  // The S partial tiles (each in the region of the wavefront that made it, at its first or second place) are added in ascending slice order by
  // the tile's first wavefront, which asks for its epilogue factors before it waits for the others.
  Acc* const mine = reinterpret_cast<Acc*>(stage);
  if (S > 1) {
    wave_lds_order();
#pragma unroll
    for (int v = 0; v < VS; ++v) mine[v * kWave + lane] = acc[v];
  }
  float rf[4], bs[4];
  const int nq = n0 + 4 * g, m = i;
  const bool bias_f32 = a.bias && a.bias_dtype == LX_F32;
  if (wave_in_tile == 0) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int n = min(nq + r, a.N - 1);
      rf[r] = I8 ? reinterpret_cast<const float*>(a.scale)[n] : row_factor(F, a.scale, a.global, n);
      bs[r] = bias_f32 ? static_cast<const float*>(a.bias)[n] : 0.0f;
    }
  }
  if (S > 1) __syncthreads();
  if (wave_in_tile != 0 || m >= a.M || tile_raw >= n_tiles) return;
  Acc sum = acc[0];
  for (int sl = 1; sl < S; ++sl) {
    const int region = a.x_phased ? sl % waves_per_tile : sl / VS, sub = a.x_phased ? sl / waves_per_tile : sl % VS;
    sum += reinterpret_cast<const Acc*>(tile_lds + region * kStageBytes)[sub * kWave + lane];
  }
  const float xs = I8 ? a.xscale[m] : 1.0f;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    if (nq + r < a.N) {
      const float b = bias_f32 || !a.bias ? bs[r] : load_as_f32(a.bias, a.bias_dtype, nq + r);
      write_out(a, m, nq + r, static_cast<float>(sum[r]), I8 ? rf[r] * xs : rf[r], b);
    }
  }
}

// ---- up to 64 activation rows: the windowed tile kernel --------------------------------------------------------
//
// The arithmetic of the kernels above (one 16-row weight tile per S wavefronts, wavefront w taking the contiguous K
// slice of steps_per_wave load steps [w * spw, (w + 1) * spw) as one ascending chain from zero, the S partial tiles
// added in ascending order through LDS) for MT tiles of 16 activation rows at once, with an activation image that is
// small whatever M and K are: it holds, for every slice, only a window of WIN load steps (2, 4, or 8 = one weight
// batch), and moves along the slices with the wavefronts. A workgroup is `tiles_per_wg` tiles (their wavefronts share
// the image); the window is restaged between two barriers whenever the wavefronts cross into the next one (they all
// do so at the same step of their own slices). Neither the window nor the number of tiles per workgroup enters a
// sum, so a row's bits are those of every other kernel here.
//
// Loads return in the order they were asked for, so what a wavefront waits for decides what stays in flight behind
// it. The order here: a window's activations are asked for one window ahead and wait in registers; the next batch's
// weights are asked for two loads at a time right before each place where a window may be crossed, so the wait for
// the activations at a crossing always leaves weight loads in flight; between the two barriers of a crossing there
// are only LDS writes. The loops are peeled (first batch: no crossing at its start; last batch: nothing to ask for)
// so that every wait is a fixed count.
// MATH as in tile16_kernel; a step past the end of the row is skipped (its clamped loads are not multiplied).
template <int F, int MATH, bool XF32, int MT>
__global__ void __launch_bounds__(kMaxSplit* kWave) window_kernel(const GemmArgs a) {
  extern __shared__ __align__(16) f32x4 lds4[];
  constexpr bool I8 = MATH != LX_MATH_BF16;
  constexpr int E = Fmt<F>::kElems, J = I8 ? 1 : E / 8;
  constexpr int CB = I8 ? 16 : E * 2;  // image bytes under one lane's 16-byte weight chunk
  constexpr int SB = 4 * CB;           // image bytes of one load step
  constexpr int SP = SB / 16;          // and its 16-byte pieces
  using Acc = typename std::conditional<MATH == LX_MATH_INT8, i32x4, f32x4>::type;
  const int lane = threadIdx.x & (kWave - 1), wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int S = a.S, tile_in_wg = wave / S, w = wave - tile_in_wg * S;
  const int n_tiles = (a.N + kTileRows - 1) / kTileRows;
  const int tile_raw = blockIdx.x * a.tiles_per_wg + tile_in_wg;
  const int n0 = min(tile_raw, n_tiles - 1) * kTileRows;  // a tile past the last repeats it and writes nothing
  const int valid = min(kTileRows, a.N - n0);
  const int g = lane >> 4, i = lane & 15;
  uint8_t* const lds_bytes = reinterpret_cast<uint8_t*>(lds4);
  uint8_t* const tile_lds = lds_bytes + tile_in_wg * S * kStageBytes;
  uint8_t* const stage = tile_lds + w * kStageBytes;
  uint8_t* const ximg = lds_bytes + (blockDim.x / kWave) * kStageBytes;
  const int spw = a.steps_per_wave, WIN = a.win, kWinShift = a.win_steps_shift;

  // The image of window p: row m holds, slice after slice, the activations under steps [ws * spw + p * WIN, + WIN) of
  // slice ws; zero from K on. Pieces of 16 image bytes, numbered row by row; S is a power of two, so a piece's row,
  // slice and place in the window are shifts and masks of its number. A thread holds kAhead pieces (the launcher
  // sizes the window so that this covers the image).
  constexpr int kAhead = XF32 ? 2 : 4;
  const char* const xsrc = I8 ? reinterpret_cast<const char*>(a.xq) : static_cast<const char*>(a.xs.x);
  const int64_t x_ld_bytes = I8 ? a.K : a.xs.ld * (XF32 ? 4 : 2);
  const int win_shift = a.win_shift, row_shift = a.row_shift;  // log2 of the pieces in a window, in an image row
  const int pieces = a.M << row_shift;
  u32x4 xr[kAhead][XF32 ? 2 : 1];
  auto window_load = [&](int p) {
#pragma unroll
    for (int u = 0; u < kAhead; ++u) {
      const int v = min(static_cast<int>(threadIdx.x) + u * static_cast<int>(blockDim.x), pieces - 1);
      const int m = v >> row_shift, c = v & ((1 << row_shift) - 1);
      const int ws = c >> win_shift, cc = c & ((1 << win_shift) - 1);
      const int piece = min((ws * spw + p * WIN) * SP + cc, a.x_vecs - 1);  // of the activation row; clamped, zeroed when stored
      const char* src = xsrc + m * x_ld_bytes + static_cast<int64_t>(piece) * (XF32 ? 32 : 16);
      xr[u][0] = *reinterpret_cast<const u32x4*>(src);
      if constexpr (XF32) xr[u][1] = *reinterpret_cast<const u32x4*>(src + 16);
    }
  };
  auto window_store = [&](int p) {
#pragma unroll
    for (int u = 0; u < kAhead; ++u) {
      const int v = threadIdx.x + u * blockDim.x;
      const int m = v >> row_shift, c = v & ((1 << row_shift) - 1);
      const int ws = c >> win_shift, cc = c & ((1 << win_shift) - 1);
      const int piece = (ws * spw + p * WIN) * SP + cc;
      u32x4 val = xr[u][0];
      if constexpr (XF32) {
        bf16x2 q[4] = {pack_bf16(__uint_as_float(xr[u][0].x), __uint_as_float(xr[u][0].y)),
                       pack_bf16(__uint_as_float(xr[u][0].z), __uint_as_float(xr[u][0].w)),
                       pack_bf16(__uint_as_float(xr[u][1].x), __uint_as_float(xr[u][1].y)),
                       pack_bf16(__uint_as_float(xr[u][1].z), __uint_as_float(xr[u][1].w))};
        val = __builtin_bit_cast(u32x4, q);
      }
      if (piece >= a.x_vecs) val = u32x4{0u, 0u, 0u, 0u};
      // No branch around the store (a piece past the image goes to a spare slot behind it): a branch would make the
      // wait for these pieces a wait for every load in flight, the weights included.
      *reinterpret_cast<u32x4*>(ximg + (v < pieces ? m * a.x_pitch + c * 16 : a.M * a.x_pitch)) = val;
    }
  };
  const int n_windows = (spw + WIN - 1) >> kWinShift;
  window_load(0);

  // This lane's loads: rows 4 q + g of the tile, chunk i of each 4-step group (256 contiguous bytes per 16 lanes).
  const uint8_t* const tile_w = a.w + static_cast<int64_t>(n0) * a.row_bytes;
  uint32_t row_off[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) row_off[q] = static_cast<uint32_t>(min(4 * q + g, valid - 1)) * static_cast<uint32_t>(a.row_bytes);
  const uint8_t* const own_scale = a.scale + (static_cast<int64_t>(n0) + min(i, valid - 1)) * a.scale_row_bytes;  // NVFP4 only
  const int t_begin = w * spw;
  u32x4 raw[2][4];
  uint32_t sc[8];
  auto issue_group = [&](int tb, int grp) {
    const uint32_t c = static_cast<uint32_t>(min(4 * (tb + 4 * grp) + i, a.chunks - 1)) * 16u;
#pragma unroll
    for (int q = 0; q < 4; ++q) raw[grp][q] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(tile_w + (row_off[q] + c)));
    if constexpr (F == LX_W_NVFP4) {
#pragma unroll
      for (int u = 0; u < 4; ++u)
        sc[4 * grp + u] = __builtin_nontemporal_load(reinterpret_cast<const uint16_t*>(own_scale) + min(4 * (tb + 4 * grp + u) + g, a.chunks - 1));
    }
  };
  issue_group(t_begin, 0);
  issue_group(t_begin, 1);
  window_store(0);
  if (n_windows > 1) window_load(1);
  __syncthreads();

  u32x4* const put = reinterpret_cast<u32x4*>(stage + g * kStagePitch + i * 16);
  const u32x4* const get = reinterpret_cast<const u32x4*>(stage + i * kStagePitch + g * 16);
  const uint8_t* xrow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) xrow[mt] = ximg + min(mt * 16 + i, a.M - 1) * a.x_pitch + w * WIN * SB + g * CB;
  Acc acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = Acc{0, 0, 0, 0};
  for (int off = 0; off < spw; off += 8) {  // the same trip count for every wavefront: the loop holds barriers
#pragma unroll
    for (int grp = 0; grp < 2; ++grp) {
      uint32_t scales[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) scales[u] = F == LX_W_NVFP4 ? sc[4 * grp + u] : 0u;
#pragma unroll
      for (int q = 0; q < 4; ++q) put[q * (4 * kStagePitch / 16)] = raw[grp][q];
      if (off + 8 < spw) issue_group(t_begin + off + 8, grp);  // the same group of the next batch
      wave_lds_order();
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const int so = off + 4 * grp + 2 * half;  // step within the slice
        const int in_window = so & (WIN - 1);
        if (so > 0 && in_window == 0) {
          const int p = so >> kWinShift;
          __syncthreads();  // every wavefront is done with the window before
          window_store(p);
          if (p + 1 < n_windows) window_load(p + 1);
          __syncthreads();
        }
        u32x4 wv[2];
#pragma unroll
        for (int st = 0; st < 2; ++st) wv[st] = get[(2 * half + st) * 4];
#pragma unroll
        for (int st = 0; st < 2; ++st) {
          if (t_begin + so + st < a.steps) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
              const uint8_t* xs = xrow[mt] + (in_window + st) * SB;
              if constexpr (I8) {
                acc[mt] = byte_mfma<MATH>(__builtin_bit_cast(i32x4, wv[st]), *reinterpret_cast<const i32x4*>(xs), acc[mt]);
              } else {
#pragma unroll
                for (int j = 0; j < J; ++j)
                  acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(weight_fragment<F>(wv[st], scales[2 * half + st], j),
                                                                    *reinterpret_cast<const bf16x8*>(xs + 16 * j), acc[mt], 0, 0, 0);
              }
            }
          }
        }
      }
      wave_lds_order();
    }
  }

  // The S partial tiles, added in ascending slice order by the tile's first wavefront.
  Acc* const mine = reinterpret_cast<Acc*>(stage);
  if (S > 1) {
    wave_lds_order();
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) mine[mt * kWave + lane] = acc[mt];
  }
  float rf[4], bs[4];
  const int nq = n0 + 4 * g;
  const bool bias_f32 = a.bias && a.bias_dtype == LX_F32;
  if (w == 0) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int n = min(nq + r, a.N - 1);
      rf[r] = I8 ? reinterpret_cast<const float*>(a.scale)[n] : row_factor(F, a.scale, a.global, n);
      bs[r] = bias_f32 ? static_cast<const float*>(a.bias)[n] : 0.0f;
    }
  }
  if (S > 1) __syncthreads();
  if (w != 0 || tile_raw >= n_tiles) return;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + i;
    if (m >= a.M) continue;
    Acc sum = acc[mt];
    for (int sl = 1; sl < S; ++sl) sum += reinterpret_cast<const Acc*>(tile_lds + sl * kStageBytes)[mt * kWave + lane];
    const float xscale = I8 ? a.xscale[m] : 1.0f;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      if (nq + r < a.N) {
        const float b = bias_f32 || !a.bias ? bs[r] : load_as_f32(a.bias, a.bias_dtype, nq + r);
        write_out(a, m, nq + r, static_cast<float>(sum[r]), I8 ? rf[r] * xscale : rf[r], b);
      }
    }
  }
}

// Launches the windowed kernel for a.M <= 64 rows; false when no window fits (K slices too many for one workgroup).
template <int F, int MATH>
bool launch_window(GemmArgs a, int* status, hipStream_t stream) {
  constexpr bool I8 = MATH != LX_MATH_BF16;
  constexpr int SB = 4 * (I8 ? 16 : Fmt<F>::kElems * 2);
  const int S = a.S, spw = a.steps_per_wave;
  if (S > kMaxSplit || (S & (S - 1)) != 0 || spw % 8 != 0) return false;
  const bool xf32 = !I8 && a.xs.dtype == LX_F32;
  const unsigned n_tiles = static_cast<unsigned>((a.N + kTileRows - 1) / kTileRows);
  auto image = [&](int win) { return static_cast<size_t>(a.M) * (static_cast<size_t>(S) * win * SB + 16) + 16; };
  auto lds_for = [&](int tpw, int win) { return static_cast<size_t>(tpw) * S * kStageBytes + image(win); };
  // Tiles to a workgroup: four at most (the more tiles share an image, the less the activations cost, but workgroups
  // of sixteen wavefronts are too few to cover the device: 16384 x 4096 at 32 rows 24.7 -> 20.9 us with four tiles).
  int tpw = kMaxSplit / S < 4 ? kMaxSplit / S : 4;
  // Up to 32 rows, fewer tiles where that fills the device better: 512 tiles in fours are 128 workgroups for 256 compute
  // units, in twos one each (8192 x 4096 fp8 at 16 / 32 rows: 13.0 / 17.5 -> 11.5 / 15.0 us).
  if (a.M <= 32) {
    const int cus = compute_units();
    auto fill = [&](int t) {
      const int wgs = (static_cast<int>(n_tiles) + t - 1) / t, rounds = (wgs + cus - 1) / cus;
      return static_cast<double>(wgs) / (static_cast<double>(rounds) * cus);
    };
    while (tpw > 1 && fill(tpw) < 0.6 && fill(tpw / 2) > fill(tpw)) tpw /= 2;
  }
  // The window: the largest of 8, 4, 2 steps whose image fits LDS and whose pieces its threads can hold.
  const size_t held = (xf32 ? 2u : 4u) * tpw * S * kWave;
  int win = 8;
  while (win > 2 && (lds_for(tpw, win) > kLdsMax - 1024 || static_cast<size_t>(a.M) * S * win * (SB / 16) > held)) win /= 2;
  if (lds_for(tpw, win) > kLdsMax - 1024 || static_cast<size_t>(a.M) * S * win * (SB / 16) > held) return false;
  auto log2i = [](int v) { int l = 0; while ((1 << l) < v) ++l; return l; };
  a.tiles_per_wg = tpw;
  a.win = win;
  a.win_steps_shift = log2i(win);
  a.win_shift = log2i(win * (SB / 16));
  a.row_shift = log2i(S * win * (SB / 16));
  a.x_vecs = a.K * (I8 ? 1 : 2) / 16;
  a.x_pitch = S * win * SB + 16;
  const size_t lds = lds_for(tpw, win);
  const unsigned threads = tpw * S * kWave, grid = (n_tiles + tpw - 1) / tpw;
  auto launch = [&](auto kernel) {
    if (lds > 48 * 1024) allow_lds(reinterpret_cast<const void*>(kernel), kLdsMax);
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(threads), lds, stream, a);
    return status_of(hipGetLastError());
  };
  auto with_mt = [&](auto mt_tag) {
    constexpr int MT = decltype(mt_tag)::value;
    auto with_x = [&](auto x_tag) {
      constexpr bool XF = decltype(x_tag)::value;
      return launch(window_kernel<F, MATH, XF, MT>);
    };
    if constexpr (I8) return with_x(std::false_type{});
    else return xf32 ? with_x(std::true_type{}) : with_x(std::false_type{});
  };
  switch ((a.M + 15) / 16) {
    case 1: *status = with_mt(std::integral_constant<int, 1>{}); break;
    case 2: *status = with_mt(std::integral_constant<int, 2>{}); break;
    case 3: *status = with_mt(std::integral_constant<int, 3>{}); break;
    default: *status = with_mt(std::integral_constant<int, 4>{}); break;
  }
  return true;
}

// ---- up to 64 activation rows, many tiles: the slab kernel ------------------------------------------------------
//
// The same arithmetic once more (a tile's K slices, each one ascending chain from zero, added in ascending order), laid
// out so that the activations cost little: a workgroup takes ONE K slice (blockIdx.y) of many tiles, so its image is
// the slice's columns of the M rows and nothing else, staged once; its wavefronts then walk their tiles' slices without
// ever meeting again (no window to cross, no barrier after the first). With S > 1 the slices of a tile are in different
// workgroups: each writes its partial tile to `partial`, and slab_reduce_kernel adds them in ascending slice order and
// runs the epilogue, which is what the other kernels' first wavefront does through LDS. Neither the tiles a workgroup
// takes nor which wavefront takes which enters a sum.
template <int F, int MATH, bool XF32, int MT>
__global__ void __launch_bounds__(kMaxSplit* kWave) slab_kernel(const GemmArgs a) {
  extern __shared__ __align__(16) f32x4 lds4[];
  constexpr bool I8 = MATH != LX_MATH_BF16;
  constexpr int E = Fmt<F>::kElems, J = I8 ? 1 : E / 8;
  constexpr int CB = I8 ? 16 : E * 2;  // image bytes under one lane's 16-byte weight chunk
  constexpr int SB = 4 * CB;           // image bytes of one load step
  constexpr int SP = SB / 16;          // and its 16-byte pieces
  using Acc = typename std::conditional<MATH == LX_MATH_INT8, i32x4, f32x4>::type;
  const int lane = threadIdx.x & (kWave - 1), wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int waves = blockDim.x / kWave;
  // This launch takes steps [pass_begin, pass_begin + pass_steps) of every slice (the whole slice where its image fits).
  const int S = a.S, w = blockIdx.y, spw = a.pass_steps, t_begin = w * a.steps_per_wave + a.pass_begin;
  const int n_tiles = (a.N + kTileRows - 1) / kTileRows;
  const int tile_first = blockIdx.x * a.tiles_per_wg, tile_end = min(n_tiles, tile_first + a.tiles_per_wg);
  const int g = lane >> 4, i = lane & 15;
  uint8_t* const ximg = reinterpret_cast<uint8_t*>(lds4);

  // A tile's loads, straight into the lanes that feed the matrix instruction: lane (g, i) takes chunk 4 s + g of row i
  // for load step s (64 contiguous bytes of each of the tile's 16 rows per instruction). The LDS belongs to the image.
  struct TilePtrs {
    const uint8_t* row;        // this lane's row of the tile
    const uint8_t* own_scale;  // NVFP4: its block scales
  };
  auto ptrs_of = [&](int t) {
    TilePtrs p;
    const int n0 = min(t, n_tiles - 1) * kTileRows, valid = min(kTileRows, a.N - n0);
    const int64_t n = static_cast<int64_t>(n0) + min(i, valid - 1);
    p.row = a.w + n * a.row_bytes;
    p.own_scale = a.scale + n * a.scale_row_bytes;
    return p;
  };
  u32x4 raw[2][4];
  uint32_t sc[8];
  auto issue_group = [&](const TilePtrs& p, int tb, int grp) {
#pragma unroll
    for (int st = 0; st < 4; ++st) {
      const int c = min(4 * (tb + 4 * grp + st) + g, a.chunks - 1);
      raw[grp][st] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p.row + static_cast<uint32_t>(c) * 16u));
      if constexpr (F == LX_W_NVFP4) sc[4 * grp + st] = __builtin_nontemporal_load(reinterpret_cast<const uint16_t*>(p.own_scale) + c);
    }
  };
  int tile = tile_first + wave;
  TilePtrs cur = ptrs_of(tile);

  // The image: row m holds the activations under steps [t_begin, t_begin + spw), zero from K on, in pieces of 16 image
  // bytes. Loads return in the order they were asked for: the first round of activations is asked for BEFORE the
  // weights, so the image is complete (and the matrix instructions can start on the first weights) while most of the
  // weights are still on their way; asked for behind them, the activations would arrive last and the whole slab would
  // be loaded before any of it is multiplied.
  {
    const char* const xsrc = I8 ? reinterpret_cast<const char*>(a.xq) : static_cast<const char*>(a.xs.x);
    const int64_t x_ld_bytes = I8 ? a.K : a.xs.ld * (XF32 ? 4 : 2);
    const int row_pieces = spw * SP, pieces = a.M * row_pieces;
    // A piece's row and place in it: a shift and a mask where a row's pieces are a power of two (row_shift >= 0), as
    // they are for most K; a division costs a wavefront dozens of instructions per piece.
    const int row_shift = a.row_shift;
    auto row_of = [&](int v) { return row_shift >= 0 ? v >> row_shift : v / row_pieces; };
    constexpr int kAhead = XF32 ? 4 : 8;
    u32x4 xr[kAhead][XF32 ? 2 : 1];
    auto ask = [&](int v0) {
#pragma unroll
      for (int u = 0; u < kAhead; ++u) {
        const int v = min(v0 + u * static_cast<int>(blockDim.x), pieces - 1);
        const int m = row_of(v), c = v - m * row_pieces;
        const int piece = min(t_begin * SP + c, a.x_vecs - 1);  // clamped, zeroed when stored
        const char* src = xsrc + m * x_ld_bytes + static_cast<int64_t>(piece) * (XF32 ? 32 : 16);
        xr[u][0] = *reinterpret_cast<const u32x4*>(src);
        if constexpr (XF32) xr[u][1] = *reinterpret_cast<const u32x4*>(src + 16);
      }
    };
    auto put = [&](int v0) {
#pragma unroll
      for (int u = 0; u < kAhead; ++u) {
        const int v = v0 + u * blockDim.x;
        const int m = row_of(min(v, pieces - 1)), c = v - m * row_pieces;
        u32x4 val = xr[u][0];
        if constexpr (XF32) {
          bf16x2 q[4] = {pack_bf16(__uint_as_float(xr[u][0].x), __uint_as_float(xr[u][0].y)),
                         pack_bf16(__uint_as_float(xr[u][0].z), __uint_as_float(xr[u][0].w)),
                         pack_bf16(__uint_as_float(xr[u][1].x), __uint_as_float(xr[u][1].y)),
                         pack_bf16(__uint_as_float(xr[u][1].z), __uint_as_float(xr[u][1].w))};
          val = __builtin_bit_cast(u32x4, q);
        }
        if (t_begin * SP + c >= a.x_vecs) val = u32x4{0u, 0u, 0u, 0u};
        // A piece past the image goes to a spare slot behind it (no branch around the store).
        *reinterpret_cast<u32x4*>(ximg + (v < pieces ? m * a.x_pitch + c * 16 : a.M * a.x_pitch)) = val;
      }
    };
    ask(threadIdx.x);
    // (A wavefront without a tile asks for a valid one's all the same: behind a branch the compiler could not count the
    // loads in flight and would make the stores below wait for all of them.)
    issue_group(cur, t_begin, 0);
    issue_group(cur, t_begin, 1);
    put(threadIdx.x);
    for (int v0 = threadIdx.x + kAhead * blockDim.x; v0 < pieces; v0 += kAhead * blockDim.x) {
      ask(v0);
      put(v0);
    }
  }
  __syncthreads();

  const uint8_t* xrow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) xrow[mt] = ximg + min(mt * 16 + i, a.M - 1) * a.x_pitch + g * CB;
  const bool bias_f32 = a.bias && a.bias_dtype == LX_F32;
  for (; tile < tile_end; tile += waves) {
    const int next_tile = tile + waves;
    const TilePtrs next = ptrs_of(next_tile < tile_end ? next_tile : tile);
    // A slice taken in several launches goes on from where the launch before left its chain (the partial tile).
    Acc* const part = static_cast<Acc*>(a.partial) + ((static_cast<int64_t>(w) * n_tiles + tile) * MT) * kWave + lane;
    Acc acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = a.pass_continues ? part[mt * kWave] : Acc{0, 0, 0, 0};
    for (int off = 0; off < spw; off += 8) {
#pragma unroll
      for (int grp = 0; grp < 2; ++grp) {
        uint32_t scales[4];
        u32x4 grp_w[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          scales[u] = F == LX_W_NVFP4 ? sc[4 * grp + u] : 0u;
          grp_w[u] = raw[grp][u];
        }
        // The same group of the next batch: of this tile, or of the wavefront's next one.
        if (off + 8 < spw) issue_group(cur, t_begin + off + 8, grp);
        else if (next_tile < tile_end) issue_group(next, t_begin, grp);
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          const int so = off + 4 * grp + 2 * half;  // step within the slice
          u32x4 wv[2];
#pragma unroll
          for (int st = 0; st < 2; ++st) wv[st] = grp_w[2 * half + st];
#pragma unroll
          for (int st = 0; st < 2; ++st) {
            if (t_begin + so + st < a.steps) {
#pragma unroll
              for (int mt = 0; mt < MT; ++mt) {
                const uint8_t* xs = xrow[mt] + (so + st) * SB;
                if constexpr (I8) {
                  acc[mt] = byte_mfma<MATH>(__builtin_bit_cast(i32x4, wv[st]), *reinterpret_cast<const i32x4*>(xs), acc[mt]);
                } else {
#pragma unroll
                  for (int j = 0; j < J; ++j)
                    acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(weight_fragment<F>(wv[st], scales[2 * half + st], j),
                                                                      *reinterpret_cast<const bf16x8*>(xs + 16 * j), acc[mt], 0, 0, 0);
                }
              }
            }
          }
        }
      }
    }
    // The tile's slice is done: the partial tile, or with one slice the result itself.
    const int nq = tile * kTileRows + 4 * g;
    if (a.partial) {
      // Partial tiles lie as the wavefront holds them: [slice][tile][16 activation rows][lane] vectors of four words, so a
      // store instruction writes 1 KB of whole cache lines (rows of the output would be 64-byte halves of lines, which
      // the cache has to fetch first).
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) part[mt * kWave] = acc[mt];
    } else {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + i;
        if (m >= a.M) continue;
        const float xscale = I8 ? a.xscale[m] : 1.0f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int n = nq + r;
          if (n < a.N) {
            const float rf = I8 ? reinterpret_cast<const float*>(a.scale)[n] : row_factor(F, a.scale, a.global, n);
            const float b = !a.bias ? 0.0f : bias_f32 ? static_cast<const float*>(a.bias)[n] : load_as_f32(a.bias, a.bias_dtype, n);
            write_out(a, m, n, static_cast<float>(acc[mt][r]), I8 ? rf * xscale : rf, b);
          }
        }
      }
    }
    cur = next;
  }
}

// The slab kernel's second half for S > 1: out[m, n] from the S partial sums of (m, n), added in ascending slice order
// from slice 0's, then the epilogue. One thread per (m, four consecutive n).
template <int F, int MATH>
__global__ void __launch_bounds__(256) slab_reduce_kernel(const GemmArgs a, int mts) {
  constexpr bool I8 = MATH != LX_MATH_BF16;
  using Acc = typename std::conditional<MATH == LX_MATH_INT8, i32x4, f32x4>::type;
  const int n_tiles = (a.N + kTileRows - 1) / kTileRows;
  const int64_t vectors = static_cast<int64_t>(n_tiles) * mts * kWave;  // of one slice
  const int64_t item = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (item >= vectors) return;
  const int lane = static_cast<int>(item & (kWave - 1)), mt = static_cast<int>((item >> 6) % mts), tile = static_cast<int>((item >> 6) / mts);
  const int m = mt * 16 + (lane & 15), n0 = tile * kTileRows + 4 * (lane >> 4);
  const Acc* p = static_cast<const Acc*>(a.partial) + item;
  // Up to eight slices' vectors are asked for at once (a slice past the last repeats it and is not added).
  Acc sum = *p;
  for (int base = 1; base < a.S; base += 8) {
    Acc part[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) part[u] = p[min(base + u, a.S - 1) * vectors];
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (base + u < a.S) sum += part[u];
  }
  if (m >= a.M) return;
  const bool bias_f32 = a.bias && a.bias_dtype == LX_F32;
  const float xscale = I8 ? a.xscale[m] : 1.0f;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int n = n0 + r;
    if (n < a.N) {
      const float rf = I8 ? reinterpret_cast<const float*>(a.scale)[n] : row_factor(F, a.scale, a.global, n);
      const float b = !a.bias ? 0.0f : bias_f32 ? static_cast<const float*>(a.bias)[n] : load_as_f32(a.bias, a.bias_dtype, n);
      write_out(a, m, n, static_cast<float>(sum[r]), I8 ? rf * xscale : rf, b);
    }
  }
}

// The slab kernel's partial tiles live in a buffer the library keeps per (device, stream): calls on one stream run one
// after the other, so they can share it. A product never makes one (it neither allocates nor synchronises, and does the
// same under graph capture as outside): the buffer is made when the stream is (lx_rt_stream_create), or when a host
// that brings its own streams reserves one (lx_rt_stream_reserve), and a call on a stream without one takes the windowed
// kernel.
constexpr size_t kSlabScratchBytes = 64u << 20;

struct SlabBuffers {
  std::mutex lock;
  std::map<std::pair<int, hipStream_t>, void*> of;
};
SlabBuffers& slab_buffers() {
  static auto* b = new SlabBuffers;
  return *b;
}

void* slab_scratch(hipStream_t stream, size_t bytes) {
  if (bytes > kSlabScratchBytes) return nullptr;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  SlabBuffers& b = slab_buffers();
  std::lock_guard<std::mutex> g(b.lock);
  auto it = b.of.find({dev, stream});
  return it == b.of.end() ? nullptr : it->second;
}

// Which of the tile kernels' own choices the variant table fixes ("gemm_w_<format>": 4 = never the slab kernel,
// 5 = the slab kernel wherever it fits); anything else leaves the measured rule.
constexpr int kVariantWindow = 4, kVariantSlab = 5, kVariantWalkParts = 6, kVariantWalkSplit = 7;

template <int F>
const char* gemm_key() {
  return F == LX_W_BF16 ? "gemm_w_bf16" : F == LX_W_INT8 ? "gemm_w_int8" : F == LX_W_FP8 ? "gemm_w_fp8" : "gemm_w_nvfp4";
}

// Where the slab kernel is tried before the windowed one. Measured on MI355X (fp8, int8 and bf16 weights, bf16
// activations): it wins where the windowed kernel's workgroups, which each stage all of K, are few or long: more than 32
// rows with at most 400 tiles (6144 x 4096 at 48 rows: 22.7 -> 18.7 us, at 64: 26.2 -> 22.4 us; 4096 x 4096 at 64:
// 21.5 -> 17.6 us), and more than 16 rows with K >= 8192 and few tiles (4096 x 8192 at 32 rows: 21.3 -> 15.3 us, at 64:
// 35.7 -> 22.7 us). With many tiles (14336 x 4096) its second pass over the partial tiles costs more than the windows do.
inline bool slab_wanted(int M, int n_tiles, int64_t K, int tuned) {
  if (tuned == kVariantWindow) return false;
  if (tuned == kVariantSlab) return true;
  return n_tiles <= 400 && (M > 32 || (M > 16 && K >= 8192));
}

// Launches the slab kernel for a.M <= 64 rows; false when it does not apply: the slice's image does not fit LDS, the
// matrix has too few tiles to give every compute unit a slab, or (S > 1) the stream has no buffer for the partial tiles.
template <int F, int MATH>
bool launch_slab(GemmArgs a, int* status, hipStream_t stream) {
  constexpr bool I8 = MATH != LX_MATH_BF16;
  constexpr int SB = 4 * (I8 ? 16 : Fmt<F>::kElems * 2);
  const int S = a.S, spw = a.steps_per_wave;
  if (spw % 8 != 0 || S < 1) return false;
  const bool xf32 = !I8 && a.xs.dtype == LX_F32;
  const int n_tiles = (a.N + kTileRows - 1) / kTileRows;
  // A slice whose image does not fit LDS is taken in several launches of `part` steps each (whole batches of eight): a
  // launch leaves its chains in the partial tiles and the next one goes on from them, so the sums are those of one pass.
  int part = spw;
  while (part > 8 && static_cast<size_t>(a.M) * (static_cast<size_t>(part) * SB + 16) + 16 > kLdsMax - 1024) part -= 8;
  const int passes = (spw + part - 1) / part;
  if (passes > 1 && S == 1) return false;  // the chain is handed on through the partial tiles, which one slice has none of
  if (passes > 3) return false;
  const size_t pitch = static_cast<size_t>(part) * SB + 16;
  const size_t image = static_cast<size_t>(a.M) * pitch + 16;
  // One slab per compute unit and slice round: tiles_per_wg tiles of one slice, up to sixteen wavefronts on them.
  const int slabs = compute_units() / S > 0 ? compute_units() / S : 1;
  const int tpw = (n_tiles + slabs - 1) / slabs;
  const int waves = tpw < 4 ? 4 : tpw > kMaxSplit ? kMaxSplit : tpw;
  const size_t lds = image;
  if (lds > kLdsMax - 1024) return false;
  if (n_tiles * S < compute_units() * 4) return false;  // too little work to give every unit a slab of several tiles
  void* partial = nullptr;
  if (S > 1) {
    const size_t mts = static_cast<size_t>((a.M + 15) / 16);
    partial = slab_scratch(stream, sizeof(float) * 4 * kWave * mts * n_tiles * S);
    if (!partial) return false;
  }
  a.partial = partial;
  a.tiles_per_wg = tpw;
  a.x_vecs = a.K * (I8 ? 1 : 2) / 16;
  a.x_pitch = static_cast<int>(pitch);
  const dim3 grid((n_tiles + tpw - 1) / tpw, S);
  auto launch = [&](auto kernel) {
    if (lds > 48 * 1024) allow_lds(reinterpret_cast<const void*>(kernel), kLdsMax);
    hipLaunchKernelGGL(kernel, grid, dim3(waves * kWave), lds, stream, a);
    return status_of(hipGetLastError());
  };
  auto with_mt = [&](auto mt_tag) {
    constexpr int MT = decltype(mt_tag)::value;
    if constexpr (I8) return launch(slab_kernel<F, MATH, false, MT>);
    else return xf32 ? launch(slab_kernel<F, MATH, true, MT>) : launch(slab_kernel<F, MATH, false, MT>);
  };
  int st = kOk;
  for (int begin = 0; begin < spw && !st; begin += part) {
    a.pass_begin = begin;
    a.pass_steps = spw - begin < part ? spw - begin : part;
    a.pass_continues = begin > 0;
    const int row_pieces = a.pass_steps * (SB / 16);
    a.row_shift = -1;
    for (int sh = 0; sh < 20; ++sh)
      if ((1 << sh) == row_pieces) a.row_shift = sh;
    switch ((a.M + 15) / 16) {
      case 1: st = with_mt(std::integral_constant<int, 1>{}); break;
      case 2: st = with_mt(std::integral_constant<int, 2>{}); break;
      case 3: st = with_mt(std::integral_constant<int, 3>{}); break;
      default: st = with_mt(std::integral_constant<int, 4>{}); break;
    }
  }
  if (!st && S > 1) {
    const int mts = (a.M + 15) / 16;
    const int64_t items = static_cast<int64_t>(n_tiles) * mts * kWave;
    hipLaunchKernelGGL((slab_reduce_kernel<F, MATH>), dim3(static_cast<unsigned>((items + 255) / 256)), dim3(256), 0, stream, a, mts);
    st = status_of(hipGetLastError());
  }
  *status = st;
  return true;
}

// Launches the lean tile kernel for a.M <= 16 rows when its LDS image fits; false if it does not.
template <int F, int MATH>
bool launch_tile16(GemmArgs a, int* status, hipStream_t stream) {
  constexpr bool I8 = MATH != LX_MATH_BF16;
  const int S = a.S;
  const unsigned n_tiles = static_cast<unsigned>((a.N + kTileRows - 1) / kTileRows);
  // The activation image: rows as long as the slices it serves (all of them, or half of them at a time), zero past K.
  const int esize = I8 ? 1 : 2;
  const int step_bytes = 4 * (I8 ? 16 : Fmt<F>::kElems * 2);  // image bytes of one load step
  // Several activation rows: the image takes the LDS more workgroups would need, so a wavefront takes two slices,
  // one in each half of K, the image holds half of K at a time and the workgroup more tiles.
  // (With slices of several batches and few rows the image is small and one slice a wavefront keeps more wavefronts
  // busy.)
  const bool two_slices = a.M >= 2 && S % 2 == 0 && n_tiles >= 512 && (a.steps_per_wave == kLoadsInFlight || a.M > 4);
  const int waves_per_tile = two_slices ? S / 2 : S;
  int tiles_per_wg = 1, row_bytes = 0;
  size_t best = 0, image = 0;
  auto lds_for = [&](int tpw) { return static_cast<size_t>(tpw) * waves_per_tile * kStageBytes + image; };
  // The image of all of K if a compute unit then still holds sixteen wavefronts, else (two slices a wavefront) of half
  // of K at a time, staged twice.
  for (int phased = 0; phased <= (two_slices ? 1 : 0); ++phased) {
    row_bytes = (phased ? waves_per_tile : S) * a.steps_per_wave * step_bytes;
    image = static_cast<size_t>(a.M) * (row_bytes + 16) + 16;  // and a spare slot
    tiles_per_wg = 1;
    best = 0;
    // Tiles to a workgroup: whichever lets a compute unit hold most wavefronts.
    for (int tpw = 1; tpw * waves_per_tile <= kMaxSplit; tpw *= 2) {
      if (lds_for(tpw) > kLdsMax || (tpw > 1 && n_tiles < 512)) break;
      const size_t by_lds = kLdsMax / lds_for(tpw), by_waves = 32 / (tpw * waves_per_tile);
      const size_t waves = (by_lds < by_waves ? by_lds : by_waves) * tpw * waves_per_tile;
      if (waves >= best) best = waves, tiles_per_wg = tpw;
    }
    a.x_phased = phased;
    if (best >= 16) break;
  }
  const size_t lds = lds_for(tiles_per_wg);
  if (lds > kLdsMax) return false;
  // Fewer than eight wavefronts on a compute unit cannot keep it fed: the general kernel does better then.
  if (best < 8) return false;
  a.tiles_per_wg = tiles_per_wg;
  a.x_vecs = a.K * esize / 16;
  a.x_row_vecs = row_bytes / 16;
  a.x_pitch = row_bytes + 16;
  const unsigned threads = tiles_per_wg * waves_per_tile * kWave, grid = (n_tiles + tiles_per_wg - 1) / tiles_per_wg;
  auto launch = [&](auto kernel) {
    if (lds > 48 * 1024) {
      static thread_local bool raised = false;
      if (!raised) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsMax) != hipSuccess)
          (void)hipGetLastError();
        raised = true;
      }
    }
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(threads), lds, stream, a);
    return status_of(hipGetLastError());
  };
  if (two_slices) {
    if constexpr (I8) *status = launch(tile16_kernel<F, MATH, false, 2>);
    else *status = a.xs.dtype == LX_F32 ? launch(tile16_kernel<F, MATH, true, 2>) : launch(tile16_kernel<F, MATH, false, 2>);
    return true;
  }
  if constexpr (I8) *status = launch(tile16_kernel<F, MATH, false, 1>);
  else *status = a.xs.dtype == LX_F32 ? launch(tile16_kernel<F, MATH, true, 1>) : launch(tile16_kernel<F, MATH, false, 1>);
  return true;
}

// ---- the INT8 math: int8 weights times per-token quantised activations, exact int32 sums ---------------
//
// The weights go into v_mfma_i32_16x16x64_i8 as they are stored (a lane's 16-byte chunk is one operand), so
// nothing is decoded; the sums are exact, so the K split needs no order. The epilogue is the reference's
// (engine/cpu/gemm.cpp:21-34): t = (rowscale * xscale) * f32(sum), + bias, * alpha, + beta * y.
// XL (MT == 1): the activation rows are staged in LDS (rows x_pitch bytes apart, zero from K to the end of the
// last weight batch), several tiles to a workgroup; otherwise the fragments are read from global memory.
template <int MATH, int MT, bool XL>
__global__ void __launch_bounds__(kMaxSplit* kWave) skinny_i8_kernel(const GemmArgs a) {
  constexpr int F = MATH == LX_MATH_INT8 ? LX_W_INT8 : LX_W_FP8;
  using Acc = typename std::conditional<MATH == LX_MATH_INT8, i32x4, f32x4>::type;
  extern __shared__ __align__(16) f32x4 lds4[];
  static_assert(!XL || MT == 1, "only one activation tile is staged in LDS");
  constexpr int kRegion = wave_region_bytes<1, MT>();
  const int lane = threadIdx.x & (kWave - 1), wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int S = a.S, tile_in_wg = XL ? wave / S : 0, slice = XL ? wave - tile_in_wg * S : wave;
  const int tile_raw = blockIdx.x * (XL ? a.tiles_per_wg : 1) + tile_in_wg;
  const int n_tiles = (a.N + kTileRows - 1) / kTileRows;
  const bool tile_live = tile_raw < n_tiles;
  const int n0 = min(tile_raw, n_tiles - 1) * kTileRows;
  const TileRows tiles[1] = {{a.w + n0 * a.row_bytes, a.scale, min(kTileRows, a.N - n0)}};
  uint8_t* const lds_bytes = reinterpret_cast<uint8_t*>(lds4);
  uint8_t* const tile_lds = lds_bytes + tile_in_wg * S * kRegion;
  int8_t* const ximg = reinterpret_cast<int8_t*>(lds_bytes + (blockDim.x / kWave) * kRegion);
  const int8_t* xrow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = min(mt * 16 + (lane & 15), a.M - 1);
    xrow[mt] = XL ? ximg + m * a.x_pitch : a.xq + static_cast<int64_t>(m) * a.K;
  }
  // The image's rows in 16-byte pieces: slots (row m, pass j) in row-major order, the first four asked for before
  // the weights.
  u32x4 xr[4];
  auto x_piece = [&](int m, int j) {
    const int v = min(static_cast<int>(threadIdx.x) + j * static_cast<int>(blockDim.x), a.x_vecs - 1);
    return *reinterpret_cast<const u32x4*>(a.xq + static_cast<int64_t>(min(m, a.M - 1)) * a.K + v * 16);
  };
  auto x_store = [&](int m, int j, u32x4 val) {
    const int v = threadIdx.x + j * blockDim.x;
    if (v >= a.x_vecs) val = u32x4{0u, 0u, 0u, 0u};
    if (v < a.x_row_vecs) *reinterpret_cast<u32x4*>(ximg + m * a.x_pitch + v * 16) = val;
  };
  if constexpr (XL) {
    int m = 0, j = 0;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      xr[u] = x_piece(m, j);
      if (++j == a.x_iters) j = 0, ++m;
    }
  }
  const TileStream<F, 1> ts(tiles, a.row_bytes, 0, a.chunks, tile_lds + slice * kRegion);
  WeightBatch<F, 1> wb;
  const int t_begin = min(a.steps, slice * a.steps_per_wave), t_end = min(a.steps, t_begin + a.steps_per_wave);
  if (t_begin < t_end) ts.issue(wb, t_begin);
  // The epilogue's factors: a lane always finishes the same four weight rows and, per tile, the same activation row.
  const bool bias_f32 = a.bias && a.bias_dtype == LX_F32;
  float rf[4], bs[4];
  {
    const int nq = n0 + 4 * (lane >> 4);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int n = min(nq + r, a.N - 1);
      rf[r] = reinterpret_cast<const float*>(a.scale)[n];
      bs[r] = bias_f32 ? static_cast<const float*>(a.bias)[n] : 0.0f;
    }
  }
  if constexpr (XL) {
    int m = 0, j = 0;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (m < a.M) x_store(m, j, xr[u]);
      if (++j == a.x_iters) j = 0, ++m;
    }
    while (m < a.M) {
      x_store(m, j, x_piece(m, j));
      if (++j == a.x_iters) j = 0, ++m;
    }
    __syncthreads();
  }
  Acc acc[1][MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[0][mt] = Acc{0, 0, 0, 0};
  const int k_end = min(a.K, 4 * t_end * 16);
  for (int tb = t_begin; tb < t_end; tb += kLoadsInFlight) {
    if (tb != t_begin) ts.issue(wb, tb);
    ts.template consume_bytes<MT, XL, MATH>(wb, tb, xrow, a.K, k_end, acc);
  }
  auto finish = [&](int mt, int q, const Acc& sum) {
    const int m = mt * 16 + (q & 15), nq = n0 + 4 * (q >> 4);  // q % 64 == lane: rf and bs are this slot's
    if (m < a.M && tile_live) {
      const float xs = a.xscale[m];
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (nq + r < a.N)
          write_out(a, m, nq + r, static_cast<float>(sum[r]), rf[r] * xs,
                    bias_f32 || !a.bias ? bs[r] : load_as_f32(a.bias, a.bias_dtype, nq + r));
    }
  };
  if (S == 1) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) finish(mt, lane, acc[0][mt]);
    return;
  }
  wave_lds_order();
  Acc* const mine = reinterpret_cast<Acc*>(tile_lds + slice * kRegion);
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) mine[mt * kWave + lane] = acc[0][mt];
  __syncthreads();
  for (int item = slice * kWave + lane; item < MT * kWave; item += S * kWave) {
    const int mt = item / kWave, q = item % kWave;
    Acc sum = reinterpret_cast<const Acc*>(tile_lds)[mt * kWave + q];
    for (int w = 1; w < S; ++w) sum += reinterpret_cast<const Acc*>(tile_lds + w * kRegion)[mt * kWave + q];
    finish(mt, q, sum);
  }
}

// Any alignment: one wavefront per output column, lanes striding over k; exact int32 sums (INT8) or f32 sums of the
// exact e4m3 products (FP8).
template <int MATH>
__global__ void __launch_bounds__(256) gemm_bytes_plain_kernel(const GemmArgs a) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t n = static_cast<int64_t>(blockIdx.x) * 4 + threadIdx.x / kWave;
  if (n >= a.N) return;
  const uint8_t* wrow = a.w + n * a.K;
  for (int m = 0; m < a.M; ++m) {
    const uint8_t* xrow = reinterpret_cast<const uint8_t*>(a.xq) + static_cast<int64_t>(m) * a.K;
    float sum;
    if constexpr (MATH == LX_MATH_INT8) {
      int acc = 0;
      for (int k = lane; k < a.K; k += kWave) acc += static_cast<int>(static_cast<int8_t>(xrow[k])) * static_cast<int>(static_cast<int8_t>(wrow[k]));
#pragma unroll
      for (int off = 1; off < kWave; off <<= 1) acc += __shfl_xor(acc, off);
      sum = static_cast<float>(acc);
    } else {
      float acc = 0.0f;
      for (int k = lane; k < a.K; k += kWave) acc = __builtin_fmaf(e4m3_byte_to_f32<0>(xrow[k]), e4m3_byte_to_f32<0>(wrow[k]), acc);
      sum = wave_sum(acc);
    }
    if (lane == 0)
      write_out(a, m, static_cast<int>(n), sum, reinterpret_cast<const float*>(a.scale)[n] * a.xscale[m],
                a.bias ? load_as_f32(a.bias, a.bias_dtype, n) : 0.0f);
  }
}

// Any shape and alignment: one wavefront per output column, lanes striding over k, activation rows eight at a
// time. x is rounded to bf16 first when `round_x` (the BF16 math on f32 activations).
__global__ void __launch_bounds__(256) gemm_plain_kernel(const GemmArgs a, int wtype, int round_x) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t n = static_cast<int64_t>(blockIdx.x) * 4 + threadIdx.x / kWave;
  if (n >= a.N) return;
  for (int m0 = 0; m0 < a.M; m0 += 8) {
    float acc[8];
#pragma unroll
    for (int m = 0; m < 8; ++m) acc[m] = 0.0f;
    for (int k = lane; k < a.K; k += kWave) {
      const float w = weight_element(wtype, a.w, a.scale, n, k, a.K);
#pragma unroll
      for (int m = 0; m < 8; ++m) {
        if (m0 + m < a.M) {
          float xv = load_as_f32(a.xs.x, a.xs.dtype, (m0 + m) * a.xs.ld + k);
          if (round_x) xv = bf16_bits_to_f32(f32_to_bf16_bits(xv));
          acc[m] = __builtin_fmaf(xv, w, acc[m]);
        }
      }
    }
#pragma unroll
    for (int m = 0; m < 8; ++m) {
      const float s = wave_sum(acc[m]);
      if (lane == 0 && m0 + m < a.M) write_out(a, wtype, m0 + m, static_cast<int>(n), s);
    }
  }
}

template <int F, int MT, bool XF32, bool XL, int LEAN = 0>
int launch_skinny_x(const GemmArgs& a, size_t lds, unsigned grid, unsigned threads, hipStream_t stream) {
  auto kernel = skinny_kernel<F, MT, XF32, XL, LEAN>;
  if (lds > 48 * 1024) {
    static thread_local bool raised = false;
    if (!raised) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsMax) != hipSuccess)
        (void)hipGetLastError();
      raised = true;
    }
  }
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(threads), lds, stream, a);
  return status_of(hipGetLastError());
}

// The walk kernel (gemm_walk.h) where it is the faster family. Measured on MI355X (bf16 activations, 9 .. 64 rows): it
// wins where a wavefront's walk is at most 16 groups of four load steps (K = 4096 of one-byte weights) and the matrix
// has the tiles to give most compute units a workgroup: 14336 x 4096 int8 at 16 / 32 / 64 rows 16.0 / 20.7 / 29.9 ->
// 15.2 / 18.1 / 25.4 us, 16384 x 4096 fp8 at 32 rows 21.5 -> 17.5 us, 6144 x 4096 14.2 -> 12.7 us, 4096 x 4096
// 13.6 -> 12.7 us; on 4096 x 8192 (32 groups) and at 8 rows and fewer the tile kernels are faster. The variant table
// ("gemm_w_<format>": 0 = the tile kernels by their own rule, 1 .. 3 = walk with 1, 2, 4 tiles a workgroup, 4 / 5 = the
// tile kernels without / with the slab kernel) overrides; no variant changes a sum.
template <int F>
bool try_walk(const GemmArgs& a, int* status, hipStream_t stream) {
  if (a.xs.dtype != LX_BF16) return false;
  const int n_tiles = (a.N + kTileRows - 1) / kTileRows;
  const int tuned = tuned_variant(gemm_key<F>(), a.M, a.N, a.K);
  int W;
  if (tuned == 0 || tuned >= kVariantWindow) return false;
  if (tuned >= 1 && tuned <= 3) {
    W = 1 << (tuned - 1);
  } else {
    // From sweeps of every variant (16 / 32 / 48 / 64 rows): a walk of at most 16 groups wins from 9 rows on; longer walks
    // (bf16, K >= 8192) win once the batch is large, where the tile kernels' activation reads grow with every row tile:
    // 8192 x 8192 fp8 at 32 / 64 rows 28.4 -> 24.6 / 50.4 -> 39.4 us, bf16 40.6 -> 36.7 / 58.8 -> 43.4 us, 14336 x 4096 bf16
    // at 64 rows 39.3 -> 35.3 us, 14336 x 8192 fp8 at 48 rows 47.5 -> 41.6 us. Few tiles (4096 rows) stay with the tile kernels.
    const int walk_groups = (a.steps + 3) >> 2;
    if (a.M <= 8 || n_tiles < 192) return false;
    if (walk_groups > 16) {
      if (n_tiles < 512 || walk_groups > 64) return false;
      // Many tiles: the windowed kernel holds on to 40 rows, except on the longest walks of the one-byte formats
      // (14336 x 14336 fp8 at 16 / 32 rows: 46.0 / 58.8 -> 41.0 / 51.3 us) and on NVFP4, whose values are twice as many
      // per byte (16384 x 14336 at 16 rows 55.5 -> 41.1 us, 14336 x 8192 at 48 rows 49.6 -> 41.2).
      const bool long_walks = n_tiles >= 768 && (F == LX_W_NVFP4 || (F != LX_W_BF16 && walk_groups > 32));
      // Below 768 tiles from 25 rows; the one-byte formats and NVFP4 from 17 rows on walks of more than 32 groups or fewer than
      // 576 tiles (at 17 .. 24 rows fp8 8192 x 14336 38.7 -> 32.4 us, 9216 x 11008 39.6 -> 31.3, 8192 x 8192 24.4 -> 21.2; with 32
      // groups on 576 .. 688 tiles the windowed kernel stays 4 - 7 % ahead).
      const int walk_from = n_tiles >= 768 ? 32 + 8 : F != LX_W_BF16 && (walk_groups > 32 || n_tiles < 576) ? 16 : 24;
      if (!long_walks && a.M <= walk_from) return false;
    }
    // (Rows that are not whole walks start every workgroup at the row's start, and four tiles a workgroup are ahead from
    // 576 tiles: at 32 rows fp8 9216 x 11008 40.2 -> 32.6 us, 11008 x 11008 41.1 -> 34.4, 11008 x 13824 49.9 -> 40.2; on the
    // 512 tiles of 8192 x 11008 two are: 28.1 against 31.9.)
    const bool whole_walks = a.steps % 16 == 0 && static_cast<int64_t>(a.steps) * 4 * Fmt<F>::kElems == a.K;
    W = n_tiles >= (walk_groups <= 16 ? 512 : whole_walks ? 768 : 576) ? 4 : 2;
  }
  auto launch = [&](int w) {
    if constexpr (F == LX_W_BF16) return launch_walk_bf16(a, w, status, stream);
    else if constexpr (F == LX_W_INT8) return launch_walk_int8(a, w, status, stream);
    else if constexpr (F == LX_W_FP8) return launch_walk_fp8(a, w, status, stream);
    else return launch_walk_nvfp4(a, w, status, stream);
  };
  if (launch(W)) return true;
  // The rule's two tiles a workgroup can be too many staging registers a lane (NVFP4 from 33 rows): four tiles then.
  return tuned < 0 && W == 2 && launch(4);
}

// The walk kernel for a matrix of few tiles and long rows: a workgroup of eight tiles (four where eight do not divide the
// window's pieces or do not fit LDS) walks one slice (two where a slice's groups are not fours), the slices' sums go
// through the stream's partial-tile buffer, and the slab kernel's second half adds them and runs the epilogue. False
// when it does not apply (one slice, ragged slices, a stream without the buffer).
template <int F>
bool launch_walk_parts(GemmArgs a, int* status, hipStream_t stream) {
  if (a.xs.dtype != LX_BF16) return false;
  const int spw = a.steps_per_wave;
  if (spw < 8 || spw % 8 != 0) return false;
  const int slices = (a.steps + spw - 1) / spw, gps = spw >> 2;
  if (slices < 2 || slices > a.S) return false;
  // A walk is groups in fours: two slices to a workgroup where one is not (the launcher then wants whole slices in pairs,
  // or rows for its kernels that fill a walk up).
  const int per_wg = gps % 4 == 0 ? 1 : 2;
  const int n_tiles = (a.N + kTileRows - 1) / kTileRows, mts = (a.M + 15) / 16;
  void* const partial = slab_scratch(stream, sizeof(float) * 4 * kWave * mts * n_tiles * slices);
  if (!partial) return false;
  a.partial = partial;
  a.walk_slices = per_wg;
  auto launch = [&](int w, int* st) {
    if constexpr (F == LX_W_BF16) return launch_walk_bf16(a, w, st, stream);
    else if constexpr (F == LX_W_INT8) return launch_walk_int8(a, w, st, stream);
    else if constexpr (F == LX_W_FP8) return launch_walk_fp8(a, w, st, stream);
    else return launch_walk_nvfp4(a, w, st, stream);
  };
  int st = kOk;
  // Eight tiles a workgroup from 17 rows; up to 16 rows four, which make twice the workgroups (at 16 rows NVFP4 4096 x 8192
  // 16.5 -> 12.3 us, 5120 x 5120 16.2 -> 11.9, 4096 x 14336 17.5 -> 15.9; fp8 4096 x 28672 31.6 -> 24.2, 4096 x 14336 16.9 -> 16.4;
  // at 32 and 64 rows eight are ahead by 5 - 20 %).
  if (mts == 1 ? (!launch(4, &st) && !launch(8, &st)) : (!launch(8, &st) && !launch(4, &st))) return false;
  if (!st) {
    a.S = slices;  // the reducer adds the slices that were written
    const int64_t items = static_cast<int64_t>(n_tiles) * mts * kWave;
    hipLaunchKernelGGL((slab_reduce_kernel<F, LX_MATH_BF16>), dim3(static_cast<unsigned>((items + 255) / 256)), dim3(256), 0, stream, a, mts);
    st = status_of(hipGetLastError());
  }
  *status = st;
  return true;
}

// The walk kernel with a tile's slices split over the four (or two) wavefronts of a workgroup; false when it does not
// apply (slices that do not divide, a short last slice, windows that do not fit).
template <int F>
bool launch_walk_split(GemmArgs a, int* status, hipStream_t stream) {
  if (a.xs.dtype != LX_BF16) return false;
  const int spw = a.steps_per_wave;
  if (spw < 8 || spw % 8 != 0 || a.steps % spw != 0) return false;
  const int slices = a.steps / spw;
  auto launch = [&](int w, int* st) {
    a.walk_split = w;
    a.walk_slices = (slices + w - 1) / w;  // the last wavefront takes what is left
    if constexpr (F == LX_W_BF16) return launch_walk_bf16(a, w, st, stream);
    else if constexpr (F == LX_W_INT8) return launch_walk_int8(a, w, st, stream);
    else if constexpr (F == LX_W_FP8) return launch_walk_fp8(a, w, st, stream);
    else return launch_walk_nvfp4(a, w, st, stream);
  };
  return launch(4, status) || launch(2, status);
}

// Where a tile's slices are split over a workgroup's wavefronts without a table entry: a tile per compute unit at most
// (the windows of four wavefronts fill a unit's LDS, so a second workgroup waits for the first: 5120 x 4096 fp8 at 16 / 32
// rows 9.6 / 12.1 -> 12.3 / 18.1 us) and up to 32 rows of short K, where the whole walk is a few wavefronts' long chains:
// 4096 x 4096 at 16 / 32 rows fp8 9.3 / 12.1 -> 7.3 / 10.2 us, int8 11.4 / 14.2 -> 7.7 / 10.6, bf16 10.6 / 14.4 -> 9.0 / 11.7,
// nvfp4 at 16 rows 12.6 -> 9.6; 2048 x 4096 fp8 8.3 / 11.7 -> 6.5 / 9.7; 4096 x 8192 fp8 at 16 rows 13.3 -> 11.2 (at 32 rows
// the single-slice walks and the slab kernel do better there, as they do on long rows: 4096 x 14336 fp8 at 16 / 32 rows 16.8 /
// 24.2 us split against 16.9 / 19.0). Two wavefronts a tile, whose windows leave room for two
// workgroups a unit, do not carry it to 257 .. 512 tiles (6144 x 4096 fp8 at 32 rows 12.2 -> 15.0 us).
inline bool walk_split_wanted(int M, int n_tiles, int64_t K, int tuned) {
  if (tuned >= 0) return tuned == kVariantWalkSplit;
  return M > 8 && M <= 32 && n_tiles <= compute_units() && (K <= 4096 || (M <= 16 && K <= 8192));
}

// Where the single-slice walks are taken without a table entry. From sweeps of every variant over 2048 .. 8192 rows of
// 4096 .. 28672 values at 16 / 32 / 64 activation rows: they win where the activations weigh most against the weights
// (many rows, long K; NVFP4 earlier, whose values are half a byte), by up to 2 x (4096 x 14336 fp8 at 64 rows
// 44.9 -> 28.0 us, 8192 x 28672 112 -> 66 us; nvfp4 4096 x 28672 at 32 rows 75 -> 41 us), and lose 5 .. 30 % on short rows.
template <int F>
bool walk_parts_wanted(int M, int n_tiles, int64_t K, int tuned) {
  if (tuned >= 0) return tuned == kVariantWalkParts;
  if (M <= 8) return false;
  const int mts = (M + 15) / 16;
  if (F == LX_W_NVFP4) {
    // With many tiles the whole walk of four tiles a workgroup is ahead at every row count (14336 x 4096 at 48 rows
    // 32.8 -> 25.5 us); below that the single slices from 33 rows, from 17 rows for K >= 8192, from 9 for K >= 14336
    // (8192 x 14336 at 16 rows 38.0 -> 29.5 us); K >= 11008 since the walks take rows that are not whole walks (at 16 rows
    // 9216 x 11008 39.7 -> 30 us, 11008 x 11008 40.5 -> 32, 5120 x 13824 33.4 -> 27; a tie on 4096 and 8192 x 11008).
    // With four tiles a workgroup up to 16 rows they are also ahead there on 257 .. 512 tiles from K = 5120 (at 16 rows
    // 5120 x 5120 16.4 -> 11.9 us, 6144 x 7168 20.4 -> 15.8, 8192 x 8192 21.6 -> 17.7; at 24 / 32 rows 6144 x 7168 25.3 -> 21; on 576
    // tiles and more the whole walk is).
    if (n_tiles >= 768) return false;
    return mts >= 3 || (mts == 2 && K >= 8192) || K >= 11008 || (K >= 5120 && n_tiles > 256 && n_tiles <= 512);
  }
  // Rows of 5120 .. 7168 values (bf16 from 6144) on at most 384 tiles, where neither the whole walks nor the tile kernels
  // fill the device: 5120 x 5120 fp8 at 32 / 48 / 64 rows 19.2 / 23.8 / 27.1 -> 13 / 15 / 17 us, 6144 x 7168 23.3 / 32.6 / 39.0
  // -> 17.5 / 20 / 23, 4096 x 6144 at 48 / 64 rows 20.3 / 23.3 -> 15 / 16.5, bf16 6144 x 6144 24.0 / 29.6 / 33.0 -> 21 / 26 / 27
  // (at worst a tie: 6144 x 5120, and 6144 x 6144 one-byte at 32 rows 5 % behind); at 17 .. 32 rows 4096-row matrices
  // stay with the split walk and the slab kernel, which tie.
  const int64_t mid_k = F == LX_W_BF16 ? 6144 : 5120;
  if (mts >= 3) return K >= 8192 || (K >= mid_k && n_tiles <= 384);
  if (K >= 28672 || (K >= 14336 && n_tiles <= 256)) return true;
  // (Up to 16 rows of one-byte weights also K >= 13824 on at most 512 tiles: 8192 x 14336 fp8 27.6 -> 24.5 us, 5120 x 13824 25.1 -> 20.7.)
  if (mts == 1 && F != LX_W_BF16 && K >= 13824 && n_tiles <= 512) return true;
  return K >= mid_k && K < 8192 && n_tiles > 256 && n_tiles <= 384;
}

template <int F, int MT>
int launch_skinny(GemmArgs a, hipStream_t stream) {
  const int S = a.S;
  const unsigned n_tiles = static_cast<unsigned>((a.N + kTileRows - 1) / kTileRows);
  {
    int st = kOk;
    if (walk_parts_wanted<F>(a.M, static_cast<int>(n_tiles), a.K, tuned_variant(gemm_key<F>(), a.M, a.N, a.K)) && launch_walk_parts<F>(a, &st, stream)) return st;
    if (walk_split_wanted(a.M, static_cast<int>(n_tiles), a.K, tuned_variant(gemm_key<F>(), a.M, a.N, a.K)) && launch_walk_split<F>(a, &st, stream)) return st;
    if (try_walk<F>(a, &st, stream)) return st;
  }
  // More than eight rows: the windowed kernel (for 9 .. 16 rows where the matrix has the tiles to fill its
  // sixteen-wavefront workgroups; the lean kernel's image of all of K leaves too few of them resident there).
  const int tuned = tuned_variant(gemm_key<F>(), a.M, a.N, a.K);
  if (MT > 1 || (a.M > 8 && n_tiles >= 320) || tuned == kVariantWindow || tuned == kVariantSlab) {
    int st = kOk;
    if (slab_wanted(a.M, static_cast<int>(n_tiles), a.K, tuned) && launch_slab<F, LX_MATH_BF16>(a, &st, stream)) return st;
    if (launch_window<F, LX_MATH_BF16>(a, &st, stream)) return st;
  }
  if constexpr (MT == 1) {
    int st = kOk;
    if (launch_tile16<F, LX_MATH_BF16>(a, &st, stream)) return st;
    // The activation image: rows as long as the last weight batch reaches, zero past K.
    constexpr int kBatchElems = (kLoadsInFlight / 1) * 4 * Fmt<F>::kElems;
    const int row_elems = (a.K + kBatchElems - 1) / kBatchElems * kBatchElems;
    const size_t image = static_cast<size_t>(a.M) * (row_elems + 8) * 2;
    // Two tiles to a workgroup when they fit: twice the wavefronts behind one image.
    int tiles_per_wg = 2 * S <= kMaxSplit && n_tiles >= 512 ? 2 : 1;
    if (tile_lds_bytes(tiles_per_wg * S, 1, 1) + image > kLdsMax) tiles_per_wg = 1;
    const size_t lds = tile_lds_bytes(tiles_per_wg * S, 1, 1) + image;
    if (lds <= kLdsMax) {
      const unsigned threads = tiles_per_wg * S * kWave;
      a.tiles_per_wg = tiles_per_wg;
      a.x_vecs = a.K / 8;
      a.x_row_vecs = row_elems / 8;
      a.x_pitch = row_elems + 8;
      a.x_iters = (a.x_row_vecs + threads - 1) / threads;
      const unsigned grid = (n_tiles + tiles_per_wg - 1) / tiles_per_wg;
      return a.xs.dtype == LX_F32 ? launch_skinny_x<F, 1, true, true>(a, lds, grid, threads, stream)
                                  : launch_skinny_x<F, 1, false, true>(a, lds, grid, threads, stream);
    }
  }
  // No kernel with an activation image takes the call (rows too long for the image of the rows' count): the walks of
  // single slices, whose windows fit whatever K is, before the kernel that reads its activations where they lie (NVFP4
  // 4096 x 14336 at 1 / 8 rows in the batch-invariant mode 17.8 / 19.6 -> 16.5 / 16.7 us, 8192 x 14336 40.5 / 35.7 -> 24.0 / 24.2).
  if (tuned < 0) {
    int st = kOk;
    if (launch_walk_parts<F>(a, &st, stream)) return st;
  }
  const size_t lds = tile_lds_bytes(S, 1, MT);
  if constexpr (F == LX_W_NVFP4) {
    if (S <= 8 && wide_scales_fit(a.scale, a.scale_row_bytes, a.chunks)) {
      if (S <= 4)
        return a.xs.dtype == LX_F32 ? launch_skinny_x<F, MT, true, false, 4>(a, lds, n_tiles, S * kWave, stream)
                                    : launch_skinny_x<F, MT, false, false, 4>(a, lds, n_tiles, S * kWave, stream);
      return a.xs.dtype == LX_F32 ? launch_skinny_x<F, MT, true, false, 8>(a, lds, n_tiles, S * kWave, stream)
                                  : launch_skinny_x<F, MT, false, false, 8>(a, lds, n_tiles, S * kWave, stream);
    }
  }
  return a.xs.dtype == LX_F32 ? launch_skinny_x<F, MT, true, false>(a, lds, n_tiles, S * kWave, stream)
                              : launch_skinny_x<F, MT, false, false>(a, lds, n_tiles, S * kWave, stream);
}

template <int F>
int launch_format(GemmArgs a, const char* x0, char* y0, int M, int x_esize, int y_esize, hipStream_t stream) {
  const int64_t rb = row_bytes<F>(a.K);
  const bool aligned = rb % 16 == 0 && reinterpret_cast<uintptr_t>(a.w) % 16 == 0 &&
                       (F != LX_W_NVFP4 || reinterpret_cast<uintptr_t>(a.scale) % 2 == 0) &&
                       reinterpret_cast<uintptr_t>(x0) % 16 == 0 && (a.xs.ld * x_esize) % 16 == 0 && a.K % 8 == 0;
  if (!aligned) {
    a.M = M;
    hipLaunchKernelGGL(gemm_plain_kernel, dim3(static_cast<unsigned>((a.N + 3) / 4)), dim3(256), 0, stream, a, F,
                       a.xs.dtype == LX_F32 ? 1 : 0);
    return status_of(hipGetLastError());
  }
  a.row_bytes = rb;
  a.scale_row_bytes = F == LX_W_NVFP4 ? a.K / 16 : 0;
  a.chunks = static_cast<int>(rb / 16);
  a.steps = load_steps_for<F>(a.K);
  int S = split_for_shape<F>(a.K, a.N);
  // Slices are whole weight batches (the row's last one may be cut short by the row's end).
  a.steps_per_wave = ((a.steps + S - 1) / S + kLoadsInFlight - 1) / kLoadsInFlight * kLoadsInFlight;
  a.S = S;
  const float* const act_scale0 = a.act_scale;
  // Up to 64 activation rows a pass; every pass is the same arithmetic per row.
  for (int m0 = 0; m0 < M; m0 += 64) {
    a.M = M - m0 < 64 ? M - m0 : 64;
    a.xs.x = x0 + static_cast<int64_t>(m0) * a.xs.ld * x_esize;
    a.y = y0 + static_cast<int64_t>(m0) * a.ld_y * y_esize;
    if (act_scale0) a.act_scale = act_scale0 + m0;
    int st;
    switch ((a.M + 15) / 16) {
      case 1: st = launch_skinny<F, 1>(a, stream); break;
      case 2: st = launch_skinny<F, 2>(a, stream); break;
      case 3: st = launch_skinny<F, 3>(a, stream); break;
      default: st = launch_skinny<F, 4>(a, stream); break;
    }
    if (st) return st;
  }
  return kOk;
}

bool valid_dtype(int d) { return d == LX_F32 || d == LX_BF16; }

bool valid_weight(const lx_weight* w, int64_t K) {
  if (!w || !w->data) return false;
  switch (w->type) {
    case LX_W_BF16: return true;
    case LX_W_INT8:
    case LX_W_FP8: return w->scale != nullptr;
    case LX_W_NVFP4: return w->scale != nullptr && K % 16 == 0;
    default: return false;
  }
}

}  // namespace

// The matrix-core product of any format: BF16 math (x rounded to bf16), any M. Validation follows
// engine/cpu/gemm.cpp:189-197.
int gemm_bf16_scaled(const void* x, int x_dtype, int64_t ld_x, const lx_weight& w, const void* bias, int bias_dtype, void* y,
                     int y_dtype, int64_t ld_y, int M, int N, int K, float alpha, float beta, const float* act_scale, void* stream);

int gemm_bf16_math(const void* x, int x_dtype, int64_t ld_x, const lx_weight& w, const void* bias, int bias_dtype, void* y,
                   int y_dtype, int64_t ld_y, int M, int N, int K, float alpha, float beta, void* stream) {
  return gemm_bf16_scaled(x, x_dtype, ld_x, w, bias, bias_dtype, y, y_dtype, ld_y, M, N, K, alpha, beta, nullptr, stream);
}

// act_scale (or null): one factor per activation row, multiplied into the row factor in the epilogue: the rows are a
// quantised math's activation images (act_images) and these their scales.
int gemm_bf16_scaled(const void* x, int x_dtype, int64_t ld_x, const lx_weight& w, const void* bias, int bias_dtype, void* y,
                     int y_dtype, int64_t ld_y, int M, int N, int K, float alpha, float beta, const float* act_scale, void* stream) {
  if (M == 0 || N == 0) return kOk;
  if (M < 0 || N < 0 || K <= 0 || ld_x < K || ld_y < N) return fail(kInvalid);
  if (!valid_dtype(x_dtype) || !valid_dtype(y_dtype) || (bias && !valid_dtype(bias_dtype))) return fail(kInvalid);
  if (w.type == LX_W_BF16X) return fail(kNotSupported);
  if (!x || !y || !valid_weight(&w, K)) return fail(kInvalid);
  GemmArgs a{};
  a.xs = XRows{x, x_dtype, ld_x};
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
  a.act_scale = act_scale;
  const int xe = x_dtype == LX_BF16 ? 2 : 4, ye = y_dtype == LX_BF16 ? 2 : 4;
  hipStream_t s = as_stream(stream);
  switch (w.type) {
    case LX_W_BF16: return launch_format<LX_W_BF16>(a, static_cast<const char*>(x), static_cast<char*>(y), M, xe, ye, s);
    case LX_W_INT8: return launch_format<LX_W_INT8>(a, static_cast<const char*>(x), static_cast<char*>(y), M, xe, ye, s);
    case LX_W_FP8: return launch_format<LX_W_FP8>(a, static_cast<const char*>(x), static_cast<char*>(y), M, xe, ye, s);
    default: return launch_format<LX_W_NVFP4>(a, static_cast<const char*>(x), static_cast<char*>(y), M, xe, ye, s);
  }
}

// The INT8 and FP8 maths of lx_gemm_w (engine/cpu/gemm.cpp:203-209,231-288) on weights of the math's own type (int8,
// fp8; NVFP4 weights under the FP8 math answer 801 here): the activations are quantised per token into the
// workspace (scales first, rows 64 bytes further, as the reference lays it out). INT8 sums are exact; FP8 products
// are exact and summed in f32 (the reference sums them in double: equal to f32 rounding of the sums).
template <int MATH>
int gemm_bytes_math(const void* x, int x_dtype, int64_t ld_x, const lx_weight& w, const void* bias, int bias_dtype, void* y,
                    int y_dtype, int64_t ld_y, int M, int N, int K, float alpha, float beta, void* workspace, void* stream) {
  constexpr int F = MATH == LX_MATH_INT8 ? LX_W_INT8 : LX_W_FP8;
  if (M == 0 || N == 0) return kOk;
  if (M < 0 || N < 0 || K <= 0 || ld_x < K || ld_y < N) return fail(kInvalid);
  if (!valid_dtype(x_dtype) || !valid_dtype(y_dtype) || (bias && !valid_dtype(bias_dtype))) return fail(kInvalid);
  if (w.type == LX_W_BF16X) return fail(kNotSupported);
  if (!x || !y || !valid_weight(&w, K)) return fail(kInvalid);
  if (w.type != F) return fail(kNotSupported);
  hipStream_t s = as_stream(stream);
  const size_t ws_bytes = static_cast<size_t>((static_cast<int64_t>(M) * 4 + 63) / 64 * 64 + static_cast<int64_t>(M) * K);
  void* own = nullptr;
  if (!workspace) {  // the reference falls back to scratch of its own
    if (hipMallocAsync(&own, ws_bytes, s) != hipSuccess) return fail(kNoMemory);
    workspace = own;
  }
  float* const scales = static_cast<float*>(workspace);
  int8_t* const q = static_cast<int8_t*>(workspace) + (static_cast<int64_t>(M) * 4 + 63) / 64 * 64;
  int st = quantize_act_rows(x, x_dtype, ld_x, MATH, q, K, scales, nullptr, 0, M, K, s);
  GemmArgs a{};
  a.w = static_cast<const uint8_t*>(w.data);
  a.scale = static_cast<const uint8_t*>(w.scale);
  a.global = 1.0f;
  a.bias = bias;
  a.bias_dtype = bias_dtype;
  a.y_dtype = y_dtype;
  a.ld_y = ld_y;
  a.N = N;
  a.K = K;
  a.alpha = alpha;
  a.beta = beta;
  a.row_bytes = K;
  const bool aligned = K % 16 == 0 && reinterpret_cast<uintptr_t>(a.w) % 16 == 0 && reinterpret_cast<uintptr_t>(q) % 16 == 0;
  const int ye = y_dtype == LX_BF16 ? 2 : 4;
  if (!st && !aligned) {
    a.M = M;
    a.xq = q;
    a.xscale = scales;
    a.y = y;
    hipLaunchKernelGGL(gemm_bytes_plain_kernel<MATH>, dim3(static_cast<unsigned>((N + 3) / 4)), dim3(256), 0, s, a);
    st = status_of(hipGetLastError());
  } else if (!st) {
    a.chunks = K / 16;
    a.steps = load_steps_for<F>(K);
    const int S = split_for_shape<F>(K, N);
    a.S = S;
    a.steps_per_wave = ((a.steps + S - 1) / S + kLoadsInFlight - 1) / kLoadsInFlight * kLoadsInFlight;
    const unsigned n_tiles = static_cast<unsigned>((N + kTileRows - 1) / kTileRows);
    for (int m0 = 0; m0 < M && !st; m0 += 64) {
      a.M = M - m0 < 64 ? M - m0 : 64;
      a.xq = q + static_cast<int64_t>(m0) * K;
      a.xscale = scales + m0;
      a.y = static_cast<char*>(y) + static_cast<int64_t>(m0) * ld_y * ye;
      auto launch = [&](auto kernel, size_t lds, unsigned grid, unsigned threads) {
        if (lds > 48 * 1024) {
          static thread_local bool raised = false;
          if (!raised) {
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsMax) != hipSuccess)
              (void)hipGetLastError();
            raised = true;
          }
        }
        hipLaunchKernelGGL(kernel, dim3(grid), dim3(threads), lds, s, a);
        return status_of(hipGetLastError());
      };
      const int mt = (a.M + 15) / 16;
      if ((mt > 1 || (a.M > 8 && n_tiles >= 320)) && slab_wanted(a.M, static_cast<int>(n_tiles), K, tuned_variant(gemm_key<F>(), a.M, N, K)) && launch_slab<F, MATH>(a, &st, s)) continue;
      if ((mt > 1 || (a.M > 8 && n_tiles >= 320)) && launch_window<F, MATH>(a, &st, s)) continue;
      if (mt == 1 && launch_tile16<F, MATH>(a, &st, s)) continue;
      if (mt == 1) {
        // The activation image: rows as long as the last weight batch reaches, zero past K.
        constexpr int kBatchBytes = kLoadsInFlight * 4 * 16;
        const int row_bytes = (K + kBatchBytes - 1) / kBatchBytes * kBatchBytes;
        const size_t image = static_cast<size_t>(a.M) * (row_bytes + 16);
        int tiles_per_wg = 2 * S <= kMaxSplit && n_tiles >= 512 ? 2 : 1;
        if (tile_lds_bytes(tiles_per_wg * S, 1, 1) + image > kLdsMax) tiles_per_wg = 1;
        const size_t lds = tile_lds_bytes(tiles_per_wg * S, 1, 1) + image;
        if (lds <= kLdsMax) {
          const unsigned threads = tiles_per_wg * S * kWave;
          a.tiles_per_wg = tiles_per_wg;
          a.x_vecs = K / 16;
          a.x_row_vecs = row_bytes / 16;
          a.x_pitch = row_bytes + 16;
          a.x_iters = (a.x_row_vecs + threads - 1) / threads;
          st = launch(skinny_i8_kernel<MATH, 1, true>, lds, (n_tiles + tiles_per_wg - 1) / tiles_per_wg, threads);
          continue;
        }
      }
      const unsigned threads = S * kWave;
      switch (mt) {
        case 1: st = launch(skinny_i8_kernel<MATH, 1, false>, tile_lds_bytes(S, 1, 1), n_tiles, threads); break;
        case 2: st = launch(skinny_i8_kernel<MATH, 2, false>, tile_lds_bytes(S, 1, 2), n_tiles, threads); break;
        case 3: st = launch(skinny_i8_kernel<MATH, 3, false>, tile_lds_bytes(S, 1, 3), n_tiles, threads); break;
        default: st = launch(skinny_i8_kernel<MATH, 4, false>, tile_lds_bytes(S, 1, 4), n_tiles, threads); break;
      }
    }
  }
  if (own) (void)hipFreeAsync(own, s);
  return st;
}

// The FP8 math on NVFP4 weights and the FP4 math (engine/cpu/gemm.cpp:207-212,246-288): the activations are quantised
// per token by the math's rule, their exact values go back into bf16 rows (an e4m3 value, or an e2m1 code times its e4m3
// block scale, fits bf16), and the BF16-math kernels multiply those rows by the exactly expanded weights (exact products,
// f32 sums; the reference sums them in double) with the rows' scales in the epilogue: t = (rowfactor * xscale) * sum.
// Workspace as the reference lays it out: the scales first, the rows 64 bytes further (here: the bf16 images, then the
// quantiser's bytes).
int gemm_image_math(int math, const void* x, int x_dtype, int64_t ld_x, const lx_weight& w, const void* bias, int bias_dtype, void* y,
                    int y_dtype, int64_t ld_y, int M, int N, int K, float alpha, float beta, void* workspace, void* stream) {
  if (M == 0 || N == 0) return kOk;
  if (M < 0 || N < 0 || K <= 0 || ld_x < K || ld_y < N) return fail(kInvalid);
  if (!valid_dtype(x_dtype) || !valid_dtype(y_dtype) || (bias && !valid_dtype(bias_dtype))) return fail(kInvalid);
  if (w.type == LX_W_BF16X) return fail(kNotSupported);
  if (!x || !y || !valid_weight(&w, K)) return fail(kInvalid);
  if (math == LX_MATH_FP8 && w.type != LX_W_FP8 && w.type != LX_W_NVFP4) return fail(kNotSupported);
  if (math == LX_MATH_FP4 && (w.type != LX_W_NVFP4 || K % 16 != 0)) return fail(kNotSupported);
  hipStream_t s = as_stream(stream);
  const int64_t head = (static_cast<int64_t>(M) * 4 + 63) / 64 * 64;
  void* own = nullptr;
  if (!workspace) {  // the reference falls back to scratch of its own
    if (hipMallocAsync(&own, static_cast<size_t>(head + static_cast<int64_t>(M) * K * 4), s) != hipSuccess) return fail(kNoMemory);
    workspace = own;
  }
  float* const scales = static_cast<float*>(workspace);
  uint16_t* const xhat = reinterpret_cast<uint16_t*>(static_cast<char*>(workspace) + head);
  uint8_t* const q = reinterpret_cast<uint8_t*>(xhat + static_cast<int64_t>(M) * K);
  int st = act_images(x, x_dtype, ld_x, math, q, xhat, scales, M, K, s);
  if (!st) st = gemm_bf16_scaled(xhat, LX_BF16, K, w, bias, bias_dtype, y, y_dtype, ld_y, M, N, K, alpha, beta, scales, stream);
  if (own) (void)hipFreeAsync(own, s);
  return st;
}

// The stream's buffer for the slab kernel's partial tiles (runtime.hip makes one with every stream it creates).
int slab_reserve(hipStream_t stream) {
  int dev = 0;
  if (int e = status_of(hipGetDevice(&dev))) return e;
  SlabBuffers& b = slab_buffers();
  std::lock_guard<std::mutex> g(b.lock);
  void*& slot = b.of[{dev, stream}];
  if (slot) return kOk;
  if (hipMalloc(&slot, kSlabScratchBytes) != hipSuccess) {
    (void)hipGetLastError();
    b.of.erase({dev, stream});
    return fail(kNoMemory);
  }
  return kOk;
}

int slab_release(hipStream_t stream) {
  int dev = 0;
  if (int e = status_of(hipGetDevice(&dev))) return e;
  void* buffer = nullptr;
  {
    SlabBuffers& b = slab_buffers();
    std::lock_guard<std::mutex> g(b.lock);
    auto it = b.of.find({dev, stream});
    if (it == b.of.end()) return kOk;
    buffer = it->second;
    b.of.erase(it);
  }
  return status_of(hipFree(buffer));
}

}  // namespace dro

using namespace dro;

extern "C" {

int lx_gemv_w(const void* x, lx_dtype x_dtype, int ld_x, const lx_weight* w, const void* bias, lx_dtype bias_dtype, void* y,
              lx_dtype y_dtype, int ld_y, int M, int N, int K, float alpha, float beta, void* stream) {
  if (!w) return fail(kInvalid);
  // engine/cpu/gemm.cpp:356-357: lossless rows have their own entry point.
  if (w->type == LX_W_BF16X) return lx_gemv_bf16x(x, x_dtype, ld_x, w->data, bias, bias_dtype, y, y_dtype, ld_y, M, N, K, alpha, beta, stream);
  // Batch-invariant mode: bf16 activations take the matrix-core kernel, whose sums are the same for every row
  // count from 1 up (lx_gemm_w runs the same kernel). f32 activations keep the exact f32 product.
  if (batch_invariant() && x_dtype == LX_BF16 && M >= 1 && M <= 8 && N > 0)
    return gemm_bf16_math(x, x_dtype, ld_x, *w, bias, bias_dtype, y, y_dtype, ld_y, M, N, K, alpha, beta, stream);
  return gemv_any(x, x_dtype, ld_x, *w, bias, bias_dtype, y, y_dtype, ld_y, M, N, K, alpha, beta, stream);
}

int lx_gemm_w(const void* x, lx_dtype x_dtype, int ld_x, const lx_weight* w, lx_math math, const void* bias, lx_dtype bias_dtype,
              void* y, lx_dtype y_dtype, int ld_y, int M, int N, int K, float alpha, float beta, void* workspace, void* stream) {
  if (!w) return fail(kInvalid);
  if (math != LX_MATH_BF16 && math != LX_MATH_INT8 && math != LX_MATH_FP8 && math != LX_MATH_FP4) return fail(kInvalid);
  if (math == LX_MATH_INT8)
    return gemm_bytes_math<LX_MATH_INT8>(x, x_dtype, ld_x, *w, bias, bias_dtype, y, y_dtype, ld_y, M, N, K, alpha, beta, workspace, stream);
  if (math == LX_MATH_FP8 && w->type != LX_W_NVFP4)
    return gemm_bytes_math<LX_MATH_FP8>(x, x_dtype, ld_x, *w, bias, bias_dtype, y, y_dtype, ld_y, M, N, K, alpha, beta, workspace, stream);
  if (math != LX_MATH_BF16)
    return gemm_image_math(math, x, x_dtype, ld_x, *w, bias, bias_dtype, y, y_dtype, ld_y, M, N, K, alpha, beta, workspace, stream);
  return gemm_bf16_math(x, x_dtype, ld_x, *w, bias, bias_dtype, y, y_dtype, ld_y, M, N, K, alpha, beta, stream);
}

int64_t lx_gemm_workspace_bytes(int M, int K, lx_math math) {
  if (M <= 0 || K <= 0) return 0;
  const int64_t elem = math == LX_MATH_INT8 ? 1 : 4;
  const int64_t bytes = (static_cast<int64_t>(M) * 4 + 63) / 64 * 64 + static_cast<int64_t>(M) * K * elem;
  return (bytes + 255) / 256 * 256;
}

int lx_gemm_skinny(const void* x, lx_dtype x_dtype, int ld_x, const lx_weight* w, const void* bias, lx_dtype bias_dtype, void* y,
                   lx_dtype y_dtype, int ld_y, int M, int N, int K, float alpha, float beta, void* stream) {
  if (!w) return fail(kInvalid);
  if (x_dtype != LX_BF16 && M > 0 && N > 0) return fail(kNotSupported);  // bf16 activations only, as the reference
  return gemm_bf16_math(x, x_dtype, ld_x, *w, bias, bias_dtype, y, y_dtype, ld_y, M, N, K, alpha, beta, stream);
}

}  // extern "C"
