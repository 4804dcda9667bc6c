// The matrix-core product shared by the skinny GEMM and the grouped experts.
//
// One wavefront multiplies NT tiles of 16 weight rows by up to 64 activation rows (MT tiles of 16) over a slice
// of K with v_mfma_f32_16x16x32_bf16. The weights are the A operand, so a lane ends up holding four
// consecutive output columns n of one activation row m (D[i = 4 * (lane / 16) + r][j = lane % 16], i the
// weight row, j the activation row): a 16-byte store per lane.
//
// Weights are read as they lie, 16 bytes per lane per load, 256 contiguous bytes of a row per instruction, and
// handed through LDS to the lanes of the matrix instruction: lane (g = lane / 16, i = lane % 16) works on chunk
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

// The K split of a dense product of N rows: the split by K alone gives every wavefront one batch; with many tiles
// fewer, longer slices do better (measured on MI355X: about 2500 wavefronts in all, each walking its slice in
// batches). A function of (F, K, N) only, never of M, so a row's bits do not depend on the batch.
template <int F>
inline int split_for_shape(int64_t K, int64_t N) {
  const int by_k = split_for<F>(K, 1);
  const double want = 2560.0 / static_cast<double>((N + kTileRows - 1) / kTileRows);
  int S = 1;
  while (S < kMaxSplit && static_cast<double>(S) * 1.4142135623730951 <= want) S *= 2;  // nearest power of two, ties up
  // Eight slices where the rounding went up (321 .. 452 tiles) would be slices of one batch each for K = 4096: four
  // slices of two batches do better at every row count there (6144 x 4096 fp8: 8.9 -> 7.6 us at one row in the
  // batch-invariant mode, 11.4 -> 9.9 at 16, 15.1 -> 13.9 at 32; measured also at 5632 and 7168 rows, bf16 and int8).
  // NVFP4's steps are twice as long and keep the eight.
  if (S == 8 && static_cast<double>(S) > want && load_steps_for<F>(K) / S < 16 && F != LX_W_NVFP4) S = 4;
  // Two slices where the rounding went down from 2.4 or more (906 .. 1066 tiles) leave the device short of wavefronts: four
  // do better while a slice still holds two batches (16384 x 4096 fp8 at one / four rows in the batch-invariant mode
  // 15.5 / 16.0 -> 13.2 / 13.8 us, bf16 28.8 / 29.3 -> 22.9 / 23.2; 20480 rows and more are better off with two).
  if (S == 2 && want >= 2.4 && load_steps_for<F>(K) / 4 >= 16) S = 4;
  return S < by_k ? S : by_k;
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

// Where a wavefront's activation fragments come from (XS): rows of bf16 (kXGlobalBf16) or f32 (kXGlobalF32) in
// global memory whose addresses and strides are multiples of 16 bytes, or rows of bf16 staged in LDS (kXLds, the
// rows a multiple of 16 bytes apart). The caller resolves each lane's row pointers (one per activation tile,
// clamped into the matrix: the columns of a clamped row are computed and never written).
constexpr int kXGlobalBf16 = 0, kXGlobalF32 = 1, kXLds = 2;

template <int XS>
struct XFrag {
  u32x4 raw[XS == kXGlobalF32 ? 2 : 1];
};

// x[row, k .. k + 8) as loaded; in global memory k is clamped into the row (a fragment past K is zeroed when it
// is used); an LDS image covers every k that is asked for.
template <int XS>
__device__ __forceinline__ void load_x_fragment(XFrag<XS>& f, const void* row, int k, int K) {
  if constexpr (XS == kXGlobalF32) {
    const u32x4* p = reinterpret_cast<const u32x4*>(static_cast<const float*>(row) + min(k, K - 8));
    f.raw[0] = p[0];
    f.raw[1] = p[1];
  } else if constexpr (XS == kXGlobalBf16) {
    f.raw[0] = *reinterpret_cast<const u32x4*>(static_cast<const uint16_t*>(row) + min(k, K - 8));
  } else {
    f.raw[0] = *reinterpret_cast<const u32x4*>(static_cast<const uint16_t*>(row) + k);
  }
}

// The fragment as the B operand: bf16 as it is, f32 rounded to bf16 (nearest even); zero past K when MASK (an
// activation image that is itself zero past K needs none).
template <int XS, bool MASK>
__device__ __forceinline__ bf16x8 x_operand(const XFrag<XS>& f, int k, int K) {
  u32x4 v;
  if constexpr (XS == kXGlobalF32) {
    bf16x2 q[4] = {pack_bf16(__uint_as_float(f.raw[0].x), __uint_as_float(f.raw[0].y)),
                   pack_bf16(__uint_as_float(f.raw[0].z), __uint_as_float(f.raw[0].w)),
                   pack_bf16(__uint_as_float(f.raw[1].x), __uint_as_float(f.raw[1].y)),
                   pack_bf16(__uint_as_float(f.raw[1].z), __uint_as_float(f.raw[1].w))};
    v = __builtin_bit_cast(u32x4, q);
  } else {
    v = f.raw[0];
  }
  if constexpr (MASK)
    if (k >= K) v = u32x4{0u, 0u, 0u, 0u};
  return __builtin_bit_cast(bf16x8, v);
}

// Load steps whose activation fragments are held at once: from global memory, bounded by the registers they
// take (steps x instructions per step x activation tiles x 4 or 8 registers), at most kLoadsInFlight / NT; from
// LDS the steps of one staging group or fewer (the reads are short and sit right before their use).
template <int F, int NT, int MT, int XS>
constexpr int batch_steps() {
  constexpr int J = Fmt<F>::kElems / 8;
  if (XS == kXLds) return J * MT <= 2 ? 4 : J * MT <= 4 ? 2 : 1;
  int u = 8 / (J * MT * (XS == kXGlobalF32 ? 2 : 1));
  const int cap = kLoadsInFlight / NT;
  u = u > cap ? cap : u;
  return u >= 8 ? 8 : u >= 4 ? 4 : u >= 2 ? 2 : 1;  // a power of two: it divides the weight batch
}

// Sixteen consecutive weight rows starting at `data` (their scale rows at `scale`), of which the first `valid`
// exist: a row past them stands for the last valid one (its outputs are computed and never written).
struct TileRows {
  const uint8_t* data;
  const uint8_t* scale;
  int valid;
};

// A wavefront's private LDS: the staging image of one tile's 4 load steps (16 rows x 16 chunks, and behind each
// row room for its 32 bytes of NVFP4 block scales; the rows 48 bytes apart in the banks so that both the row-wise
// writes and the fragment reads are conflict-free), reused afterwards for the wavefront's partial sums.
constexpr int kStageRow = 16 * 16;
constexpr int kStagePitch = kStageRow + 48;
constexpr int kStageBytes = kTileRows * kStagePitch;

template <int NT, int MT>
constexpr int wave_region_bytes() {
  return NT * MT * kWave * 16 > kStageBytes ? NT * MT * kWave * 16 : kStageBytes;
}

inline size_t tile_lds_bytes(int S, int NT, int MT) {
  const size_t partial = static_cast<size_t>(NT) * MT * kWave * 16;
  return S * (partial > kStageBytes ? partial : static_cast<size_t>(kStageBytes));
}

// Whether the block scales of every row of a stack of NVFP4 rows can be read eight bytes (a load step's four
// chunks) at a time: whole steps in a row, and every row's scales eight-byte aligned.
inline bool wide_scales_fit(const void* scale, int64_t scale_row_bytes, int chunks) {
  return chunks > 0 && chunks % 4 == 0 && scale_row_bytes % 8 == 0 && reinterpret_cast<uintptr_t>(scale) % 8 == 0;
}

// Orders this wavefront's LDS accesses as written (the hardware runs a wavefront's LDS instructions in order;
// this keeps the compiler from moving one lane's read above another lane's write).
__device__ __forceinline__ void wave_lds_order() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// The weights of one batch (kLoadsInFlight / NT load steps of NT tiles) as they arrive from memory.
template <int F, int NT>
struct WeightBatch {
  static constexpr int WU = kLoadsInFlight / NT;
  static_assert(WU % 4 == 0, "weight steps are staged four at a time");
  u32x4 raw[WU / 4][NT][4];
  uint32_t sc[WU][NT];     // NVFP4 block scales a step at a time (rows whose scales do not come in whole, aligned groups)
  u32x2 scq[WU / 4][NT];   // ... or a 4-step group of one row's at once: lane (g, i) holds step g's eight bytes of row i
};

// One 16-byte chunk of byte weights against the same 16 k of byte activations, added to acc.
template <int MATH>
__device__ __forceinline__ i32x4 byte_mfma(const i32x4& w, const i32x4& x, const i32x4& acc) {
  static_assert(MATH == LX_MATH_INT8, "int32 sums are the INT8 math's");
  return __builtin_amdgcn_mfma_i32_16x16x64_i8(w, x, acc, 0, 0, 0);
}

template <int MATH>
__device__ __forceinline__ f32x4 byte_mfma(const i32x4& w, const i32x4& x, const f32x4& acc) {
  static_assert(MATH == LX_MATH_FP8, "f32 sums are the FP8 math's");
  const long w_lo = (static_cast<long>(static_cast<unsigned>(w.y)) << 32) | static_cast<unsigned>(w.x);
  const long w_hi = (static_cast<long>(static_cast<unsigned>(w.w)) << 32) | static_cast<unsigned>(w.z);
  const long x_lo = (static_cast<long>(static_cast<unsigned>(x.y)) << 32) | static_cast<unsigned>(x.x);
  const long x_hi = (static_cast<long>(static_cast<unsigned>(x.w)) << 32) | static_cast<unsigned>(x.z);
  const f32x4 half = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(w_lo, x_lo, acc, 0, 0, 0);
  return __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(w_hi, x_hi, half, 0, 0, 0);
}

// A wavefront's view of NT tiles of weights: where its loads come from and how they reach fragment order.
// The weights of a batch are asked for at once, in the order they lie in memory: one load instruction reads 256
// contiguous bytes of each of four rows (lane -> row 4q + lane / 16, chunk lane % 16 of a 4-step group). They pass
// through `stage` (this wavefront's kStageBytes of LDS) to reach the lanes that feed them to the matrix
// instruction: lane (g, i) takes chunk 4s + g of row i for step s of the group.
template <int F, int NT, bool WIDE = false>
struct TileStream {
  static_assert(!WIDE || F == LX_W_NVFP4, "only NVFP4 has block scales to read");
  static constexpr int E = Fmt<F>::kElems;
  static constexpr int J = E / 8;  // matrix instructions per load step
  static constexpr int WU = WeightBatch<F, NT>::WU;
  static constexpr int G = WU / 4;
  const uint8_t* own_scale[NT];
  const uint8_t* stage_row[NT][4];
  u32x4* put;        // + q * 4 rows
  const u32x4* get;  // + s * 4 chunks
  u32x2* sc_put;     // a group's block scales travel behind its rows
  const uint8_t* sc_get;  // + s * 8 bytes
  int chunks, g, i;
  // NVFP4 block scales are two bytes a chunk. Read a chunk at a time they are 64 two-byte loads of 16 different
  // rows an instruction; read eight bytes a lane (WIDE: a step's four chunks) they are a quarter of the
  // instructions and whole 32-byte runs. That needs whole steps in a row and eight-byte alignment of every row's
  // scales: wide_scales_fit() says whether a stack of rows has both.

  __device__ __forceinline__ TileStream(const TileRows (&tiles)[NT], int64_t row_bytes, int64_t scale_row_bytes, int chunks_,
                                        uint8_t* stage)
      : chunks(chunks_) {
    const int lane = threadIdx.x & (kWave - 1);
    g = lane >> 4;
    i = lane & 15;
#pragma unroll
    for (int n = 0; n < NT; ++n) {
      own_scale[n] = tiles[n].scale + min(i, tiles[n].valid - 1) * scale_row_bytes;
#pragma unroll
      for (int q = 0; q < 4; ++q) stage_row[n][q] = tiles[n].data + min(4 * q + g, tiles[n].valid - 1) * row_bytes;
    }
    put = reinterpret_cast<u32x4*>(stage + g * kStagePitch + i * 16);
    get = reinterpret_cast<const u32x4*>(stage + i * kStagePitch + g * 16);
    sc_put = reinterpret_cast<u32x2*>(stage + i * kStagePitch + kStageRow + g * 8);
    sc_get = stage + i * kStagePitch + kStageRow + g * 2;
  }

  // Asks for the batch of load steps [tb, tb + WU).
  __device__ __forceinline__ void issue(WeightBatch<F, NT>& wb, int tb) const {
#pragma unroll
    for (int grp = 0; grp < G; ++grp) {
      // A chunk past the row's end re-reads the row's last chunk: the steps it lands in are past K or skipped.
      const int c = min(4 * (tb + 4 * grp) + i, chunks - 1);
#pragma unroll
      for (int n = 0; n < NT; ++n)
#pragma unroll
        for (int q = 0; q < 4; ++q)
          wb.raw[grp][n][q] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(stage_row[n][q]) + c);
    }
    if constexpr (WIDE) {
#pragma unroll
      for (int grp = 0; grp < G; ++grp) {
        const int step = min(tb + 4 * grp + g, chunks / 4 - 1);  // past the row's end: its last step's, unused
#pragma unroll
        for (int n = 0; n < NT; ++n) wb.scq[grp][n] = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(own_scale[n]) + step);
      }
    } else {
#pragma unroll
      for (int u = 0; u < WU; ++u)
#pragma unroll
        for (int n = 0; n < NT; ++n) {
          wb.sc[u][n] = 0;
          if constexpr (F == LX_W_NVFP4)
            wb.sc[u][n] = __builtin_nontemporal_load(reinterpret_cast<const uint16_t*>(own_scale[n]) + min(4 * (tb + u) + g, chunks - 1));
        }
    }
  }

  // acc[t][mt] += the batch at tb times activation tile mt; steps from t_end on count for nothing (k_end = the
  // first k that does not count: fragments from there on are zero, by mask or by the image's own zeros).
  template <int MT, int XS>
  __device__ __forceinline__ void consume(const WeightBatch<F, NT>& wb, int tb, const void* const (&xrow)[MT], int K, int k_end,
                                          f32x4 (&acc)[NT][MT]) const {
    constexpr int U = batch_steps<F, NT, MT, XS>();
    constexpr bool MASK = XS != kXLds;
    XFrag<XS> xf[U][J][MT];
    auto load_x = [&](int ub) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int k0 = (4 * (tb + ub + u) + g) * E;
#pragma unroll
        for (int j = 0; j < J; ++j)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) load_x_fragment<XS>(xf[u][j][mt], xrow[mt], k0 + 8 * j, K);
      }
    };
    if constexpr (XS != kXLds) load_x(0);  // in flight together with the weights
    // Four steps at a time: through the staging image into fragment order, then into the matrix instructions.
    u32x4 wv[WU][NT];
    uint32_t scv[WU][NT];
#pragma unroll
    for (int ub = 0; ub < WU; ub += U) {
      if (XS != kXLds && ub > 0) load_x(ub);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if ((ub + u) % 4 == 0) {
          const int grp = (ub + u) / 4;
#pragma unroll
          for (int n = 0; n < NT; ++n) {
#pragma unroll
            for (int q = 0; q < 4; ++q) put[q * (4 * kStagePitch / 16)] = wb.raw[grp][n][q];
            // Row i's 32 scale bytes of the group behind image row i; lane (g, i) takes chunk 4 s + g's two of
            // them for step s.
            if constexpr (WIDE) *sc_put = wb.scq[grp][n];
            wave_lds_order();
#pragma unroll
            for (int sstep = 0; sstep < 4; ++sstep) {
              wv[4 * grp + sstep][n] = get[sstep * 4];
              if constexpr (WIDE) scv[4 * grp + sstep][n] = *reinterpret_cast<const uint16_t*>(sc_get + 8 * sstep);
            }
            wave_lds_order();
          }
        }
        if (XS == kXLds && u == 0) load_x(ub);
        const int k0 = (4 * (tb + ub + u) + g) * E;
#pragma unroll
        for (int j = 0; j < J; ++j) {
#pragma unroll
          for (int n = 0; n < NT; ++n) {
            const bf16x8 wf = weight_fragment<F>(wv[ub + u][n], WIDE ? scv[ub + u][n] : wb.sc[ub + u][n], j);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
              acc[n][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, x_operand<XS, MASK>(xf[u][j][mt], k0 + 8 * j, k_end), acc[n][mt], 0, 0, 0);
          }
        }
      }
    }
  }

  // The quantised maths: weights and per-token quantised activations are one byte a value and go into the matrix
  // instruction as they are stored. MATH = LX_MATH_INT8 (int8 x int8, exact int32 sums, v_mfma_i32_16x16x64_i8: a
  // lane's 16-byte chunk against the same 16 k of its activation row) or LX_MATH_FP8 (e4m3 x e4m3, exact products,
  // f32 sums, v_mfma_f32_16x16x32_fp8_fp8: the chunk's two halves in turn). xrow[mt] points at this lane's activation
  // row; XL says it is an LDS image that is zero past K (and covers every k asked for), otherwise rows in global
  // memory, clamped and masked at k_end.
  template <int MT, bool XL, int MATH, class Acc>
  __device__ __forceinline__ void consume_bytes(const WeightBatch<F, NT>& wb, int tb, const int8_t* const (&xrow)[MT], int K, int k_end,
                                                Acc (&acc)[NT][MT]) const {
    static_assert((MATH == LX_MATH_INT8 && F == LX_W_INT8) || (MATH == LX_MATH_FP8 && F == LX_W_FP8), "one byte a value on both sides");
    constexpr int U = 4;  // one staging group
    i32x4 xf[U][MT];
    auto load_x = [&](int ub) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int k0 = (4 * (tb + ub + u) + g) * 16;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) xf[u][mt] = *reinterpret_cast<const i32x4*>(xrow[mt] + (XL ? k0 : min(k0, K - 16)));
      }
    };
    if constexpr (!XL) load_x(0);
#pragma unroll
    for (int ub = 0; ub < WU; ub += U) {
      if (!XL && ub > 0) load_x(ub);
      u32x4 wv[U][NT];
#pragma unroll
      for (int n = 0; n < NT; ++n) {
#pragma unroll
        for (int q = 0; q < 4; ++q) put[q * (4 * kStagePitch / 16)] = wb.raw[ub / 4][n][q];
        wave_lds_order();
#pragma unroll
        for (int sstep = 0; sstep < 4; ++sstep) wv[sstep][n] = get[sstep * 4];
        wave_lds_order();
      }
      if constexpr (XL) load_x(ub);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int k0 = (4 * (tb + ub + u) + g) * 16;
#pragma unroll
        for (int n = 0; n < NT; ++n)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            i32x4 xv = xf[u][mt];
            if (!XL && k0 >= k_end) xv = i32x4{0, 0, 0, 0};
            acc[n][mt] = byte_mfma<MATH>(__builtin_bit_cast(i32x4, wv[u][n]), xv, acc[n][mt]);
          }
      }
    }
  }
};

// acc[t][mt] += tile t's rows times activation tile mt over load steps [t_begin, t_end).
// xrow[mt] points at this lane's activation row of tile mt. `chunks` is the number of 16-byte chunks in a weight
// row. between() runs once, after the first batch's loads are on their way and before anything is consumed: the
// place to stage activations into LDS (it may hold a workgroup barrier: every wavefront calls it).
// Steps past the slice's end (a last, partial batch) run on re-read weights against zero activations. An LDS
// image is zero from K to the end of the row's last batch, and with it every slice but the row's last is whole
// batches (the caller sees to both), so nothing is masked.
template <int F, int NT, int MT, int XS, bool WIDE = false, class Between>
__device__ __forceinline__ void mfma_slice(const TileRows (&tiles)[NT], int64_t row_bytes, int64_t scale_row_bytes, int chunks,
                                           int t_begin, int t_end, const void* const (&xrow)[MT], int K, f32x4 (&acc)[NT][MT],
                                           uint8_t* stage, Between&& between) {
  const TileStream<F, NT, WIDE> ts(tiles, row_bytes, scale_row_bytes, chunks, stage);
  WeightBatch<F, NT> wb;
  if (t_begin < t_end) ts.issue(wb, t_begin);
  between();
  const int k_end = min(K, 4 * t_end * Fmt<F>::kElems);
  for (int tb = t_begin; tb < t_end; tb += TileStream<F, NT>::WU) {
    if (tb != t_begin) ts.issue(wb, tb);
    ts.template consume<MT, XS>(wb, tb, xrow, K, k_end, acc);
  }
}

// One tile's S wavefronts (a workgroup may hold several tiles' worth: `slice` is this wavefront's index among
// its tile's S, `lds` the tile's regions): wavefront w takes load steps [w * per, (w + 1) * per), the partial
// tiles are added in ascending w through `lds` (tile_lds_bytes(S, NT, MT) bytes, a region per wavefront), and
// epi(mt, q, sums) is called once for every (activation tile mt, lane slot q) with the NT finished sums:
// sums[t][r] belongs to weight row 4 * (q / 16) + r of tile t and activation row mt * 16 + q % 16.
// Every wavefront of the workgroup must make the call: it holds workgroup barriers.
template <int F, int NT, int MT, int XS, bool WIDE = false, class Between, class Epi>
__device__ __forceinline__ void mfma_tile(const TileRows (&tiles)[NT], int64_t row_bytes, int64_t scale_row_bytes, int chunks,
                                          int steps, int steps_per_wave, const void* const (&xrow)[MT], int K, f32x4* lds, int S,
                                          int slice, Between&& between, Epi&& epi) {
  constexpr int kRegion = wave_region_bytes<NT, MT>();
  const int lane = threadIdx.x & (kWave - 1);
  uint8_t* const base = reinterpret_cast<uint8_t*>(lds);
  f32x4 acc[NT][MT];
#pragma unroll
  for (int n = 0; n < NT; ++n)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[n][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int t_begin = min(steps, slice * steps_per_wave), t_end = min(steps, t_begin + steps_per_wave);
  mfma_slice<F, NT, MT, XS, WIDE>(tiles, row_bytes, scale_row_bytes, chunks, t_begin, t_end, xrow, K, acc, base + slice * kRegion, between);
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
  wave_lds_order();
  f32x4* const mine = reinterpret_cast<f32x4*>(base + slice * kRegion);
#pragma unroll
  for (int n = 0; n < NT; ++n)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) mine[(n * MT + mt) * kWave + lane] = acc[n][mt];
  __syncthreads();
  for (int item = slice * kWave + lane; item < MT * kWave; item += S * kWave) {
    const int mt = item / kWave, q = item % kWave;
    f32x4 sums[NT];
#pragma unroll
    for (int n = 0; n < NT; ++n) {
      f32x4 s = reinterpret_cast<const f32x4*>(base)[(n * MT + mt) * kWave + q];
      for (int w = 1; w < S; ++w) s += reinterpret_cast<const f32x4*>(base + w * kRegion)[(n * MT + mt) * kWave + q];
      sums[n] = s;
    }
    epi(mt, q, sums);
  }
}

}  // namespace dro
