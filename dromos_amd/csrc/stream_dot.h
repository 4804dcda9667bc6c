// The weight-streaming dot product shared by the decode GEMV and the decode experts.
//
// A wavefront owns R weight rows at a time (a "group") and streams them whole: at step s, lane l reads the
// 16 bytes at chunk s * 64 + l of each row (one 128-bit non-temporal load, 1 KB contiguous per row per
// wave), so a row's bytes are read exactly once, in order. Loads run one batch (U steps of R rows) ahead of
// the arithmetic in a second register buffer, across group boundaries too, so a wavefront always has a
// batch in flight while it multiplies the previous one.
//
// The activations sit in LDS, laid out so that the 16 bytes a lane reads next are always 16 bytes after its
// neighbour's (no bank conflicts). Two images (XB says which):
//   f32 (XB = false, any activation type): the k values of chunk (s, l) are stored as kElems / 4 groups of
//     four, group q at word index  s * 64 * kElems + q * 256 + l * 4;  products are f32 FMAs.
//   packed bf16 (XB = true, bf16 activations): groups of eight k (four words of two bf16), group j at word
//     index  s * 32 * kElems + j * 256 + l * 4;  the weights are expanded to bf16 pairs (exactly: every stored
//     format fits) and v_dot2c_f32_bf16 adds two products per instruction: half the LDS bytes and about half
//     the instructions.
// Either image is zero past K, so a lane whose chunk lies past the end of the row (its load is clamped to the
// row's last chunk) adds exact zeros.
//
// Every (activation row, weight row) pair keeps one f32 accumulator per lane, fed in ascending step order,
// and the 64 lane sums are combined by one fixed tree (wave_sum). The order never depends on how many
// activation rows share the pass (MT), how many weight rows the wave holds (R) or the batch depth (U), so an
// output's bits depend only on its own x row (and its type), its weight row and the K split.
#pragma once

#include <type_traits>

#include "bf16x.h"
#include "common.h"

namespace dro {

// Word (4-byte) index in the f32 image of element j of chunk (s, l); see the layout above.
template <int F>
__device__ __forceinline__ int x_slot(int s, int l, int j) {
  constexpr int E = Fmt<F>::kElems;
  return s * (kWave * E) + (j >> 2) * 256 + l * 4 + (j & 3);
}

// Word index in the packed bf16 image of the pair that holds element j of chunk (s, l) (j & 1 picks the half).
template <int F>
__device__ __forceinline__ int x_pair_slot(int s, int l, int j) {
  constexpr int E = Fmt<F>::kElems;
  return s * (kWave * E / 2) + (j >> 3) * 256 + l * 4 + ((j & 7) >> 1);
}

// Word index of a lane's chunk (s, lane) in either image.
template <int F, bool XB>
__device__ __forceinline__ int x_chunk_word(int s, int lane) {
  return XB ? x_pair_slot<F>(s, lane, 0) : x_slot<F>(s, lane, 0);
}

// Words the LDS image of one x row takes for a K of `steps` wave steps.
template <int F>
__host__ __device__ constexpr int x_row_floats(int steps) {
  return steps * kWave * Fmt<F>::kElems;
}

template <int F, bool XB>
__host__ __device__ constexpr int x_row_words(int steps) {
  return steps * kWave * Fmt<F>::kElems / (XB ? 2 : 1);
}

// Wave steps that cover K values of format F.
template <int F>
__host__ __device__ inline int steps_for(int64_t K) {
  const int64_t per_step = static_cast<int64_t>(kWave) * Fmt<F>::kElems;
  return static_cast<int>((K + per_step - 1) / per_step);
}

// Steps to ask for at once for rows of `steps` steps: the largest power of two up to `cap` that leaves at most
// a third of the last batch empty (an empty slot re-reads a chunk).
inline int batch_depth(int steps, int cap) {
  for (int u = cap; u > 1; u >>= 1) {
    const int waste = (steps + u - 1) / u * u - steps;
    if (waste * 3 <= steps) return u;
  }
  return 1;
}

// Stages rows [0, M) of x (f32 or bf16, row stride ld_x, optionally gathered through row_of[m]) into the
// LDS image `xs` for MT rows of `steps` steps each; everything past K, and rows M .. MT - 1, are zero.
// Called by the whole workgroup; the caller synchronises afterwards. Rows whose address and stride allow it
// are read 16 bytes at a time, several loads in flight per thread (K is a multiple of 8 whenever the weight
// rows are streamed, so a vector never straddles the end of a row).
template <int F, int MT>
__device__ __forceinline__ void stage_x(float* xs, const void* x, int x_dtype, int64_t ld_x, const int* row_of, int M,
                                        int64_t K, int steps) {
  constexpr int E = Fmt<F>::kElems;
  const int per_row = steps * kWave * E;
  const int esize = x_dtype == LX_BF16 ? 2 : 4;
  const bool vec = reinterpret_cast<uintptr_t>(x) % 16 == 0 && (ld_x * esize) % 16 == 0 && K % 8 == 0;
  if (vec) {
    // All rows at once: item = (row m, vector v of the row), four items in flight per thread.
    const int vec_shift = x_dtype == LX_BF16 ? 3 : 2;
    const int n_vec = per_row >> vec_shift, k_vec = static_cast<int>(K) >> vec_shift;
    const int items = MT * n_vec;
    for (int it0 = threadIdx.x; it0 < items; it0 += blockDim.x * 4) {
      u32x4 r[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int it = it0 + u * blockDim.x;
        const int m = it / n_vec, v = it - m * n_vec;
        r[u] = u32x4{0u, 0u, 0u, 0u};
        if (it < items && m < M && v < k_vec) {
          const int64_t base = static_cast<int64_t>(row_of ? row_of[m] : m) * ld_x;
          r[u] = *(reinterpret_cast<const u32x4*>(static_cast<const char*>(x) + base * esize) + v);
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int it = it0 + u * blockDim.x;
        if (it < items) {
          const int m = it / n_vec, v = it - m * n_vec;
          const int k = v << vec_shift, s = k / (kWave * E), within = k % (kWave * E);
          float* at = xs + m * per_row + x_slot<F>(s, within / E, within % E);
          if (x_dtype == LX_BF16) {
            *reinterpret_cast<f32x4*>(at) = f32x4{__uint_as_float(r[u].x << 16), __uint_as_float(r[u].x & 0xffff0000u),
                                                  __uint_as_float(r[u].y << 16), __uint_as_float(r[u].y & 0xffff0000u)};
            *reinterpret_cast<f32x4*>(at + 256) = f32x4{__uint_as_float(r[u].z << 16), __uint_as_float(r[u].z & 0xffff0000u),
                                                        __uint_as_float(r[u].w << 16), __uint_as_float(r[u].w & 0xffff0000u)};
          } else {
            *reinterpret_cast<f32x4*>(at) = f32x4{__uint_as_float(r[u].x), __uint_as_float(r[u].y), __uint_as_float(r[u].z),
                                                  __uint_as_float(r[u].w)};
          }
        }
      }
    }
    return;
  }
  for (int m = 0; m < MT; ++m) {
    float* dst = xs + m * per_row;
    if (m >= M) {
      for (int i = threadIdx.x * 4; i < per_row; i += blockDim.x * 4) *reinterpret_cast<f32x4*>(dst + i) = f32x4{0.f, 0.f, 0.f, 0.f};
      continue;
    }
    const int64_t base = static_cast<int64_t>(row_of ? row_of[m] : m) * ld_x;
    for (int k0 = threadIdx.x; k0 < per_row; k0 += blockDim.x * 8) {
      float r[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int k = k0 + u * blockDim.x;
        r[u] = k < K ? load_as_f32(x, x_dtype, base + k) : 0.0f;
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int k = k0 + u * blockDim.x;
        if (k < per_row) {
          const int s = k / (kWave * E), within = k % (kWave * E);
          dst[x_slot<F>(s, within / E, within % E)] = r[u];
        }
      }
    }
  }
}

// The packed bf16 image of rows [0, M) of bf16 x (row stride ld_x, optionally gathered through row_of[m]) for
// MT rows of `steps` steps each; everything past K, and rows M .. MT - 1, are zero. As stage_x otherwise.
template <int F, int MT>
__device__ __forceinline__ void stage_x_pairs(uint32_t* xs, const uint16_t* x, int64_t ld_x, const int* row_of, int M, int64_t K,
                                              int steps) {
  constexpr int E = Fmt<F>::kElems;
  const int per_row = x_row_words<F, true>(steps);
  const bool vec = reinterpret_cast<uintptr_t>(x) % 16 == 0 && (ld_x * 2) % 16 == 0 && K % 8 == 0;
  if (vec) {
    const int n_vec = per_row >> 2, k_vec = static_cast<int>(K) >> 3;
    const int items = MT * n_vec;
    for (int it0 = threadIdx.x; it0 < items; it0 += blockDim.x * 4) {
      u32x4 r[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int it = it0 + u * blockDim.x;
        const int m = it / n_vec, v = it - m * n_vec;
        r[u] = u32x4{0u, 0u, 0u, 0u};
        if (it < items && m < M && v < k_vec) {
          const int64_t base = static_cast<int64_t>(row_of ? row_of[m] : m) * ld_x;
          r[u] = *(reinterpret_cast<const u32x4*>(x + base) + v);
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int it = it0 + u * blockDim.x;
        if (it < items) {
          const int m = it / n_vec, v = it - m * n_vec;
          const int k = v << 3, st = k / (kWave * E), within = k % (kWave * E);
          *reinterpret_cast<u32x4*>(xs + m * per_row + x_pair_slot<F>(st, within / E, within % E)) = r[u];
        }
      }
    }
    return;
  }
  uint16_t* halves = reinterpret_cast<uint16_t*>(xs);
  for (int m = 0; m < MT; ++m) {
    const int64_t base = m < M ? static_cast<int64_t>(row_of ? row_of[m] : m) * ld_x : 0;
    for (int k = threadIdx.x; k < per_row * 2; k += blockDim.x) {
      const int st = k / (kWave * E), within = k % (kWave * E);
      const int j = within % E;
      halves[2 * (m * per_row + x_pair_slot<F>(st, within / E, j)) + (j & 1)] = m < M && k < K ? x[base + k] : uint16_t{0};
    }
  }
}

// The same staging in two phases for one activation row, so a kernel can ask for x, then for its first
// weights, and only then wait for x: XRegs holds a thread's share of the row between the two calls. Usable
// when the row can be read 16 bytes at a time and a thread's share is at most kVecs vectors; otherwise
// `ready` is false and the caller falls back to stage_x.
template <int XV = 4>
struct XRegs {
  static constexpr int kVecs = XV;  // 16-byte vectors a thread holds: enough for the row, no more (they cost registers)
  u32x4 v[kVecs];
  int k_vec;  // vectors that lie inside the row: the rest of the image is zero
  bool ready;
};

template <int F, int XV>
__device__ __forceinline__ void stage_x_load(XRegs<XV>& r, const void* x, int x_dtype, int64_t ld_x, int64_t K, int steps) {
  constexpr int E = Fmt<F>::kElems;
  const int per_row = steps * kWave * E;
  const int vec_shift = x_dtype == LX_BF16 ? 3 : 2;  // elements per 16-byte vector: 8 or 4
  const int n_vec = per_row >> vec_shift, k_vec = static_cast<int>(K) >> vec_shift;
  r.k_vec = k_vec;
  r.ready = (reinterpret_cast<uintptr_t>(x) & 15) == 0 && ((ld_x << (4 - vec_shift)) & 15) == 0 && (K & 7) == 0 &&
            n_vec <= XV * static_cast<int>(blockDim.x);
  if (!r.ready) return;
  const u32x4* src = static_cast<const u32x4*>(x);
#pragma unroll
  for (int u = 0; u < XV; ++u) {
    // Clamped, not predicated (a predicated load makes the compiler wait for every load at the next use); what lies
    // past K is zeroed when it is stored.
    const int v = threadIdx.x + u * blockDim.x;
    r.v[u] = src[min(v, k_vec - 1)];
  }
}

template <int F, int XV>
__device__ __forceinline__ void stage_x_store(const XRegs<XV>& r, float* xs, int x_dtype, int steps) {
  constexpr int E = Fmt<F>::kElems;
  const int per_row = steps * kWave * E;
  const int vec_shift = x_dtype == LX_BF16 ? 3 : 2;
  const int n_vec = per_row >> vec_shift;
#pragma unroll
  for (int u = 0; u < XV; ++u) {
    const int v = threadIdx.x + u * blockDim.x;
    if (v < n_vec) {
      const int k = v << vec_shift, s = k / (kWave * E), within = k % (kWave * E);
      float* at = xs + x_slot<F>(s, within / E, within % E);
      const u32x4 w = v < r.k_vec ? r.v[u] : u32x4{0u, 0u, 0u, 0u};
      if (x_dtype == LX_BF16) {
        *reinterpret_cast<f32x4*>(at) = f32x4{__uint_as_float(w.x << 16), __uint_as_float(w.x & 0xffff0000u),
                                              __uint_as_float(w.y << 16), __uint_as_float(w.y & 0xffff0000u)};
        *reinterpret_cast<f32x4*>(at + 256) = f32x4{__uint_as_float(w.z << 16), __uint_as_float(w.z & 0xffff0000u),
                                                    __uint_as_float(w.w << 16), __uint_as_float(w.w & 0xffff0000u)};
      } else {
        *reinterpret_cast<f32x4*>(at) = f32x4{__uint_as_float(w.x), __uint_as_float(w.y), __uint_as_float(w.z), __uint_as_float(w.w)};
      }
    }
  }
}

// The second phase for the packed bf16 image (the row is bf16: its vectors go in as they are).
template <int F, int XV>
__device__ __forceinline__ void stage_x_store_pairs(const XRegs<XV>& r, uint32_t* xs, int steps) {
  constexpr int E = Fmt<F>::kElems;
  const int n_vec = x_row_words<F, true>(steps) >> 2;
#pragma unroll
  for (int u = 0; u < XV; ++u) {
    const int v = threadIdx.x + u * blockDim.x;
    if (v < n_vec) {
      const int k = v << 3, st = k / (kWave * E), within = k % (kWave * E);
      *reinterpret_cast<u32x4*>(xs + x_pair_slot<F>(st, within / E, within % E)) = v < r.k_vec ? r.v[u] : u32x4{0u, 0u, 0u, 0u};
    }
  }
}

// Two-phase staging of up to MT bf16 rows (optionally gathered through row_of[m]) into the packed image: slots
// (row m, pass j) in row-major order, a thread's piece of a slot being vector j * blockDim + thread of row m. Usable
// when the rows can be read 16 bytes at a time and there are at most kSlots slots; otherwise `ready` is false and
// the caller falls back to stage_x_pairs.
template <int SLOTS>
struct XRowRegsN {
  static constexpr int kSlots = SLOTS;
  u32x4 v[kSlots];
  int iters;  // passes per row
  bool ready;
};
using XRowRegs = XRowRegsN<4>;

template <int F, int SLOTS>
__device__ __forceinline__ void stage_rows_load(XRowRegsN<SLOTS>& r, const uint16_t* x, int64_t ld_x, const int* row_of, int M, int64_t K,
                                                int steps) {
  const int n_vec = x_row_words<F, true>(steps) >> 2, k_vec = static_cast<int>(K) >> 3;
  r.iters = (n_vec + blockDim.x - 1) / blockDim.x;
  r.ready = (reinterpret_cast<uintptr_t>(x) & 15) == 0 && ((ld_x * 2) & 15) == 0 && (K & 7) == 0 && M * r.iters <= SLOTS;
  if (!r.ready) return;
  int m = 0, j = 0;
#pragma unroll
  for (int u = 0; u < SLOTS; ++u) {
    // Clamped addresses (no predicated loads); what lies past K or M is replaced by zeros when it is stored.
    const int v = min(static_cast<int>(threadIdx.x) + j * static_cast<int>(blockDim.x), k_vec - 1);
    const int mc = min(m, M - 1);
    r.v[u] = *(reinterpret_cast<const u32x4*>(x + static_cast<int64_t>(row_of ? row_of[mc] : mc) * ld_x) + v);
    if (++j == r.iters) j = 0, ++m;
  }
}

template <int F, int MT, int SLOTS>
__device__ __forceinline__ void stage_rows_store(const XRowRegsN<SLOTS>& r, uint32_t* xs, int M, int64_t K, int steps) {
  constexpr int E = Fmt<F>::kElems;
  const int per_row = x_row_words<F, true>(steps);
  const int n_vec = per_row >> 2, k_vec = static_cast<int>(K) >> 3;
  int m = 0, j = 0;
#pragma unroll
  for (int u = 0; u < SLOTS; ++u) {
    const int v = threadIdx.x + j * blockDim.x;
    if (m < M && v < n_vec) {
      const int k = v << 3, st = k / (kWave * E), within = k % (kWave * E);
      *reinterpret_cast<u32x4*>(xs + m * per_row + x_pair_slot<F>(st, within / E, within % E)) =
          v < k_vec ? r.v[u] : u32x4{0u, 0u, 0u, 0u};
    }
    if (++j == r.iters) j = 0, ++m;
  }
  // Rows M .. MT - 1 are zero.
  for (int i = threadIdx.x; i < (MT - M) * n_vec; i += blockDim.x)
    *reinterpret_cast<u32x4*>(xs + M * per_row + i * 4) = u32x4{0u, 0u, 0u, 0u};
}

// What a lane holds of one weight row for one step: its 16 bytes, and for NVFP4 the two block scales.
template <int F>
struct Chunk {
  u32x4 w;
  uint32_t scales;  // NVFP4: two e4m3 bytes (block of dwords 0-1, block of dwords 2-3)
};
// BF16X: the eight values' sign|mantissa bytes and nibble word, and the step's four tops, which every lane loads from
// the same address; in a row's first chunk of a batch lanes 60 .. 63 load the first four words of the row's header
// instead, so the row's exceptions (nearly always at most a few) ride on a load that is waited for anyway.
template <>
struct Chunk<LX_W_BF16X> {
  uint32_t sm_lo, sm_hi, nib, tops;
};
// The format whose products a chunk enters once it is ready: BF16X rows are decoded to bf16.
template <int F>
constexpr int kProductFormat = F == LX_W_BF16X ? LX_W_BF16 : F;

// Where the streams of an [N, K] matrix's rows start: row n's chunks at data + n * rb, its second stream (NVFP4 block
// scales; BF16X span tops) at scale + n * scale_row. For BF16X `data` skips the first record's header, and both streams
// advance by a whole record.
template <int F>
struct RowBase {
  const uint8_t* data;
  const uint8_t* scale;
  int64_t rb, scale_row;
  int chunks;
  __host__ __device__ RowBase(const uint8_t* d, const uint8_t* s, int64_t K) {
    rb = row_bytes<F>(K);
    chunks = chunks_of<F>(K);
    if constexpr (F == LX_W_BF16X) {
      const bf16x::Geometry g(static_cast<int>(K));
      data = d + g.header;
      scale = d + g.tops_at();
      scale_row = rb;
    } else {
      data = d;
      scale = s;
      scale_row = F == LX_W_NVFP4 ? K / 16 : 0;
    }
  }
};

// The row pointers are the same for every lane of a wavefront; the lane's part is an unsigned 32-bit byte offset, so
// the load can take the row from scalar registers and the offset from one vector register.
template <int F>
__device__ __forceinline__ void load_chunk(Chunk<F>& c, const uint8_t* row, const uint8_t* row_scales, int chunk) {
  const uint32_t off = static_cast<uint32_t>(chunk) * 16u;
  c.w = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(row + off));
  if constexpr (F == LX_W_NVFP4)
    c.scales = __builtin_nontemporal_load(reinterpret_cast<const uint16_t*>(row_scales + (off >> 3)));
}

// A word every lane reads from the same address. A vector load on purpose: weights stream through once, and scalar
// loads of streamed data (every one a miss of the small scalar cache) have measured far slower than a broadcast
// vector load of the line the lanes' own loads fetch anyway.
__device__ __forceinline__ uint32_t uniform_word(const uint8_t* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(p));
}

// What a lane needs to stream LX_W_BF16X rows, computed once. Step s covers spans 4s .. 4s + 3 (768 bytes of the record
// after its header): lane l takes chunk l % 16 of span 4s + l / 16, i.e. 8 sign|mantissa bytes and one nibble word, and
// the span's top is byte l / 16 of the s-th word of tops, which is the same word for the whole wavefront. A lane whose
// chunk lies past the row's end takes the row's last chunk instead (its x is zero): offsets are clamped to the last
// chunk's, and in the row's last step so is the byte picked from the tops.
struct Bf16xLane {
  uint32_t sm_off, nib_off;      // this lane's byte offsets in step 0, from the first span
  uint32_t last_sm, last_nib;    // those of the row's last chunk
  uint32_t top_sel, top_sel_last;  // v_perm selectors that replicate the lane's top byte (any step / the last step)
  int hdr_bytes, slots, chunks, last_step;
  __device__ __forceinline__ void set(int K, int lane) {
    const bf16x::Geometry g(K);
    hdr_bytes = g.header;
    slots = g.slots;
    chunks = K / 8;
    last_step = (chunks - 1) / kWave;
    const uint32_t quarter = static_cast<uint32_t>(lane) >> 4, within = static_cast<uint32_t>(lane) & 15u;
    sm_off = quarter * bf16x::kSpanBytes + within * 8u;
    nib_off = quarter * bf16x::kSpanBytes + bf16x::kNibbles + within * 4u;
    const uint32_t last = static_cast<uint32_t>(chunks - 1), last_span = last >> 4;
    last_sm = __umul24(last_span, bf16x::kSpanBytes) + (last & 15u) * 8u;
    last_nib = __umul24(last_span, bf16x::kSpanBytes) + bf16x::kNibbles + (last & 15u) * 4u;
    top_sel = quarter * 0x01010101u;
    top_sel_last = min(quarter, last_span & 3u) * 0x01010101u;
  }
};

__device__ __forceinline__ void load_chunk_bf16x(Chunk<LX_W_BF16X>& c, const uint8_t* row, const uint8_t* tops, int s, bool with_head,
                                                 const Bf16xLane& g) {
  const uint32_t step_off = static_cast<uint32_t>(s) * (4u * bf16x::kSpanBytes);
  const u32x2 sm = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(row + min(g.sm_off + step_off, g.last_sm)));
  c.sm_lo = sm.x;
  c.sm_hi = sm.y;
  c.nib = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(row + min(g.nib_off + step_off, g.last_nib)));
  const uint32_t lane = threadIdx.x & (kWave - 1);
  c.tops = uniform_word(with_head && lane >= kWave - 4 ? row - g.hdr_bytes + 4u * (lane - (kWave - 4)) : tops + 4 * s);
}

// The chunk as the bf16 kernel would have loaded it: four words of two bf16 each.
__device__ __forceinline__ u32x4 decode_chunk_bf16x(const Chunk<LX_W_BF16X>& c, int s, const Bf16xLane& g) {
  const uint32_t tops = __builtin_amdgcn_readfirstlane(c.tops);
  const uint32_t top4 = __builtin_amdgcn_perm(tops, tops, s == g.last_step ? g.top_sel_last : g.top_sel);
  const u32x2 a = bf16x::quad_bits(c.sm_lo, top4 - (c.nib & 0x0f0f0f0fu));
  const u32x2 b = bf16x::quad_bits(c.sm_hi, top4 - ((c.nib >> 4) & 0x0f0f0f0fu));
  return u32x4{a.x, a.y, b.x, b.y};
}

// One exception word applied to the lane's decoded chunk (index `chunk`) if it names one of its values.
__device__ __forceinline__ u32x4 patch_chunk_bf16x(u32x4 w, uint32_t word, uint32_t chunk) {
  const uint32_t k = word >> 8;
  if ((k >> 3) == chunk) {
    const uint32_t sh = (k & 1u) * 16u + 7u;
    const uint32_t keep = ~(0xffu << sh), bits = (word & 0xffu) << sh;
    const uint32_t d = (k >> 1) & 3u;
    w.x = d == 0 ? (w.x & keep) | bits : w.x;
    w.y = d == 1 ? (w.y & keep) | bits : w.y;
    w.z = d == 2 ? (w.z & keep) | bits : w.z;
    w.w = d == 3 ? (w.w & keep) | bits : w.w;
  }
  return w;
}

// A row's exceptions as the products of one batch use them, the same in every lane. Up to four words sit in scalar
// registers (kVacant: none); they came with the batch's loads and cover nearly every row that has any. A row with more
// (its fourth word is taken and the header has further slots, or it has a spill record) costs one more load: lane l
// takes word l of the list into `listed`, up to 64 of them; a list longer than that (`beyond` > 0) is walked in
// memory for the rest. `steps` says which of the batch's steps hold an exception (bit u: step s0 + u), so that the
// chunks of the other steps spend nothing.
struct Bf16xExceptions {
  uint32_t word[4];
  uint32_t steps;
  bool wide;           // the words are in `listed`, not in word[]
  uint32_t listed;     // per lane
  const uint32_t* list;
  uint32_t count;      // words in the list (an upper bound: a kVacant ends it early)
  // `first`: the row's first chunk of the batch, whose lanes 60 .. 63 hold the header's first four words; rec: the
  // row record; U: the batch's steps.
  template <int U>
  __device__ __forceinline__ Bf16xExceptions(const Chunk<LX_W_BF16X>& first, const uint8_t* rec, int slots, int s0, std::integral_constant<int, U>) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t v = __builtin_amdgcn_readlane(first.tops, kWave - 4 + i);
      word[i] = i < slots ? v : bf16x::kVacant;  // a header of fewer than four words: the rest are tops
    }
    const bool spilled = word[0] != bf16x::kVacant && (word[0] & bf16x::kSpilled);
    wide = spilled || (slots > 4 && word[3] != bf16x::kVacant);
    steps = 0u;
    listed = bf16x::kVacant;
    list = nullptr;
    count = 0;
    if (!wide) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t d = (word[i] >> 17) - static_cast<uint32_t>(s0);  // a word's step: k / 512
        if (word[i] != bf16x::kVacant && d < 32u) steps |= 1u << d;
      }
    } else {
      const bf16x::Exceptions ex(rec, slots);
      list = ex.words;
      count = ex.limit;
      const uint32_t lane = threadIdx.x & (kWave - 1);
      if (lane < count) listed = list[lane];
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (__ballot(listed != bf16x::kVacant && (listed >> 17) == static_cast<uint32_t>(s0 + u)) != 0) steps |= 1u << u;
      if (count > static_cast<uint32_t>(kWave)) steps = ~0u;
    }
  }

  // The exceptions that fall into the lane's decoded chunk (index `chunk`), applied.
  __device__ __forceinline__ u32x4 apply(u32x4 w, uint32_t chunk) const {
    if (!wide) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (word[i] != bf16x::kVacant) w = patch_chunk_bf16x(w, word[i], chunk);
      return w;
    }
    const uint32_t n = count < static_cast<uint32_t>(kWave) ? count : static_cast<uint32_t>(kWave);
    for (uint32_t i = 0; i < n; ++i) {
      const uint32_t v = __builtin_amdgcn_readlane(listed, i);
      if (v == bf16x::kVacant) return w;
      w = patch_chunk_bf16x(w, v, chunk);
    }
    for (uint32_t i = kWave; i < count; ++i) {  // a list of more than 64 words: a row of noise, not of weights
      const uint32_t v = list[i];
      if (v == bf16x::kVacant) break;
      w = patch_chunk_bf16x(w, v, chunk);
    }
    return w;
  }
};

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

// The pairs of one dword of a chunk as bf16 (exact for every format): BF16 1, INT8 / FP8 2, NVFP4 4 pairs.
template <int F>
__device__ __forceinline__ void dword_pairs(uint32_t d, bf16x2* out);

template <>
__device__ __forceinline__ void dword_pairs<LX_W_BF16>(uint32_t d, bf16x2* out) {
  out[0] = as_bf16x2(d);
}

template <>
__device__ __forceinline__ void dword_pairs<LX_W_INT8>(uint32_t d, bf16x2* out) {
  float v[4];
  decode_dword<LX_W_INT8>(d, v);
  const f32x2 lo = {v[0], v[1]}, hi = {v[2], v[3]};
  out[0] = __builtin_convertvector(lo, bf16x2);
  out[1] = __builtin_convertvector(hi, bf16x2);
}

template <>
__device__ __forceinline__ void dword_pairs<LX_W_FP8>(uint32_t d, bf16x2* out) {
  out[0] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(d, 1.0f, false);
  out[1] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(d, 1.0f, true);
}

template <>
__device__ __forceinline__ void dword_pairs<LX_W_NVFP4>(uint32_t d, bf16x2* out) {
  out[0] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(d, 1.0f, 0);
  out[1] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(d, 1.0f, 1);
  out[2] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(d, 1.0f, 2);
  out[3] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(d, 1.0f, 3);
}

// chunk_fma on the packed bf16 image: xs points at the image's words of row 0 for this lane's chunk, per_row words
// separate the rows; a += w0 * x0 + w1 * x1 per instruction, pairs in ascending k.
template <int F, int MT>
__device__ __forceinline__ void chunk_dot2(const Chunk<F>& c, const uint32_t* xs, int per_row, float (&acc)[MT]) {
  constexpr int P = DwordVals<F>::kCount / 2;  // pairs per dword
  if constexpr (F == LX_W_NVFP4) {
    // Two blocks of 16 codes (two dwords, i.e. two groups of eight k): summed from zero, scaled once.
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const float scale = b == 0 ? e4m3_byte_to_f32<0>(c.scales) : e4m3_byte_to_f32<1>(c.scales);
      float part[MT];
#pragma unroll
      for (int m = 0; m < MT; ++m) part[m] = 0.0f;
#pragma unroll
      for (int d = 0; d < 2; ++d) {
        bf16x2 w[4];
        dword_pairs<F>(c.w[2 * b + d], w);
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          const u32x4 xv = *reinterpret_cast<const u32x4*>(xs + m * per_row + (2 * b + d) * 256);
#pragma unroll
          for (int p = 0; p < 4; ++p) part[m] = __builtin_amdgcn_fdot2_f32_bf16(w[p], as_bf16x2(xv[p]), part[m], false);
        }
      }
#pragma unroll
      for (int m = 0; m < MT; ++m) acc[m] = __builtin_fmaf(part[m], scale, acc[m]);
    }
  } else {
    constexpr int G = 4 * P / 4;  // groups of eight k in the chunk: BF16 1, INT8 / FP8 2
#pragma unroll
    for (int g = 0; g < G; ++g) {
      bf16x2 w[4];
      if constexpr (P == 1) {
#pragma unroll
        for (int d = 0; d < 4; ++d) dword_pairs<F>(c.w[d], w + d);
      } else {
        dword_pairs<F>(c.w[2 * g], w);
        dword_pairs<F>(c.w[2 * g + 1], w + 2);
      }
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        const u32x4 xv = *reinterpret_cast<const u32x4*>(xs + m * per_row + g * 256);
#pragma unroll
        for (int p = 0; p < 4; ++p) acc[m] = __builtin_amdgcn_fdot2_f32_bf16(w[p], as_bf16x2(xv[p]), acc[m], false);
      }
    }
  }
}

// Streams a sequence of groups of R rows through a wavefront.
//
//   RowStreamer<F, MT, R, U, XB> st(chunks, s_begin, s_end, per_row);      // per_row in words of the image XB names
//   st.prefetch(rows_fn, first_group, group_stride, n_groups);   // weights do not depend on x: ask first
//   ... stage x in LDS, __syncthreads() ...
//   st.run(rows_fn, done_fn, first_group, group_stride, n_groups);
//
// rows_fn(group, rows, scales, xs) fills the R row pointers (and NVFP4 scale rows) of group `group` and, per row,
// the LDS image its products read (one image for all rows in a GEMV; one per row where every row meets its own
// activations); done_fn(group, acc) receives the lane sums acc[MT][R] of a finished group (the caller reduces
// them across the wave). Steps [s_begin, s_end) of every row are taken, in batches of U.
// ONE: the stream is a single group whose steps fit one batch (s_end - s_begin <= U): one buffer, no loop.
template <int F, int MT, int R, int U, bool XB = false, bool ONE = false>
struct RowStreamer {
  Chunk<F> buf_a[U][R], buf_b[ONE ? 1 : U][ONE ? 1 : R];
  int chunks, s_begin, s_end, per_row, batches, lane;
  // BF16X: the row pointers of rows_fn point at a record's first span (its header lies before), the scale pointers at
  // its tops; a row with exceptions (its first word says so) takes them from the header.
  Bf16xLane x12;

  __device__ __forceinline__ void set_bf16x(int K) { x12.set(K, threadIdx.x & (kWave - 1)); }

  __device__ __forceinline__ RowStreamer(int chunks_, int s_begin_, int s_end_, int per_row_)
      : chunks(chunks_), s_begin(s_begin_), s_end(s_end_), per_row(per_row_) {
    const int n = s_end - s_begin;
    batches = n > 0 ? (n + U - 1) / U : 1;
    lane = threadIdx.x & (kWave - 1);
  }

  template <class RowsFn>
  __device__ __forceinline__ void issue(Chunk<F> (&buf)[U][R], RowsFn& rows_fn, int group, int batch) {
    const uint8_t* rows[R];
    const uint8_t* scales[R];
    const float* xs[R];
    rows_fn(group, rows, scales, xs);
    const int last_step = s_end > s_begin ? s_end - 1 : s_begin;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      // A step past the range, or a chunk past the row's end, re-reads a valid chunk; it is never multiplied
      // (the step is skipped) or multiplies zeros (the x image is zero there).
      const int s = min(s_begin + batch * U + u, last_step);
      if constexpr (F == LX_W_BF16X) {
#pragma unroll
        for (int r = 0; r < R; ++r) load_chunk_bf16x(buf[u][r], rows[r], scales[r], s, u == 0, x12);
      } else {
        const int chunk = min(s * kWave + lane, chunks - 1);
#pragma unroll
        for (int r = 0; r < R; ++r) load_chunk<F>(buf[u][r], rows[r], scales[r], chunk);
      }
    }
  }

  // The chunk as the products take it: BF16X is decoded to bf16 bits here (s: the chunk's step). FIX: the row's
  // exceptions `ex` are applied; a word's step (k / 512) is the same for the whole wavefront, so only the chunks of
  // that step spend vector instructions on it.
  template <bool FIX, class Ex>
  __device__ __forceinline__ Chunk<kProductFormat<F>> ready(const Chunk<F>& c, const Ex& ex, const uint8_t* row, int s, int u) const {
    if constexpr (F == LX_W_BF16X) {
      Chunk<LX_W_BF16> o;
      o.w = decode_chunk_bf16x(c, s, x12);
      if constexpr (FIX) {
        if ((ex.steps >> u) & 1u) o.w = ex.apply(o.w, static_cast<uint32_t>(min(s * kWave + lane, chunks - 1)));
      }
      o.scales = 0;
      return o;
    } else {
      return c;
    }
  }

  // Whether any row of the batch lists exceptions (BF16X; the same answer in every lane).
  __device__ __forceinline__ bool any_exceptions(const Chunk<F> (&buf)[U][R]) const {
    if constexpr (F == LX_W_BF16X) {
      bool any = false;
#pragma unroll
      for (int r = 0; r < R; ++r) any |= __builtin_amdgcn_readlane(buf[0][r].tops, kWave - 4) != bf16x::kVacant;
      return any;
    } else {
      return false;
    }
  }

  struct NoExceptions {};

  // Row r's chunk of step s (buffer slot u) into the sums.
  template <bool FIX, class Ex>
  __device__ __forceinline__ void consume_one(const Chunk<F>& c, const Ex& ex, const uint8_t* row, const float* x_image, int s, int u, int s_off,
                                              int r, float (&acc)[MT][R]) {
    const int slot = x_chunk_word<F, XB>(s - s_off, lane);
    float a[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) a[m] = acc[m][r];
    constexpr int PF = kProductFormat<F>;
    const Chunk<PF> ready_chunk = ready<FIX>(c, ex, row, s, u);
    if constexpr (XB) chunk_dot2<PF, MT>(ready_chunk, reinterpret_cast<const uint32_t*>(x_image) + slot, per_row, a);
    else chunk_fma<PF, MT>(ready_chunk, x_image + slot, per_row, a);
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[m][r] = a[m];
  }

  // The steps [lo, hi) of the batch in `buf` (whose first step is s0), against images whose first step is s_off, in
  // the order the loads were asked for (step by step). With exceptions about (FIX) it goes row by row instead, so
  // that one row's words are live at a time; a row's sums see its steps in ascending order either way.
  template <bool FIX>
  __device__ __forceinline__ void consume_range(const Chunk<F> (&buf)[U][R], const uint8_t* const (&rows)[R], const float* const (&xs)[R],
                                                int s0, int lo, int hi, int s_off, float (&acc)[MT][R]) {
    if constexpr (FIX && F == LX_W_BF16X) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const Bf16xExceptions ex(buf[0][r], rows[r] - x12.hdr_bytes, x12.slots, s0, std::integral_constant<int, U>{});
#pragma unroll
        for (int u = 0; u < U; ++u)
          if (s0 + u >= lo && s0 + u < hi) consume_one<true>(buf[u][r], ex, rows[r], xs[r], s0 + u, u, s_off, r, acc);
      }
    } else {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (s0 + u >= lo && s0 + u < hi) {
#pragma unroll
          for (int r = 0; r < R; ++r) consume_one<false>(buf[u][r], NoExceptions{}, rows[r], xs[r], s0 + u, u, s_off, r, acc);
        }
      }
    }
  }

  // A batch none of whose rows lists exceptions (nearly every batch) runs as one straight block.
  __device__ __forceinline__ void consume_checked(const Chunk<F> (&buf)[U][R], const uint8_t* const (&rows)[R], const float* const (&xs)[R],
                                                  int s0, int lo, int hi, int s_off, float (&acc)[MT][R]) {
    if (any_exceptions(buf)) consume_range<true>(buf, rows, xs, s0, lo, hi, s_off, acc);
    else consume_range<false>(buf, rows, xs, s0, lo, hi, s_off, acc);
  }

  __device__ __forceinline__ void consume(const Chunk<F> (&buf)[U][R], const uint8_t* const (&rows)[R], const float* const (&xs)[R],
                                          int batch, float (&acc)[MT][R]) {
    const int s0 = s_begin + batch * U;
    consume_checked(buf, rows, xs, s0, s0, s_end, 0, acc);
  }

  // The steps [lo, hi) of the single batch in `buf`, against an image whose first step is s_off.
  __device__ __forceinline__ void consume_steps(const Chunk<F> (&buf)[U][R], const uint8_t* const (&rows)[R], const float* const (&xs)[R],
                                                int lo, int hi, int s_off, float (&acc)[MT][R]) {
    consume_checked(buf, rows, xs, s_begin, lo, hi < s_end ? hi : s_end, s_off, acc);
  }

  // ONE only: the group's batch against two images in turn, the first holding steps [0, split), the second the
  // rest; restage() swaps them (the whole workgroup calls this: restage holds barriers). The sums see the steps
  // in the same ascending order as with one image.
  template <class RowsFn, class DoneFn, class Restage>
  __device__ __forceinline__ void run_two_images(RowsFn& rows_fn, DoneFn& done_fn, int group, int split, Restage&& restage) {
    static_assert(ONE, "one batch");
    float acc[MT][R];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int r = 0; r < R; ++r) acc[m][r] = 0.0f;
    const uint8_t* rows[R];
    const uint8_t* scales[R];
    const float* xs[R];
    rows_fn(group, rows, scales, xs);
    consume_steps(buf_a, rows, xs, 0, split, 0, acc);
    restage();
    consume_steps(buf_a, rows, xs, split, s_end, split, acc);
    done_fn(group, acc);
  }

  // Asks for the first two batches of a stream of n_groups groups (the second one only if there is one).
  template <class RowsFn>
  __device__ __forceinline__ void prefetch(RowsFn& rows_fn, int first_group, int stride, int n_groups) {
    issue(buf_a, rows_fn, first_group, 0);
    if constexpr (!ONE) {
      if (batches > 1) issue(buf_b, rows_fn, first_group, 1);
      else if (n_groups > 1) issue(buf_b, rows_fn, first_group + stride, 0);
    }
  }

  // ONE, several groups a wavefront (first_group, first_group + stride, ..., n_groups of them; prefetch() has asked for
  // the first): as soon as a step's chunks have been multiplied, their registers take the same step of the next group,
  // so a wavefront keeps a whole batch on its way while it multiplies, in the registers of one. Every load sits outside
  // any branch (the last group, which asks for nothing, is a copy of its own): a load under a condition would turn every
  // later wait into a wait for all of them. Not for BF16X (its exceptions ride on a batch's first chunk).
  // pre_fn(g) asks for what group g's epilogue needs and finish_fn(g, acc, that) uses it: asked for before the next
  // group's chunks, it is there when the sums are (loads return in order: asked for at the end, it would wait for all
  // of the next group).
  template <class RowsFn, class PreFn, class FinishFn>
  __device__ __forceinline__ void run_rolling(RowsFn& rows_fn, PreFn& pre_fn, FinishFn& finish_fn, int first_group, int stride, int n_groups) {
    static_assert(ONE && F != LX_W_BF16X, "one buffer, plain chunks");
    float acc[MT][R];
    auto zero = [&] {
#pragma unroll
      for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int r = 0; r < R; ++r) acc[m][r] = 0.0f;
    };
    zero();
    const int last_step = s_end > s_begin ? s_end - 1 : s_begin;
    const uint8_t* rows[R];
    const uint8_t* scales[R];
    const float* xs[R];
    rows_fn(first_group, rows, scales, xs);
    int g = first_group;
    auto step = [&](int u) {
      if (s_begin + u < s_end) {
#pragma unroll
        for (int r = 0; r < R; ++r) consume_one<false>(buf_a[u][r], NoExceptions{}, rows[r], xs[r], s_begin + u, u, 0, r, acc);
      }
    };
    // A row pointer is the same in every lane: said so, the loads take it from scalar registers.
    auto uniform = [](const uint8_t* p) {
      const uint64_t v = reinterpret_cast<uint64_t>(p);
      const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v)), hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
      return reinterpret_cast<const uint8_t*>((static_cast<uint64_t>(hi) << 32) | lo);
    };
    for (int t = 1; t < n_groups; ++t) {
      const uint8_t* next_rows[R];
      const uint8_t* next_scales[R];
      const float* next_xs[R];
      rows_fn(g + stride, next_rows, next_scales, next_xs);
#pragma unroll
      for (int r = 0; r < R; ++r) next_rows[r] = uniform(next_rows[r]), next_scales[r] = uniform(next_scales[r]);
      const auto epilogue = pre_fn(g);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        step(u);
        // The scheduler is held to this order: left alone it asks for the next group's chunks early, in registers of
        // their own, and the kernel loses the wavefronts those registers would have held.
        __builtin_amdgcn_sched_barrier(0);
        const int chunk = min(min(s_begin + u, last_step) * kWave + lane, chunks - 1);
#pragma unroll
        for (int r = 0; r < R; ++r) load_chunk<F>(buf_a[u][r], next_rows[r], next_scales[r], chunk);
        __builtin_amdgcn_sched_barrier(0);
      }
      finish_fn(g, acc, epilogue);
      zero();
      g += stride;
#pragma unroll
      for (int r = 0; r < R; ++r) rows[r] = next_rows[r], scales[r] = next_scales[r], xs[r] = next_xs[r];
    }
    const auto epilogue = pre_fn(g);
#pragma unroll
    for (int u = 0; u < U; ++u) step(u);
    finish_fn(g, acc, epilogue);
  }

  // Groups first_group, first_group + stride, ... (n_groups of them); prefetch() has asked for the first two
  // batches.
  template <class RowsFn, class DoneFn>
  __device__ __forceinline__ void run(RowsFn& rows_fn, DoneFn& done_fn, int first_group, int stride, int n_groups) {
    float acc[MT][R];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int r = 0; r < R; ++r) acc[m][r] = 0.0f;
    if constexpr (ONE) {
      const uint8_t* rows[R];
      const uint8_t* scales[R];
      const float* xs[R];
      rows_fn(first_group, rows, scales, xs);
      consume(buf_a, rows, xs, 0, acc);
      done_fn(first_group, acc);
    } else {
    int group = first_group, batch = 0, left = n_groups;
    bool first = true;  // the first half-iteration's next batch is already on its way
    // One half-iteration: ask for the batch after (group, batch) into `next`, multiply `cur`.
    auto half = [&](const Chunk<F>(&cur)[U][R], Chunk<F>(&next)[U][R]) {
      const bool last_batch = batch + 1 == batches;
      const int ng = last_batch ? group + stride : group, nb = last_batch ? 0 : batch + 1;
      if (!(last_batch && left == 1) && !first) issue(next, rows_fn, ng, nb);
      first = false;
      const uint8_t* rows[R];
      const uint8_t* scales[R];
      const float* xs[R];
      rows_fn(group, rows, scales, xs);
      consume(cur, rows, xs, batch, acc);
      if (last_batch) {
        done_fn(group, acc);
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
          for (int r = 0; r < R; ++r) acc[m][r] = 0.0f;
        --left;
      }
      group = ng;
      batch = nb;
    };
    while (left > 0) {
      half(buf_a, buf_b);
      if (left == 0) break;
      half(buf_b, buf_a);
    }
    }
  }
};

}  // namespace dro
