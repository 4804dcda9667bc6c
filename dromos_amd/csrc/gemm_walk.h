// The walk kernel (a template on the weight format; one source per format instantiates it): the matrix-core product for up to 64 bf16 activation rows (BF16 math) in which a wavefront walks
// along a tile's rows instead of taking one short piece of them.
//
// The arithmetic is the tile kernels' (tile_mfma.h): a tile is 16 weight rows; K is cut into S contiguous slices of
// steps_per_wave load steps; a slice's products are one ascending chain of v_mfma_f32_16x16x32_bf16 from zero, the S
// partial tiles are added in ascending slice order, then the epilogue. S depends on (format, K, N) only, so a row's
// bits are those of every other kernel of the library, whatever M is (engine/cuda/kernels.h:453-477).
//
// A wavefront takes all S slices of its tile one after the other and keeps their sums apart (in an LDS area of its own)
// until the end, where it adds them in ascending order: no two wavefronts ever exchange partial tiles. The W
// wavefronts of a workgroup (W tiles) are at the same k at the same time, so the activation image is one window of
// four load steps, twice, whatever K, M and S are. Workgroup b starts with slice b % S and goes round: weight rows are
// a power of two apart, and a device whose wavefronts all read the same offset of their rows at the same moment keeps
// hitting the same few memory channels (measured: a plain read in that pattern takes 11.4 us where 9.8 us is possible).
// What keeps the memory busy is depth: a wavefront always has four groups of four load steps (16 KB) on their way,
// asked for one group at a time as the oldest is used, so the device's requests are paced instead of arriving all at
// once, and the activations are asked for two windows ahead, just before the weights of the same distance (loads come
// back in the order they were asked for). One barrier per window.
//
// Inside an image a 16-byte piece of k of the 16 rows of an activation tile is one 256-byte block, the rows rotated by
// four slots per piece, so that the fragment reads (16 rows of one piece) and the staging writes (4 rows x 4 pieces per
// 16 lanes) touch every bank once. The one-byte formats take another rotation (eight slots on odd pieces, staging items of
// eight rows of a whole step): the LDS serves a 16-byte read at its full 256 bytes a clock only when the four 16-lane
// groups of the wavefront address their blocks at the same rotation, and a fragment read of those formats takes pieces
// that are all even or all odd (measured: C2 int8 at 64 rows 25.7 -> 23.8 us, the bank-conflict counter 2.8 M -> 1.0 M). The weights arrive in memory order (256 contiguous bytes of each of four rows per
// instruction) and pass through a 4 KB image of the wavefront's own (chunk c of row r at slot c ^ r) into fragment order.
#pragma once

#include <type_traits>

#include "common.h"
#include "gemm_args.h"
#include "tile_mfma.h"

namespace dro {
namespace walk {

template <int N>
using Tag = std::integral_constant<int, N>;

// MODE kRot: the workgroups start at different slices (see above) and a wavefront keeps every slice's sum in LDS until the
// end. kPlain: every workgroup starts at slice 0 and the sums are added as the slices end, in registers: the form for
// shapes whose images leave no room for the sums. kPart: the matrix has too few tiles to fill the device with whole
// walks, so workgroup (bx, by) walks only slices [by * walk_slices, (by + 1) * walk_slices) of its tiles and leaves every
// slice's sum in a.partial ([slice][tile][16 rows][lane] x 4 floats); the caller's second kernel adds them in ascending
// order and runs the epilogue, so the sums are the same. kSplit, for the same matrices while they are small (few tiles
// and short rows: a whole walk is then a few wavefronts' long chains of dependent steps, and single slices pay a second
// launch): the W wavefronts of a workgroup take one tile between them, wavefront w slices [w * walk_slices,
// (w + 1) * walk_slices), each with windows of its own (no barrier until the end: a wavefront stages what it reads), and
// the slices' sums meet in LDS, where the first wavefront adds them in ascending order.
constexpr int kPlain = 0, kRot = 1, kPart = 2, kSplit = 3;
// A wavefront's own image: 4 KB of weights (16 rows x 256 bytes) and, for NVFP4, the group's block scales behind them
// (16 rows x 32 bytes, the rows 40 bytes apart).
constexpr int kScalePitch = 40;
template <int F>
constexpr int stage_bytes() {
  return F == LX_W_NVFP4 ? 4096 + 16 * kScalePitch : 4096;
}
// RAGGED (kPlain and kPart): rows that are not whole walks, that is, whose load steps are not a multiple of 16 or whose
// last step is cut short by K. A walk still runs in fours of groups: past the row's end the loads are clamped to the row's
// last 16 bytes (weights, block scales and activations alike) and the activation pieces from K on are zeroed on their way
// into the image, so the groups and chunks that are not there add zeros to the row's last slice.
template <int F, int MT, int W, int MODE, bool RAGGED = false>
__global__ void __launch_bounds__(W* kWave) walk_kernel(const GemmArgs a) {
  constexpr bool ROT = MODE == kRot, PART = MODE == kPart, SPLIT = MODE == kSplit;
  static_assert(!RAGGED || MODE == kPlain || MODE == kPart, "rows that are not whole walks: from the row's start, or single slices");
  extern __shared__ __align__(16) f32x4 lds4[];
  constexpr int E = Fmt<F>::kElems, J = E / 8;
  constexpr int PB = 4 * J;          // 16-byte pieces of an image row under one load step
  constexpr int WS = SPLIT ? 1 : W;  // the wavefronts that share a window
  constexpr int Q = MT * 4 * J / WS;  // staging pieces a lane holds per window
  static_assert(Q * WS == MT * 4 * J && Q >= 1, "the wavefronts share a window's pieces evenly");
  constexpr int kImage = MT * 4 * PB * 256;  // one window
  const int lane = threadIdx.x & (kWave - 1), wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int tw = SPLIT ? 0 : wave;  // tile of the workgroup, and the wavefront's place among those that share its windows
  const int n_tiles = (a.N + kTileRows - 1) / kTileRows;
  const int tile = SPLIT ? blockIdx.x : blockIdx.x * W + tw;
  const int n0 = min(tile, n_tiles - 1) * kTileRows, valid = min(kTileRows, a.N - n0);  // a tile past the last repeats it
  const int g = lane >> 4, i = lane & 15;
  uint8_t* const lds = reinterpret_cast<uint8_t*>(lds4);
  constexpr int kStage = stage_bytes<F>();
  uint8_t* const stage = lds + wave * kStage;
  uint8_t* const img = lds + W * kStage + (SPLIT ? wave * 2 * kImage : 0);  // + buffer * kImage
  const int gps = a.steps_per_wave >> 2;  // groups of four load steps in a slice (the row's last slice may be shorter)
  const int row_groups = RAGGED ? (a.steps + 3) >> 2 : a.steps >> 2;  // and in a row
  const int slices = (row_groups + gps - 1) / gps;  // the slices that hold steps (a.S may count empty ones behind them: their sums are zero)
  const int first_slice = ROT ? blockIdx.x % slices : PART ? blockIdx.y * a.walk_slices : SPLIT ? wave * a.walk_slices : 0, rot = first_slice * gps;
  const int real_groups = PART || SPLIT ? min(a.walk_slices * gps, row_groups - rot) : row_groups;
  const int groups = RAGGED ? (real_groups + 3) & ~3 : real_groups, last = groups - 1;  // the groups this wavefront walks
  // The l-th group this wavefront takes (l past the end repeats the last one).
  auto group_of = [&](int l) {
    const int gq = min(l, last) + rot;
    return ROT && gq >= row_groups ? gq - row_groups : gq;  // kRot goes round; RAGGED: groups past the row's end hold nothing
  };

  // Staging: item idx = (tile of rows * 4 + step of the window) * J + quad of pieces; wavefront tw takes
  // items tw, tw + W, ... A lane's piece of an item: row 4 (lane / 16) + (lane % 16) / 4, piece lane % 4 of the quad.
  // (J == 2, the one-byte formats: an item is instead eight rows of a whole step, lane (g, i) holding row 8 h + i / 2,
  // piece 2 g + i % 2, and a piece's rows are rotated by eight slots on odd pieces: writes and reads both touch every
  // bank once, and the four 16-lane groups of a fragment read, whose pieces are all even or all odd, share one rotation,
  // which is what the LDS serves at full rate.)
  const int r = 4 * g + (i >> 2), e3 = i & 3;
  const uint32_t lds_lane = e3 * 256 + ((r + 4 * e3) & 15) * 16;
  const char* const xbase = static_cast<const char*>(a.xs.x);
  const uint32_t ld_bytes = static_cast<uint32_t>(a.xs.ld) * 2u;
  uint32_t x_off[Q];  // byte offset of this lane's piece of item `it` within window 0
  uint32_t x_lds[J == 2 ? Q : 1];  // J == 2: where it goes in an image
  // RAGGED: the window offset up to which the piece lies inside the row (beyond: the row's last piece, and zeros).
  uint32_t x_lim[RAGGED ? Q : 1];
  const uint32_t k_bytes = static_cast<uint32_t>(a.K) * 2u;
#pragma unroll
  for (int it = 0; it < Q; ++it) {
    const int idx = tw + it * WS;
    uint32_t k_off;
    if constexpr (J == 2) {
      const int h = idx & 1, u = (idx >> 1) & 3, mt = idx >> 3;
      const int row = 8 * h + (i >> 1), piece = 2 * g + (i & 1);
      k_off = static_cast<uint32_t>(u * 4 * E + piece * 8) * 2u;
      x_off[it] = static_cast<uint32_t>(min(16 * mt + row, a.M - 1)) * ld_bytes + k_off;
      x_lds[it] = static_cast<uint32_t>(((mt * 4 + u) * PB + piece) * 256 + ((row + 8 * (piece & 1)) & 15) * 16);
    } else {
      const int pq = idx & (J - 1), u = (idx / J) & 3, mt = idx / (4 * J);
      k_off = static_cast<uint32_t>(u * 4 * E + pq * 32 + e3 * 8) * 2u;
      x_off[it] = static_cast<uint32_t>(min(16 * mt + r, a.M - 1)) * ld_bytes + k_off;
    }
    if constexpr (RAGGED) x_lim[it] = k_bytes - 16u - k_off;  // the launcher sees to K >= a window
  }
  u32x4 xr[2][Q];  // two windows on their way
  auto stage_load = [&](auto set, int gamma) {
    const uint32_t at_k = static_cast<uint32_t>(group_of(gamma)) * (16u * E * 2u);  // a window is 16 E values of k
    const char* const src = xbase + at_k;
#pragma unroll
    for (int it = 0; it < Q; ++it) {
      if constexpr (RAGGED) xr[decltype(set)::value][it] = *reinterpret_cast<const u32x4*>(xbase + (x_off[it] + min(at_k, x_lim[it])));
      else xr[decltype(set)::value][it] = *reinterpret_cast<const u32x4*>(src + x_off[it]);
    }
  };
  auto stage_store = [&](auto set, int gamma) {
    if constexpr (RAGGED) {
      // A window that reaches past K (no load is asked for in here: the wait counts stay what they are).
      const uint32_t at_k = static_cast<uint32_t>(group_of(gamma)) * (16u * E * 2u);
      if (at_k + 16u * E * 2u > k_bytes) {
#pragma unroll
        for (int it = 0; it < Q; ++it)
          if (at_k > x_lim[it]) xr[decltype(set)::value][it] = u32x4{0u, 0u, 0u, 0u};
      }
    }
    if constexpr (J == 2) {
      uint8_t* const dst = img + (gamma & 1) * kImage;
#pragma unroll
      for (int it = 0; it < Q; ++it) *reinterpret_cast<u32x4*>(dst + x_lds[it]) = xr[decltype(set)::value][it];
    } else {
      uint8_t* const dst = img + (gamma & 1) * kImage + tw * 1024 + lds_lane;
#pragma unroll
      for (int it = 0; it < Q; ++it) *reinterpret_cast<u32x4*>(dst + it * (WS * 1024)) = xr[decltype(set)::value][it];
    }
  };

  // This lane's weight loads: rows 4 q + g of the tile, chunk i of a group (256 contiguous bytes per 16 lanes).
  const uint8_t* const tile_w = a.w + static_cast<int64_t>(n0) * a.row_bytes;
  const uint8_t* const own_scale = a.scale + (static_cast<int64_t>(n0) + min(i, valid - 1)) * a.scale_row_bytes;  // NVFP4 only
  uint32_t row_off[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) row_off[q] = static_cast<uint32_t>(min(4 * q + g, valid - 1)) * static_cast<uint32_t>(a.row_bytes) + (RAGGED ? 0u : i * 16u);
  u32x4 raw[4][4];
  // NVFP4: a group's block scales of the lane's row i, the eight bytes under piece group g (one load a group and lane,
  // 32 contiguous bytes a row; a lane's fragments need bytes 8 u + 2 g, 8 u + 2 g + 1 of the row's 32 for step u, which
  // the wavefront's image hands round).
  u32x2 sc[4];
  auto issue_group = [&](auto slot, int gamma) {
    constexpr int SL = decltype(slot)::value;
    const int gq = group_of(gamma);
    // A group is 256 bytes of a row (RAGGED: the lane's chunk, or the row's last one).
    const uint32_t c = RAGGED ? min(static_cast<uint32_t>(gq) * 256u + i * 16u, static_cast<uint32_t>(a.row_bytes) - 16u) : static_cast<uint32_t>(gq) * 256u;
#pragma unroll
    for (int q = 0; q < 4; ++q) raw[SL][q] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(tile_w + (row_off[q] + c)));
    if constexpr (F == LX_W_NVFP4) {
      const uint32_t sc_at = RAGGED ? min(32u * gq + 8u * g, static_cast<uint32_t>(a.scale_row_bytes) - 8u) : 32u * gq + 8u * g;
      sc[SL] = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(own_scale + sc_at));
    }
  };
  // Row 4 q + g, chunk i goes into the wavefront's image; row i, chunk 4 s + g comes out.
  uint32_t put_at[4], get_at[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    put_at[q] = (4 * q + g) * 256 + ((i ^ (4 * q + g)) & 15) * 16;
    get_at[q] = i * 256 + (((4 * q + g) ^ i) & 15) * 16;
  }
  u32x4 wv[4];
  uint32_t wsc[4];
  auto to_image = [&](auto slot) {
    constexpr int SL = decltype(slot)::value;
#pragma unroll
    for (int q = 0; q < 4; ++q) *reinterpret_cast<u32x4*>(stage + put_at[q]) = raw[SL][q];
    if constexpr (F == LX_W_NVFP4) {
      uint8_t* const srow = stage + 4096 + i * kScalePitch;
      *reinterpret_cast<u32x2*>(srow + 8 * g) = sc[SL];
      asm volatile("" ::: "memory");  // the wavefront's LDS instructions run in order: the reads see the writes
#pragma unroll
      for (int u = 0; u < 4; ++u) wsc[u] = *reinterpret_cast<const uint16_t*>(srow + 8 * u + 2 * g);
    } else {
#pragma unroll
      for (int u = 0; u < 4; ++u) wsc[u] = 0u;
    }
  };

  // The activations first, then the weights: what is asked for first comes back first.
  stage_load(Tag<0>{}, 0);
  stage_load(Tag<1>{}, 1);
  issue_group(Tag<0>{}, 0);
  issue_group(Tag<1>{}, 1);
  issue_group(Tag<2>{}, 2);
  issue_group(Tag<3>{}, 3);
  stage_store(Tag<0>{}, 0);
  stage_load(Tag<0>{}, 2);
  to_image(Tag<0>{});
  uint32_t scales[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) scales[u] = wsc[u];
  // (A wavefront's LDS instructions run in the order they were issued: the reads see the writes before them.)
  asm volatile("" ::: "memory");
#pragma unroll
  for (int s = 0; s < 4; ++s) wv[s] = *reinterpret_cast<const u32x4*>(stage + get_at[s]);
  asm volatile("" ::: "memory");
  issue_group(Tag<0>{}, 4);

  // A fragment read: piece g * J + j of the step, this lane's row i of the activation tile.
  uint32_t rd_lane[J];
#pragma unroll
  for (int j = 0; j < J; ++j) rd_lane[j] = (g * J + j) * 256 + ((i + (J == 2 ? 8 * j : 4 * ((g * J + j) & 3))) & 15) * 16;

  // The slice at hand; a finished slice's sum waits in the wavefront's own area behind the images.
  f32x4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  // kRot: the wavefront's own [slice][mt][lane] behind the images; kSplit: the tile's, behind every wavefront's images.
  f32x4* const sums = SPLIT ? reinterpret_cast<f32x4*>(lds + W * kStage + W * 2 * kImage) + lane
                            : reinterpret_cast<f32x4*>(img + 2 * kImage) + wave * (a.S * MT * kWave) + lane;
  f32x4 total[MT];
  // Where the walk is in the row: group `at` of slice `slice`, which ends before group `slice_end`.
  int slice = first_slice, at = rot, slice_end = min(rot + gps, row_groups);

  // The gamma-th group the workgroup takes (its fragments are in wv). TAIL: one of the walk's last four groups, which ask
  // for nothing past the walk's end (a 16-group walk would otherwise load 5 groups and 3 windows more than it uses).
  auto one_group = [&](auto phase, int gamma, auto tail) {
    constexpr int P = decltype(phase)::value;  // gamma % 4
    constexpr bool TAIL = decltype(tail)::value;
    // Every wavefront has left window gamma - 1, and window gamma is complete (kSplit: the wavefront's own window, which
    // its own LDS instructions, run in order, have written).
    if constexpr (SPLIT) asm volatile("" ::: "memory");
    else __syncthreads();
    const uint8_t* const xb = img + (P & 1) * kImage;
    // The products of the group, pair by pair (a pair = load step s, matrix instruction j of the step). A pair's
    // activation fragments are asked for two pairs ahead, the next pair's weights are expanded under this pair's matrix
    // instructions, and the group's chores (the next window into the other image, the next group through the
    // wavefront's image, their loads) are spread over the pairs. The scheduler is held to this order: left alone it
    // asks for data right before its use.
    constexpr int kPairs = 4 * J, kAhead = 2;
    bf16x8 b[kAhead + 1][MT];
    auto read_pair = [&](int p, bf16x8 (&dst)[MT]) {
      const int s = p / J, j = p % J;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) dst[mt] = *reinterpret_cast<const bf16x8*>(xb + (mt * 4 + s) * (PB * 256) + rd_lane[j]);
    };
#pragma unroll
    for (int p = 0; p < kAhead; ++p) read_pair(p, b[p]);
    bf16x8 wf = weight_fragment<F>(wv[0], scales[0], 0);
    u32x4 wv_next[4];
#pragma unroll
    for (int p = 0; p < kPairs; ++p) {
      if (p + kAhead < kPairs) read_pair(p + kAhead, b[(p + kAhead) % (kAhead + 1)]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, b[p % (kAhead + 1)][mt], acc[mt], 0, 0, 0);
      if (p + 1 < kPairs) wf = weight_fragment<F>(wv[(p + 1) / J], scales[(p + 1) / J], (p + 1) % J);
      if (p == 0 && !(TAIL && P == 3)) {
        // The next window goes into the other image, the window after the next is asked for.
        stage_store(Tag<(P + 1) & 1>{}, gamma + 1);
        if (!TAIL || P == 0) stage_load(Tag<(P + 1) & 1>{}, gamma + 3);
      }
      if (p == 1 && !(TAIL && P == 3)) {
        // The next group goes into the wavefront's image; its registers take the group four ahead of it.
        to_image(Tag<(P + 1) & 3>{});
        if (!TAIL) issue_group(Tag<(P + 1) & 3>{}, gamma + 5);
      }
      if (p == kPairs - 1 && !(TAIL && P == 3)) {
        asm volatile("" ::: "memory");
#pragma unroll
        for (int s = 0; s < 4; ++s) wv_next[s] = *reinterpret_cast<const u32x4*>(stage + get_at[s]);
        asm volatile("" ::: "memory");
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (!(TAIL && P == 3)) {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        scales[u] = wsc[u];
        wv[u] = wv_next[u];
      }
    }
    // A slice ends.
    if (++at == slice_end) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        if constexpr (ROT || SPLIT) sums[(slice * MT + mt) * kWave] = acc[mt];
        else if constexpr (PART) {
          if (tile < n_tiles) static_cast<f32x4*>(a.partial)[((static_cast<int64_t>(slice) * n_tiles + tile) * MT + mt) * kWave + lane] = acc[mt];
        } else total[mt] = slice == 0 ? acc[mt] : total[mt] + acc[mt];
        acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
      }
      if (at == row_groups) {
        if constexpr (RAGGED) slice_end = -1;  // what follows holds nothing: no slice ends again
        else at = 0, slice = 0, slice_end = min(gps, row_groups);  // round to the row's start
      } else ++slice, slice_end = min(slice_end + gps, row_groups);
    }
  };
  for (int gamma = 0; gamma < groups - 4; gamma += 4) {
    one_group(Tag<0>{}, gamma, std::false_type{});
    one_group(Tag<1>{}, gamma + 1, std::false_type{});
    one_group(Tag<2>{}, gamma + 2, std::false_type{});
    one_group(Tag<3>{}, gamma + 3, std::false_type{});
  }
  // The last four groups, with the epilogue's row factors and biases asked for one group before the end: at the end they
  // would be a memory latency nothing hides, and asked for at the start they would hold registers through the walk.
  one_group(Tag<0>{}, groups - 4, std::true_type{});
  one_group(Tag<1>{}, groups - 3, std::true_type{});
  one_group(Tag<2>{}, groups - 2, std::true_type{});
  if constexpr (PART) {
    one_group(Tag<3>{}, groups - 1, std::true_type{});
    return;
  }
  const int nq = n0 + 4 * g;
  float rf[4], bs[4];
#pragma unroll
  for (int rr = 0; rr < 4; ++rr) {
    const int n = min(nq + rr, a.N - 1);
    rf[rr] = row_factor(F, a.scale, a.global, n);
    bs[rr] = a.bias ? load_as_f32(a.bias, a.bias_dtype, n) : 0.0f;
  }
  one_group(Tag<3>{}, groups - 1, std::true_type{});

  // The slices' sums in ascending order (kRot: the wavefront reads what it wrote itself: LDS keeps its order).
  asm volatile("" ::: "memory");
  if constexpr (SPLIT) {
    __syncthreads();
    if (wave != 0) return;
  }
  if constexpr (ROT || SPLIT) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      total[mt] = sums[mt * kWave];
      for (int sl = 1; sl < slices; ++sl) total[mt] += sums[(sl * MT + mt) * kWave];
    }
  }

  if (tile >= n_tiles) return;
  // A lane holds four consecutive outputs of one activation row: one 16-byte store where y allows it.
  const bool wide = a.y_dtype == LX_F32 && a.beta == 0.0f && nq + 3 < a.N && (a.ld_y & 3) == 0 && (reinterpret_cast<uintptr_t>(a.y) & 15) == 0;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + i;
    if (m >= a.M) continue;
    if (wide) {
      const float xs = a.act_scale ? a.act_scale[m] : 1.0f;
      f32x4 out;
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
        float t = (a.act_scale ? rf[rr] * xs : rf[rr]) * total[mt][rr];
        if (a.bias) t += bs[rr];
        out[rr] = a.alpha * t;
      }
      *reinterpret_cast<f32x4*>(static_cast<float*>(a.y) + static_cast<int64_t>(m) * a.ld_y + nq) = out;
    } else {
#pragma unroll
      for (int rr = 0; rr < 4; ++rr)
        if (nq + rr < a.N) write_out(a, m, nq + rr, total[mt][rr], rf[rr], bs[rr]);
    }
  }
}

// kSplit: W wavefronts on one tile, a.walk_slices slices each (the last wavefront what is left, at least one); every
// slice taken, none short, every wavefront's groups in fours.
template <int F, int W>
int launch_split(const GemmArgs& a, hipStream_t stream) {
  constexpr int J = Fmt<F>::kElems / 8, PB = 4 * J;
  const int MT = (a.M + 15) / 16;
  if (MT * 4 * J > 16) return kNotSupported;  // a lane holds every piece of its wavefront's window twice: past 32 the kernel spills
  const int gps = a.steps_per_wave >> 2;
  if (a.steps % a.steps_per_wave != 0 || a.walk_slices < 1) return kNotSupported;
  const int slices = a.steps / a.steps_per_wave, left = slices - (W - 1) * a.walk_slices;
  if (left < 1 || left > a.walk_slices || (a.walk_slices * gps) % 4 != 0 || (left * gps) % 4 != 0) return kNotSupported;
  const size_t lds = static_cast<size_t>(W) * stage_bytes<F>() + static_cast<size_t>(W) * 2 * MT * 4 * PB * 256 + static_cast<size_t>(slices) * MT * kWave * 16;
  if (lds > kLdsMax) return kNotSupported;
  const unsigned n_tiles = static_cast<unsigned>((a.N + kTileRows - 1) / kTileRows);
  auto launch = [&](auto kernel) {
    if (lds > 48 * 1024) allow_lds(reinterpret_cast<const void*>(kernel), kLdsMax);
    hipLaunchKernelGGL(kernel, dim3(n_tiles), dim3(W * kWave), lds, stream, a);
    return status_of(hipGetLastError());
  };
  auto with_mt = [&](auto mt_tag) {
    constexpr int M16 = decltype(mt_tag)::value;
    if constexpr (M16 * 4 * J > 16) return static_cast<int>(kNotSupported);
    else return launch(walk_kernel<F, M16, W, kSplit>);
  };
  switch (MT) {
    case 1: return with_mt(Tag<1>{});
    case 2: return with_mt(Tag<2>{});
    case 3: return with_mt(Tag<3>{});
    default: return with_mt(Tag<4>{});
  }
}

// ragged: rows that are not whole walks (the RAGGED kernels: from the row's start with the sums in registers, or single
// slices; no split over a workgroup's wavefronts).
template <int F, int W>
int launch_w(const GemmArgs& a, unsigned grid, bool ragged, hipStream_t stream) {
  constexpr int J = Fmt<F>::kElems / 8, PB = 4 * J;
  const int MT = (a.M + 15) / 16;
  if (a.walk_split) {
    if (ragged) return kNotSupported;
    if constexpr (W == 2 || W == 4) return launch_split<F, W>(a, stream);
    else return kNotSupported;
  }
  // A lane holds 2 MT 4 J / W staging pieces of 16 bytes: past 32 of them the kernel spills (measured 4 .. 20 x slower).
  if (MT * 4 * J / W > 16) return kNotSupported;
  // Eight wavefronts a workgroup have 256 registers each: room for four pieces (NVFP4 from 33 rows spills with six).
  if (W == 8 && MT * 4 * J / W > 4) return kNotSupported;
  if (MT * 4 * J % W != 0) return kNotSupported;  // the wavefronts share a window's pieces evenly
  const size_t images = static_cast<size_t>(W) * stage_bytes<F>() + 2 * static_cast<size_t>(MT) * 4 * PB * 256;
  const size_t with_sums = images + static_cast<size_t>(W) * a.S * MT * kWave * 16;
  const bool part = a.partial != nullptr;
  const bool rot = !part && !ragged && with_sums <= kLdsMax;
  const size_t lds = rot ? with_sums : images;
  if (lds > kLdsMax) return kNotSupported;
  unsigned parts = 1;
  if (part) {
    // Whole slices to a workgroup, their groups in fours.
    const int gps = a.steps_per_wave >> 2, slices = (a.steps + a.steps_per_wave - 1) / a.steps_per_wave;
    // (A short last slice is whole fours of groups when every slice is; the RAGGED kernels fill the last workgroup's walk up.)
    const bool short_last = a.steps % a.steps_per_wave != 0;
    if (a.walk_slices < 1 || (a.walk_slices * gps) % 4 != 0) return kNotSupported;
    if (!ragged && (short_last ? gps % 4 != 0 : slices % a.walk_slices != 0)) return kNotSupported;
    parts = static_cast<unsigned>((slices + a.walk_slices - 1) / a.walk_slices);
  }
  auto launch = [&](auto kernel) {
    if (lds > 48 * 1024) allow_lds(reinterpret_cast<const void*>(kernel), kLdsMax);
    hipLaunchKernelGGL(kernel, dim3(grid, parts), dim3(W * kWave), lds, stream, a);
    return status_of(hipGetLastError());
  };
  auto with_mt = [&](auto mt_tag) {
    constexpr int M16 = decltype(mt_tag)::value;
    if constexpr (M16 * 4 * J % W != 0) return static_cast<int>(kNotSupported);
    else if constexpr (W == 8) {
      if (!part) return static_cast<int>(kNotSupported);
      return ragged ? launch(walk_kernel<F, M16, W, kPart, true>) : launch(walk_kernel<F, M16, W, kPart>);
    } else if (part) {
      if constexpr (W == 4) return ragged ? launch(walk_kernel<F, M16, W, kPart, true>) : launch(walk_kernel<F, M16, W, kPart>);
      else return static_cast<int>(kNotSupported);
    } else if (ragged) return launch(walk_kernel<F, M16, W, kPlain, true>);
    else return rot ? launch(walk_kernel<F, M16, W, kRot>) : launch(walk_kernel<F, M16, W, kPlain>);
  };
  switch (MT) {
    case 1: return with_mt(Tag<1>{});
    case 2: return with_mt(Tag<2>{});
    case 3: return with_mt(Tag<3>{});
    default: return with_mt(Tag<4>{});
  }
}

template <int F>
bool launch_format(const GemmArgs& a, int W, int* status, hipStream_t stream) {
  constexpr int E = Fmt<F>::kElems;
  const int S = a.S, spw = a.steps_per_wave;
  if (a.M < 1 || a.M > 64 || S < 1 || spw % 8 != 0) return false;
  // Slices of whole batches, the row's last one as long as the row reaches (S may count empty ones behind it: a zero
  // added last changes no sum). Rows that are not groups in fours of whole steps take the RAGGED kernels: at least one
  // walk of four groups long, and NVFP4 in whole steps (a step's block scales are read as one).
  if ((a.steps + spw - 1) / spw > S) return false;
  const bool whole_steps = static_cast<int64_t>(a.steps) * 4 * E == a.K;
  const bool ragged = !whole_steps || a.steps % 16 != 0;
  if (ragged && (a.steps < 16 || (F == LX_W_NVFP4 && !whole_steps) || a.K % E != 0)) return false;
  if (static_cast<int64_t>(a.M) * a.xs.ld * 2 + static_cast<int64_t>(a.K) * 2 >= (int64_t{1} << 31)) return false;
  if (static_cast<int64_t>(kTileRows) * a.row_bytes >= (int64_t{1} << 31)) return false;
  // NVFP4: a group's scales are read eight bytes at a time.
  if (F == LX_W_NVFP4 && (reinterpret_cast<uintptr_t>(a.scale) % 8 != 0 || a.scale_row_bytes % 8 != 0)) return false;
  const int n_tiles = (a.N + kTileRows - 1) / kTileRows;
  const unsigned grid = static_cast<unsigned>((n_tiles + W - 1) / W);
  int st;
  switch (W) {
    case 8: st = launch_w<F, 8>(a, grid, ragged, stream); break;
    case 4: st = launch_w<F, 4>(a, grid, ragged, stream); break;
    case 2: st = launch_w<F, 2>(a, grid, ragged, stream); break;
    case 1: st = launch_w<F, 1>(a, grid, ragged, stream); break;
    default: return false;
  }
  if (st == kNotSupported) return false;
  *status = st;
  return true;
}

}  // namespace walk
}  // namespace dro
