// Routed experts for any number of tokens on the matrix cores: lx_moe_experts_grouped, lx_moe_experts
// (contract: engine/cuda/kernels.h:220-225,495-511; CPU behaviour: engine/cpu/moe.cpp:163-329,546-581).
//
// Four launches, no host round trip (the grid sizes depend on T, top_k, E only, so the call can be captured):
//   group     one workgroup: counts the (token, slot) pairs per expert, prefix-sums the counts into the
//             expert offset table, lists the tiles (an expert's rows, 64 at a time), and places every pair
//             at a position inside its expert's range.
//   gate/up   one workgroup per (16 intermediate rows, tile): the gate tile and the up tile of the expert against
//             the tile's latent rows (gathered through the pair list) on the matrix cores (tile_mfma.h), SwiGLU
//             in the epilogue: inter[position, i] = bf16(silu(s_g * g) * (s_u * u)).
//   down      one workgroup per (16 output rows, tile): contrib[position, l] = s_l * down_l . inter[position].
//   sum       out[t, l] = w_0 * c_0 + sum_{k >= 1} w_k * c_k over the token's slots in order.
// Every pair's row is computed by the same arithmetic wherever it lands (the matrix instruction keeps rows
// apart, the K split depends on the shapes only), and the sum runs in slot order, so a token's bits depend on
// nothing but the token: not on the batch, the placement or the run.
#include <stdio.h>

#include <mutex>

#include "common.h"
#include "moe_common.h"
#include "tile_mfma.h"

namespace dro {
namespace {

constexpr int kMaxExperts = 1024;
constexpr int kTileTokens = 64;  // activation rows a tile holds at most
constexpr int kGroupedSplit = 4;  // wavefronts a tile at most: measured, four walking a tile in batches beat more with one batch each
// Wavefronts a SIMD the stage kernels are compiled for at least (512 registers a SIMD lane: 128 each at four, 168 at three), by
// what was measured (128 experts, 4096 x 1536, 32 and 64 tokens). NVFP4's nibble decode and block scales do not fit
// 128 registers: held to them it spilled 256 (gate/up) and 78 (down) and ran 470 us; with all it asks for (220, two
// wavefronts a SIMD) 390; at three a SIMD, a few dozen spilled in the wide activation tiles, 331. FP8 is 2% faster
// with three and no spills, INT8 4% faster with four and the few dozen spills of the widest activation tiles.
template <int F>
constexpr int grouped_waves() {
  return F == LX_W_NVFP4 || F == LX_W_FP8 ? 3 : 4;
}
#define DRO_GROUPED_KERNEL(F) \
  __global__ void __launch_bounds__(kGroupedSplit* kWave) __attribute__((amdgpu_waves_per_eu(grouped_waves<F>())))

struct Tables {
  int* offsets;      // [E + 1] first position of each expert
  int* order;        // [P] pair at each position
  int* pos;          // [P] position of each pair, -1 for an id outside [0, E)
  int* tile_expert;  // [max_tiles]
  int* tile_begin;   // [max_tiles] first position
  int* tile_rows;    // [max_tiles] 1 .. 64
  int* n_tiles;      // [1]
};

int max_tiles(int P, int E) { return (P < E ? P : E) + P / kTileTokens + 1; }

struct Layout {
  int64_t tables, inter, contrib, total;
  // The quantised maths: the latent rows' images and scales (by token), the intermediate rows' (by position), and the
  // quantiser's bytes.
  int64_t image1, scale1, image2, scale2, qbytes;
};

Layout layout(int T, int L, int I, int E, int top_k, int math) {
  const int64_t P = static_cast<int64_t>(T) * top_k;
  const int64_t ints = (E + 1) + 2 * P + 3 * max_tiles(static_cast<int>(P), E) + 1;
  auto up = [](int64_t b) { return (b + 255) / 256 * 256; };
  Layout l{};
  l.tables = 0;
  l.inter = up(ints * 4);
  l.contrib = l.inter + up(P * I * 2);
  l.total = l.contrib + up(P * L * 4);
  if (math != LX_MATH_BF16) {
    l.image1 = l.total;
    l.scale1 = l.image1 + up(static_cast<int64_t>(T) * L * 2);
    l.image2 = l.scale1 + up(static_cast<int64_t>(T) * 4);
    l.scale2 = l.image2 + up(P * I * 2);
    l.qbytes = l.scale2 + up(P * 4);
    const int64_t q1 = static_cast<int64_t>(T) * (L + L / 16), q2 = P * (I + I / 16);
    l.total = l.qbytes + up(q1 > q2 ? q1 : q2);
  }
  return l;
}

Tables tables_at(void* ws, int P, int E) {
  int* p = static_cast<int*>(ws);
  const int mt = max_tiles(P, E);
  Tables t;
  t.offsets = p;
  t.order = t.offsets + E + 1;
  t.pos = t.order + P;
  t.tile_expert = t.pos + P;
  t.tile_begin = t.tile_expert + mt;
  t.tile_rows = t.tile_begin + mt;
  t.n_tiles = t.tile_rows + mt;
  return t;
}

// Inclusive scan of v over the workgroup's kMaxExperts threads: every wavefront scans its 64 values in registers, the
// wavefronts' totals meet in LDS (two barriers a scan, where a scan through LDS alone took twenty).
__device__ __forceinline__ int block_scan(int v, int* buf) {
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  int x = v;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int y = __shfl_up(x, d);
    if (lane >= d) x += y;
  }
  if (lane == kWave - 1) buf[wave] = x;
  __syncthreads();
  int base = 0;
  for (int w = 0; w < wave; ++w) base += buf[w];
  __syncthreads();
  return x + base;
}

__global__ void __launch_bounds__(kMaxExperts) group_kernel(const int32_t* __restrict__ ids, int P, int E, Tables t) {
  __shared__ int count[kMaxExperts], cursor[kMaxExperts], buf[kMaxExperts];
  const int e = threadIdx.x;
  count[e] = 0;
  __syncthreads();
  for (int p = e; p < P; p += kMaxExperts) {
    const int id = ids[p];
    if (id >= 0 && id < E) atomicAdd(&count[id], 1);
  }
  __syncthreads();
  const int mine = count[e];
  const int begin = block_scan(mine, buf) - mine;
  if (e < E) t.offsets[e] = begin;
  if (e == E - 1) t.offsets[E] = begin + mine;
  cursor[e] = begin;
  __syncthreads();
  const int my_tiles = e < E ? (mine + kTileTokens - 1) / kTileTokens : 0;
  const int tile0 = block_scan(my_tiles, buf) - my_tiles;
  for (int j = 0; j < my_tiles; ++j) {
    t.tile_expert[tile0 + j] = e;
    t.tile_begin[tile0 + j] = begin + j * kTileTokens;
    t.tile_rows[tile0 + j] = min(kTileTokens, mine - j * kTileTokens);
  }
  if (e == kMaxExperts - 1) *t.n_tiles = tile0 + my_tiles;
  for (int p = e; p < P; p += kMaxExperts) {
    const int id = ids[p];
    if (id >= 0 && id < E) {
      const int g = atomicAdd(&cursor[id], 1);
      t.order[g] = p;
      t.pos[p] = g;
    } else {
      t.pos[p] = -1;
    }
  }
}

struct GroupedArgs {
  const uint16_t* latent;  // bf16 [T, L]: the latent rows, or their images under a quantised math
  const float* xs1;        // the latent rows' scales by token under a quantised math, else null
  const uint16_t* down_in; // bf16 [P, I] by position: the intermediate rows, or their images
  const float* xs2;        // the intermediate rows' scales by position, else null
  const float* weights;
  Stack gu, dn;
  Tables t;
  uint16_t* inter;  // bf16 [P, I] by position
  float* contrib;   // f32 [P, L] by position
  float* out;
  int T, L, I, top_k;
  int chunks, steps, steps_per_wave;  // of the stage's weight rows
  int64_t row_bytes, scale_row_bytes;
};

// gate/up for one (16 intermediate rows, tile of MT * 16 activation rows).
template <int F, int MT, bool WIDE>
__device__ __forceinline__ void gate_up_tile(const GroupedArgs& a, int e, int g0, int rows, f32x4* lds) {
  const int lane = threadIdx.x & (kWave - 1);
  const int i0 = blockIdx.x * kTileRows;
  const int64_t gate_row = static_cast<int64_t>(e) * 2 * a.I + i0, up_row = gate_row + a.I;
  const int valid = min(kTileRows, a.I - i0);
  const TileRows tiles[2] = {{a.gu.data + gate_row * a.row_bytes, a.gu.scale + gate_row * a.scale_row_bytes, valid},
                             {a.gu.data + up_row * a.row_bytes, a.gu.scale + up_row * a.scale_row_bytes, valid}};
  const void* xrow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int pair = a.t.order[g0 + min(mt * 16 + (lane & 15), rows - 1)];
    xrow[mt] = a.latent + static_cast<int64_t>(pair / a.top_k) * a.L;
  }
  mfma_tile<F, 2, MT, kXGlobalBf16, WIDE>(tiles, a.row_bytes, a.scale_row_bytes, a.chunks, a.steps, a.steps_per_wave, xrow, a.L, lds, blockDim.x / kWave, __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), [] {}, [&](int mt, int q, f32x4(&sums)[2]) {
    const int m = mt * 16 + (q & 15), i = i0 + 4 * (q >> 4);
    if (m >= rows) return;
    const int64_t stack_row = static_cast<int64_t>(e) * 2 * a.I + i;
    // The activation row's scale under a quantised math (engine/cpu/moe.cpp:254-268: g = s_g * (xs * sum)).
    const float xs = a.xs1 ? a.xs1[a.t.order[g0 + m] / a.top_k] : 1.0f;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      if (i + r < a.I) {
        const float g = stack_factor(F, a.gu, e, stack_row + r) * (xs * sums[0][r]);
        const float u = stack_factor(F, a.gu, e, stack_row + a.I + r) * (xs * sums[1][r]);
        a.inter[static_cast<int64_t>(g0 + m) * a.I + i + r] = f32_to_bf16_bits(silu(g) * u);
      }
    }
  });
}

// WIDE: NVFP4 block scales read eight bytes at a time (the launcher has checked that the stack allows it).
template <int F, bool WIDE>
DRO_GROUPED_KERNEL(F) grouped_gate_up_kernel(const GroupedArgs a) {
  extern __shared__ __align__(16) f32x4 lds4[];
  const int tile = blockIdx.y;
  if (tile >= *a.t.n_tiles) return;
  const int e = a.t.tile_expert[tile], g0 = a.t.tile_begin[tile], rows = a.t.tile_rows[tile];
  switch ((rows + 15) / 16) {
    case 1: gate_up_tile<F, 1, WIDE>(a, e, g0, rows, lds4); break;
    case 2: gate_up_tile<F, 2, WIDE>(a, e, g0, rows, lds4); break;
    case 3: gate_up_tile<F, 3, WIDE>(a, e, g0, rows, lds4); break;
    default: gate_up_tile<F, 4, WIDE>(a, e, g0, rows, lds4); break;
  }
}

template <int F, int MT, bool WIDE>
__device__ __forceinline__ void down_tile(const GroupedArgs& a, int e, int g0, int rows, f32x4* lds) {
  const int lane = threadIdx.x & (kWave - 1);
  const int l0 = blockIdx.x * kTileRows;
  const int64_t row = static_cast<int64_t>(e) * a.L + l0;
  const TileRows tiles[1] = {{a.dn.data + row * a.row_bytes, a.dn.scale + row * a.scale_row_bytes, min(kTileRows, a.L - l0)}};
  const void* xrow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) xrow[mt] = a.down_in + static_cast<int64_t>(g0 + min(mt * 16 + (lane & 15), rows - 1)) * a.I;
  mfma_tile<F, 1, MT, kXGlobalBf16, WIDE>(tiles, a.row_bytes, a.scale_row_bytes, a.chunks, a.steps, a.steps_per_wave, xrow, a.I, lds, blockDim.x / kWave, __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), [] {}, [&](int mt, int q, f32x4(&sums)[1]) {
    const int m = mt * 16 + (q & 15), l = l0 + 4 * (q >> 4);
    if (m >= rows) return;
    const int64_t stack_row = static_cast<int64_t>(e) * a.L + l;
    const float xs = a.xs2 ? a.xs2[g0 + m] : 1.0f;  // engine/cpu/moe.cpp:304-309: c = rf * (xs * sum)
#pragma unroll
    for (int r = 0; r < 4; ++r)
      if (l + r < a.L) a.contrib[static_cast<int64_t>(g0 + m) * a.L + l + r] = stack_factor(F, a.dn, e, stack_row + r) * (xs * sums[0][r]);
  });
}

template <int F, bool WIDE>
DRO_GROUPED_KERNEL(F) grouped_down_kernel(const GroupedArgs a) {
  extern __shared__ __align__(16) f32x4 lds4[];
  const int tile = blockIdx.y;
  if (tile >= *a.t.n_tiles) return;
  const int e = a.t.tile_expert[tile], g0 = a.t.tile_begin[tile], rows = a.t.tile_rows[tile];
  switch ((rows + 15) / 16) {
    case 1: down_tile<F, 1, WIDE>(a, e, g0, rows, lds4); break;
    case 2: down_tile<F, 2, WIDE>(a, e, g0, rows, lds4); break;
    case 3: down_tile<F, 3, WIDE>(a, e, g0, rows, lds4); break;
    default: down_tile<F, 4, WIDE>(a, e, g0, rows, lds4); break;
  }
}

// out[t, l] = w_0 * c_0 + sum_{k >= 1} w_k * c_k in slot order (engine/cpu/moe.cpp:315-327); a pair whose id
// was outside [0, E) contributes nothing.
__global__ void __launch_bounds__(256) grouped_sum_kernel(const GroupedArgs a) {
  const int64_t item = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (item >= static_cast<int64_t>(a.T) * a.L) return;
  const int t = static_cast<int>(item / a.L), l = static_cast<int>(item % a.L);
  float o = 0.0f;
  bool first = true;
  // Eight slots at a time: their positions and weights are asked for together, then their rows' elements, so a thread
  // waits for memory twice per eight slots and not twice per slot. (A slot past top_k repeats the last and is not added.)
  for (int k0 = 0; k0 < a.top_k; k0 += 8) {
    int g[8];
    float w[8], c[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int k = min(k0 + u, a.top_k - 1);
      g[u] = a.t.pos[t * a.top_k + k];
      w[u] = a.weights[t * a.top_k + k];
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) c[u] = a.contrib[static_cast<int64_t>(g[u] < 0 ? 0 : g[u]) * a.L + l];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (k0 + u < a.top_k && g[u] >= 0) {
        const float wc = w[u] * c[u];
        o = first ? wc : o + wc;
        first = false;
      }
    }
  }
  a.out[item] = o;
}

template <int F>
bool tileable(const Stack& s, int64_t K) {
  return row_bytes<F>(K) % 16 == 0 && reinterpret_cast<uintptr_t>(s.data) % 16 == 0 &&
         (F != LX_W_NVFP4 || reinterpret_cast<uintptr_t>(s.scale) % 2 == 0) && K % 8 == 0;
}

bool tileable_any(int type, const Stack& s, int64_t K) {
  switch (type) {
    case LX_W_BF16: return tileable<LX_W_BF16>(s, K);
    case LX_W_INT8: return tileable<LX_W_INT8>(s, K);
    case LX_W_FP8: return tileable<LX_W_FP8>(s, K);
    default: return tileable<LX_W_NVFP4>(s, K);
  }
}

template <int F, class Kernel>
int launch_stage(Kernel kernel, GroupedArgs a, int64_t K, int NT, int out_rows, int tiles, hipStream_t s) {
  a.row_bytes = row_bytes<F>(K);
  a.scale_row_bytes = F == LX_W_NVFP4 ? K / 16 : 0;
  a.chunks = static_cast<int>(a.row_bytes / 16);
  a.steps = load_steps_for<F>(K);
  int S = split_for<F>(K, NT);
  if (S > kGroupedSplit) S = kGroupedSplit;
  a.steps_per_wave = (a.steps + S - 1) / S;
  const int64_t P = static_cast<int64_t>(a.T) * a.top_k;
  const int mt_max = static_cast<int>(((P < kTileTokens ? P : kTileTokens) + 15) / 16);
  const size_t lds = tile_lds_bytes(S, NT, mt_max);
  if (lds > 48 * 1024) allow_lds(reinterpret_cast<const void*>(kernel), 144 * 1024);
  hipLaunchKernelGGL(kernel, dim3((out_rows + kTileRows - 1) / kTileRows, tiles), dim3(S * kWave), lds, s, a);
  return status_of(hipGetLastError());
}

}  // namespace

int64_t grouped_workspace_bytes(int T, int L, int I, int E, int top_k, int math) {
  if (T <= 0 || L <= 0 || I <= 0 || top_k <= 0 || E <= 0) return 0;
  return layout(T, L, I, E, top_k, math).total;
}

// math: LX_MATH_BF16, or a quantised math: then the latent rows are quantised per token and the intermediate rows per
// pair by lx_quantize_act's rule, their exact values go back into bf16 rows (act_images) for the same matrix-core
// kernels (exact products, f32 sums), and the rows' scales enter the epilogues as the reference applies them
// (engine/cpu/moe.cpp:241-312).
int experts_grouped(const void* latent, const int32_t* ids, const float* weights, const lx_weight& gate_up, const lx_weight& down,
                    float* out, void* workspace, int T, int L, int I, int E, int top_k, int math, hipStream_t s) {
  const int P = T * top_k;
  const Layout lay = layout(T, L, I, E, top_k, math);
  char* ws = static_cast<char*>(workspace);
  GroupedArgs a{};
  a.latent = static_cast<const uint16_t*>(latent);
  a.weights = weights;
  a.gu = as_stack(gate_up);
  a.dn = as_stack(down);
  a.t = tables_at(ws + lay.tables, P, E);
  a.inter = reinterpret_cast<uint16_t*>(ws + lay.inter);
  a.down_in = a.inter;
  a.contrib = reinterpret_cast<float*>(ws + lay.contrib);
  const bool quantised = math != LX_MATH_BF16;
  a.out = out;
  a.T = T;
  a.L = L;
  a.I = I;
  a.top_k = top_k;
  if (!tileable_any(gate_up.type, a.gu, L) || !tileable_any(down.type, a.dn, I) ||
      reinterpret_cast<uintptr_t>(latent) % 16 != 0) {
    // Shapes the tiles cannot read 16 bytes at a time: the element-wise experts (pairs independent, any T); they have
    // the weight-only and BF16 maths only.
    if (quantised) return fail(kNotSupported);
    DecodeArgs d{};
    d.latent = a.latent;
    d.ids = ids;
    d.weights = weights;
    d.gu = a.gu;
    d.dn = a.dn;
    d.inter = a.inter;
    d.out = out;
    d.T = T;
    d.L = L;
    d.I = I;
    d.top_k = top_k;
    return experts_plain(d, gate_up.type, down.type, s);
  }
  hipLaunchKernelGGL(group_kernel, dim3(1), dim3(kMaxExperts), 0, s, ids, P, E, a.t);
  if (int st = status_of(hipGetLastError())) return st;
  if (quantised) {
    uint16_t* const image1 = reinterpret_cast<uint16_t*>(ws + lay.image1);
    float* const scale1 = reinterpret_cast<float*>(ws + lay.scale1);
    if (int st = act_images(latent, LX_BF16, L, math, reinterpret_cast<uint8_t*>(ws + lay.qbytes), image1, scale1, T, L, s)) return st;
    a.latent = image1;
    a.xs1 = scale1;
  }
  const int tiles = max_tiles(P, E);
  int st;
  switch (gate_up.type) {
    case LX_W_BF16: st = launch_stage<LX_W_BF16>(grouped_gate_up_kernel<LX_W_BF16, false>, a, L, 2, I, tiles, s); break;
    case LX_W_INT8: st = launch_stage<LX_W_INT8>(grouped_gate_up_kernel<LX_W_INT8, false>, a, L, 2, I, tiles, s); break;
    case LX_W_FP8: st = launch_stage<LX_W_FP8>(grouped_gate_up_kernel<LX_W_FP8, false>, a, L, 2, I, tiles, s); break;
    default:
      st = wide_scales_fit(a.gu.scale, L / 16, static_cast<int>(row_bytes<LX_W_NVFP4>(L) / 16))
               ? launch_stage<LX_W_NVFP4>(grouped_gate_up_kernel<LX_W_NVFP4, true>, a, L, 2, I, tiles, s)
               : launch_stage<LX_W_NVFP4>(grouped_gate_up_kernel<LX_W_NVFP4, false>, a, L, 2, I, tiles, s);
      break;
  }
  if (st) return st;
  if (quantised) {
    // Every intermediate row is complete: quantise it again, per row (engine/cpu/moe.cpp:281-286). Positions past the
    // pairs routed to experts in range hold nothing and are never read.
    uint16_t* const image2 = reinterpret_cast<uint16_t*>(ws + lay.image2);
    float* const scale2 = reinterpret_cast<float*>(ws + lay.scale2);
    if ((st = act_images(a.inter, LX_BF16, I, math, reinterpret_cast<uint8_t*>(ws + lay.qbytes), image2, scale2, P, I, s))) return st;
    a.down_in = image2;
    a.xs2 = scale2;
  }
  switch (down.type) {
    case LX_W_BF16: st = launch_stage<LX_W_BF16>(grouped_down_kernel<LX_W_BF16, false>, a, I, 1, L, tiles, s); break;
    case LX_W_INT8: st = launch_stage<LX_W_INT8>(grouped_down_kernel<LX_W_INT8, false>, a, I, 1, L, tiles, s); break;
    case LX_W_FP8: st = launch_stage<LX_W_FP8>(grouped_down_kernel<LX_W_FP8, false>, a, I, 1, L, tiles, s); break;
    default:
      st = wide_scales_fit(a.dn.scale, I / 16, static_cast<int>(row_bytes<LX_W_NVFP4>(I) / 16))
               ? launch_stage<LX_W_NVFP4>(grouped_down_kernel<LX_W_NVFP4, true>, a, I, 1, L, tiles, s)
               : launch_stage<LX_W_NVFP4>(grouped_down_kernel<LX_W_NVFP4, false>, a, I, 1, L, tiles, s);
      break;
  }
  if (st) return st;
  const int64_t items = static_cast<int64_t>(T) * L;
  hipLaunchKernelGGL(grouped_sum_kernel, dim3(static_cast<unsigned>((items + 255) / 256)), dim3(256), 0, s, a);
  return status_of(hipGetLastError());
}

}  // namespace dro

using namespace dro;

extern "C" {

int lx_moe_experts_grouped(const void* latent, const int32_t* ids, const float* weights, const lx_weight* gate_up,
                           const lx_weight* down, lx_math math, float* out, void* workspace, int T, int L, int I, int E, int top_k,
                           void* stream) {
  if (T <= 0) return kOk;
  if (!latent || !ids || !weights || !out || L <= 0 || I <= 0 || top_k < 1) return fail(kInvalid);
  if (E <= 0 || !gate_up || !down) return fail(kInvalid);
  if (gate_up->type == LX_W_BF16X || down->type == LX_W_BF16X) return fail(kNotSupported);
  if (!valid_stack(*gate_up, L) || !valid_stack(*down, I)) return fail(kInvalid);
  switch (math) {  // engine/cpu/moe.cpp:555-569
    case LX_MATH_BF16: break;
    case LX_MATH_INT8:
      if (gate_up->type != LX_W_INT8 || down->type != LX_W_INT8) return fail(kNotSupported);
      break;
    case LX_MATH_FP8:
      if ((gate_up->type != LX_W_FP8 && gate_up->type != LX_W_NVFP4) || (down->type != LX_W_FP8 && down->type != LX_W_NVFP4))
        return fail(kNotSupported);
      break;
    case LX_MATH_FP4:
      if (gate_up->type != LX_W_NVFP4 || down->type != LX_W_NVFP4 || L % 16 || I % 16) return fail(kNotSupported);
      break;
    default: return fail(kInvalid);
  }
  if (E > kMaxExperts) return fail(kNotSupported);
  if (!workspace) return fail(kInvalid);
  return experts_grouped(latent, ids, weights, *gate_up, *down, out, workspace, T, L, I, E, top_k, math, as_stream(stream));
}

int64_t lx_moe_grouped_workspace_bytes(int T, int L, int I, int E, int top_k, lx_math math) {
  return grouped_workspace_bytes(T, L, I, E, top_k, math >= LX_MATH_INT8 && math <= LX_MATH_FP4 ? math : LX_MATH_BF16);
}

// The bf16-stack form without a workspace argument: the scratch is taken from and returned to the stream's
// memory pool (engine/cuda/kernels.h:220-225; the reference's kernel allocates the same way). The expert count
// is not an argument; kMaxExperts bounds the ids this call accepts.
// A decode step's few tokens take the decode kernels (one pass over each picked expert, no grouping tables): the
// result is then lx_moe_experts_decode_bf16's, and lx_moe_experts_bf16x's on the encoded stacks, to the bit, as the
// reference states of the three (engine/cuda/kernels.h:598-610). More tokens take the grouped kernels.
static bool few_tokens(int T, int top_k) { return T <= 8 && top_k <= 8; }

int lx_moe_experts(const void* latent, const int32_t* ids, const float* weights, const void* gate_up, const void* down, float* out,
                   int T, int L, int I, int top_k, void* stream) {
  if (T <= 0) return kOk;
  if (!latent || !ids || !weights || !out || L <= 0 || I <= 0 || top_k < 1 || !gate_up || !down) return fail(kInvalid);
  const lx_weight gu{LX_W_BF16, gate_up, nullptr, 1.0f, nullptr}, dn{LX_W_BF16, down, nullptr, 1.0f, nullptr};
  hipStream_t s = as_stream(stream);
  void* ws = nullptr;
  const bool few = few_tokens(T, top_k);
  const int64_t bytes = few ? lx_moe_decode_workspace_bytes(T, I, top_k) : grouped_workspace_bytes(T, L, I, kMaxExperts, top_k, LX_MATH_BF16);
  if (int st = status_of(hipMallocAsync(&ws, static_cast<size_t>(bytes), s))) return st;
  const int st = few ? experts_decode(latent, ids, weights, gu, dn, out, ws, T, L, I, top_k, s)
                     : experts_grouped(latent, ids, weights, gu, dn, out, ws, T, L, I, kMaxExperts, top_k, LX_MATH_BF16, s);
  const int fr = status_of(hipFreeAsync(ws, s));
  return st ? st : fr;
}

}  // extern "C"

// ---- lx_moe_experts for callers that cannot allocate ------------------------------------------------------
//
// The same kernels with their workspace (tables, intermediate rows, per-pair output rows) in a fixed array in device
// memory instead of the stream's pool. Every device the library runs on holds its own copy of the array at its own
// address until the process ends; the address is asked for once per device, on the first call there, with that
// device current, and only that address (never the array's name, which in host code is a stand-in and no device
// address) is handed to the kernels.
constexpr int64_t kScratchBytes = 8ll << 20;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

namespace dro {
namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_lock;
void* g_scratch_of[kMaxDevices];  // the array's address on each device, once asked for

// The array's address on the current device; null (and a recorded status) when the runtime cannot say.
void* scratch_of_current_device(int* status) {
  int dev = 0;
  if ((*status = status_of(hipGetDevice(&dev)))) return nullptr;
  if (dev < 0 || dev >= kMaxDevices) {
    *status = fail(kInvalid);
    return nullptr;
  }
  std::lock_guard<std::mutex> g(g_scratch_lock);
  if (!g_scratch_of[dev]) {
    void* ptr = nullptr;
    if ((*status = status_of(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch))))) return nullptr;
    g_scratch_of[dev] = ptr;
  }
  return g_scratch_of[dev];
}

}  // namespace
}  // namespace dro

extern "C" {

int lx_moe_experts_noalloc(const void* latent, const int32_t* ids, const float* weights, const void* gate_up, const void* down,
                           float* out, int T, int L, int I, int top_k, void* stream) {
  if (T <= 0) return kOk;
  if (!latent || !ids || !weights || !out || L <= 0 || I <= 0 || top_k < 1 || !gate_up || !down) return fail(kInvalid);
  const bool few = T <= 8 && top_k <= 8;  // as lx_moe_experts chooses
  const int64_t bytes = few ? lx_moe_decode_workspace_bytes(T, I, top_k) : grouped_workspace_bytes(T, L, I, kMaxExperts, top_k, LX_MATH_BF16);
  if (bytes > kScratchBytes) {
    fprintf(stderr, "lx_moe_experts_noalloc: T=%d L=%d I=%d top_k=%d needs %lld bytes of scratch, the fixed array holds %lld\n", T, L,
            I, top_k, static_cast<long long>(bytes), static_cast<long long>(kScratchBytes));
    return fail(kInvalid);
  }
  int st = kOk;
  void* const ws = scratch_of_current_device(&st);
  if (!ws) return st;
  const lx_weight gu{LX_W_BF16, gate_up, nullptr, 1.0f, nullptr}, dn{LX_W_BF16, down, nullptr, 1.0f, nullptr};
  if (few) return experts_decode(latent, ids, weights, gu, dn, out, ws, T, L, I, top_k, as_stream(stream));
  return experts_grouped(latent, ids, weights, gu, dn, out, ws, T, L, I, kMaxExperts, top_k, LX_MATH_BF16, as_stream(stream));
}

}  // extern "C"
