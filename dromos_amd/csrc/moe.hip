// Routing and the few-token routed experts: lx_moe_route, lx_moe_experts_decode, lx_moe_experts_decode_bf16
// (contract: engine/cuda/kernels.h:203-209,495-507,606-611; CPU behaviour: engine/cpu/moe.cpp:163-329,343-397).
//
// Decode experts (T <= 8, top_k <= 8, so at most 64 (token, slot) pairs), two launches, no host round trip:
//   gate/up   a workgroup takes one expert's pairs (found from the step's ids with a ballot) and a block of
//             intermediate rows, and streams gate row i and up row I + i of that expert once for all the
//             group's tokens (stream_dot.h): inter[pair, i] = bf16(silu(g) * u).
//   down      one workgroup per (block of output rows, token): for the token's slots in order it streams
//             the expert's down rows against inter[pair] and adds w_k * c_k in slot order, so each output
//             is written once and its bits depend on nothing but the token.
#include "common.h"
#include "moe_common.h"
#include "stream_dot.h"

namespace dro {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;
constexpr int kMaxPairs = 64;

// ---- routing ---------------------------------------------------------------------------------------------

// A biased logit as an unsigned number that orders as the float does: a greater float is a greater number, -0 and +0
// are the same number, and a NaN is 0, below every other (-inf is 0x007fffff): it is picked before nothing.
__device__ __forceinline__ uint32_t order_key(float b) {
  const uint32_t u = __float_as_uint(b);
  const uint32_t k = (u & 0x80000000u) ? ~u : u | 0x80000000u;
  return b != b ? 0u : b == 0.0f ? 0x80000000u : k;
}

// One wavefront per token; a lane keeps its NPL logits (elements lane, lane + 64, ...) in registers, so the row
// is read once. E <= 64 * NPL. The picks: with few experts (NPL <= 4) every element is ranked against all the
// others (its rank among the biased logits, ties to the lower index, is its pick number); with many, top_k
// rounds of a wave-wide argmax.
template <int NPL>
__global__ void __launch_bounds__(kThreads) route_kernel(const float* __restrict__ logits, const float* __restrict__ bias,
                                                         int32_t* __restrict__ ids, float* __restrict__ weights,
                                                         float* __restrict__ entropy, float* __restrict__ confidence, int T,
                                                         int E, int top_k) {
  __shared__ float picked_logit[kWaves][64];
  const int lane = threadIdx.x & (kWave - 1), wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int64_t t = static_cast<int64_t>(blockIdx.x) * (blockDim.x / kWave) + wave;
  if (t >= T) return;
  const float* row = logits + t * E;
  float v[NPL], biased[NPL];
#pragma unroll
  for (int j = 0; j < NPL; ++j) {
    const int i = lane + j * kWave;
    v[j] = i < E ? row[i] : -INFINITY;
    // One f32 add, as the reference selects (a NaN or a missing element is never greater).
    biased[j] = i < E ? v[j] + (bias ? bias[i] : 0.0f) : -INFINITY;
  }
  float m = -INFINITY;
#pragma unroll
  for (int j = 0; j < NPL; ++j) m = fmaxf(m, v[j]);
  m = wave_max(m);
  float z = 0.0f, p_num[NPL];
#pragma unroll
  for (int j = 0; j < NPL; ++j) {
    p_num[j] = lane + j * kWave < E ? __expf(v[j] - m) : 0.0f;
    z += p_num[j];
  }
  z = wave_sum(z);
  float h = 0.0f;
#pragma unroll
  for (int j = 0; j < NPL; ++j) {
    if (lane + j * kWave < E) {
      const float p = p_num[j] / z;
      h -= p * __logf(p > 1e-9f ? p : 1e-9f);
    }
  }
  h = wave_sum(h);
  if (lane == 0) {
    entropy[t] = h;
    confidence[t] = 1.0f / z;  // the largest probability is exp(0) / z
  }
  if constexpr (NPL <= 4) {
    // Element (u, ~index) as one 64-bit number: another element is picked before this one exactly when its number
    // is the greater (a greater biased logit, or the same and a lower index).
    uint32_t key[NPL];
    uint64_t mine64[NPL];
    int rank[NPL];
#pragma unroll
    for (int j = 0; j < NPL; ++j) {
      key[j] = order_key(biased[j]);
      mine64[j] = static_cast<uint64_t>(key[j]) << 32 | static_cast<uint32_t>(~(lane + j * kWave));
      rank[j] = 0;
    }
#pragma unroll
    for (int j2 = 0; j2 < NPL; ++j2) {
#pragma unroll
      for (int l2 = 0; l2 < kWave; ++l2) {
        const uint64_t other = static_cast<uint64_t>(static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(key[j2]), l2))) << 32 |
                               static_cast<uint32_t>(~(l2 + j2 * kWave));
#pragma unroll
        for (int j = 0; j < NPL; ++j) rank[j] += other > mine64[j];
      }
    }
    int ranked = 0;
#pragma unroll
    for (int j = 0; j < NPL; ++j) {
      const int i = lane + j * kWave;
      // A NaN ranks nowhere (it is greater than nothing and nothing is greater than it): keep it out.
      const bool ok = i < E && biased[j] == biased[j];
      ranked += __popcll(__ballot(ok));
      if (ok && rank[j] < top_k) {
        ids[t * top_k + rank[j]] = i;
        picked_logit[wave][rank[j]] = v[j];
      }
    }
    // Fewer rankable logits than picks: the rest get the id E, as a search that finds nothing returns.
    if (lane >= ranked && lane < top_k) {
      ids[t * top_k + lane] = E;
      picked_logit[wave][lane] = NAN;
    }
  } else {
    // A picked element is struck from the candidates by its bit in `taken` (bit j: this lane's element j), not by
    // its value: an element whose logit is -inf can still be picked, once, lowest index first, as the reference's
    // search over the indices not yet picked does (engine/cpu/moe.cpp:367-381).
    uint64_t taken = 0;
    for (int r = 0; r < top_k; ++r) {
      float best = -INFINITY;
      int best_i = E;
#pragma unroll
      for (int j = 0; j < NPL; ++j) {
        const int i = lane + j * kWave;
        if (i < E && !((taken >> j) & 1) && (biased[j] > best || (biased[j] == best && i < best_i))) {
          best = biased[j];
          best_i = i;
        }
      }
#pragma unroll
      for (int off = 1; off < kWave; off <<= 1) {
        const float ov = __shfl_xor(best, off);
        const int oi = __shfl_xor(best_i, off);
        if (ov > best || (ov == best && oi < best_i)) {
          best = ov;
          best_i = oi;
        }
      }
#pragma unroll
      for (int j = 0; j < NPL; ++j) {
        if (lane + j * kWave == best_i) {
          ids[t * top_k + r] = best_i;
          picked_logit[wave][r] = v[j];
          taken |= 1ull << j;
        }
      }
      if (best_i >= E && lane == 0) {
        ids[t * top_k + r] = E;
        picked_logit[wave][r] = NAN;
      }
    }
  }
  __builtin_amdgcn_wave_barrier();
  __threadfence_block();
  // Weights: softmax over the picks of their unbiased logits, summed in pick order. Lane r takes pick r's logit.
  const float mine = lane < top_k ? picked_logit[wave][lane] : NAN;
  float lmax = -INFINITY;
  for (int r = 0; r < top_k; ++r) {
    const float p = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(mine), r));
    lmax = p > lmax ? p : lmax;
  }
  const float ex = __expf(mine - lmax);
  float esum = 0.0f;
  for (int r = 0; r < top_k; ++r) esum += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(ex), r));
  if (lane < top_k) weights[t * top_k + lane] = ex / esum;
}

// One intermediate row i per wavefront (i = blockIdx.x * waves + wave) of expert e for the cnt <= MT pairs at
// sorted positions first..: the pair (gate row i, up row I + i) is the wavefront's two streamed rows, all of
// their loads in flight before the activations are waited for. MT only sets how many activation rows share
// the pass; a row's arithmetic is the same for any MT. The whole workgroup calls it (it stages x).
template <int F, int U, int MT, bool ONE>
__device__ __forceinline__ void gate_up_rows(const DecodeArgs& a, float* lds, int e, int first, int cnt, const int* s_order,
                                             const int* s_rows) {
  const int steps = steps_for<F>(a.L);
  const int per_row = x_row_words<F, true>(steps);  // the packed bf16 image: the latent rows are bf16
  const RowBase<F> base(a.gu.data, a.gu.scale, a.L);
  const int64_t rb = base.rb, scale_row = base.scale_row;
  const int chunks = base.chunks;
  const int lane = threadIdx.x & (kWave - 1), wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int64_t stack_row0 = static_cast<int64_t>(e) * 2 * a.I;
  const int i = blockIdx.x * (blockDim.x / kWave) + wave;
  // The two rows' factors are asked for now: the epilogue should not wait for a load of its own.
  const int64_t my_gate_row = stack_row0 + min(i, a.I - 1);
  const float sg = stack_factor(F, a.gu, e, my_gate_row), su = stack_factor(F, a.gu, e, my_gate_row + a.I);
  auto rows_fn = [&](int ii, const uint8_t* (&rows)[2], const uint8_t* (&scales)[2], const float* (&x_image)[2]) {
    const int64_t gate_row = stack_row0 + min(ii, a.I - 1), up_row = gate_row + a.I;
    rows[0] = base.data + gate_row * rb;
    rows[1] = base.data + up_row * rb;
    scales[0] = base.scale + gate_row * scale_row;
    scales[1] = base.scale + up_row * scale_row;
    x_image[0] = lds;
    x_image[1] = lds;
  };
  auto done_fn = [&](int ii, float (&acc)[MT][2]) {
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      acc[m][0] = wave_sum(acc[m][0]);
      acc[m][1] = wave_sum(acc[m][1]);
    }
    if (lane == 0 && ii < a.I) {
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        if (m < cnt) {
          const float g = sg * acc[m][0], u = su * acc[m][1];
          const int pair = s_order ? s_order[first + m] : first + m;
          a.inter[static_cast<int64_t>(pair) * a.I + ii] = f32_to_bf16_bits(silu(g) * u);
        }
      }
    }
  };
  RowStreamer<F, MT, 2, U, true, ONE> st(chunks, 0, steps, per_row);
  if constexpr (F == LX_W_BF16X) st.set_bf16x(a.L);
  uint32_t* const image = reinterpret_cast<uint32_t*>(lds);
  if constexpr (MT == 1) {
    // Ask for x, then for the weights, and only then wait for x: loads return in order.
    const int token = s_rows ? s_rows[0] : first / a.top_k;
    const uint16_t* xrow = a.latent + static_cast<int64_t>(token) * a.L;
    // Vectors of the latent row a thread holds: what a one-batch row needs over 256 threads, four otherwise.
    constexpr int XV = ONE ? (U * Fmt<F>::kElems / 32 < 1 ? 1 : U * Fmt<F>::kElems / 32 > 4 ? 4 : U * Fmt<F>::kElems / 32) : 4;
    XRegs<XV> xr;
    stage_x_load<F>(xr, xrow, LX_BF16, a.L, a.L, steps);
    st.prefetch(rows_fn, i, 0, 1);
    if (xr.ready) stage_x_store_pairs<F>(xr, image, steps);
    else stage_x_pairs<F, 1>(image, xrow, a.L, nullptr, 1, a.L, steps);
  } else {
    st.prefetch(rows_fn, i, 0, 1);
    stage_x_pairs<F, MT>(image, a.latent, a.L, s_rows, cnt, a.L, steps);
  }
  __syncthreads();
  st.run(rows_fn, done_fn, i, 0, 1);
}

// grid = (I / wavefronts per workgroup, group slots); mt_cap (a power of two, the LDS image's rows) bounds a
// pass's pairs. One token: every slot is its own group; more: a slot whose pair is the first of its expert takes all
// of that expert's pairs, the other slots' workgroups leave at once.
// ONE: a row's steps fit one batch of U.
// SINGLE: one token (its own kernel: the many-row paths would set the registers of all).
template <int F, int U, bool ONE, bool SINGLE>
__global__ void __launch_bounds__(kThreads) decode_gate_up_kernel(const DecodeArgs a, int mt_cap) {
  extern __shared__ __align__(16) float lds[];
  if constexpr (SINGLE) {
    if (static_cast<int>(blockIdx.y) >= a.top_k) return;
    const int e = __builtin_amdgcn_readfirstlane(a.ids[blockIdx.y]);
    gate_up_rows<F, U, 1, ONE>(a, lds, e, blockIdx.y, 1, nullptr, nullptr);
    return;
  }
  // Slot blockIdx.y of the grid is pair blockIdx.y: the workgroup goes on if no earlier pair has that pair's expert, and
  // then takes every pair of the expert, in pair order. Each wavefront finds that from the step's ids (64 at most, one
  // per lane) with one comparison and a ballot; nothing is sorted and no table is read.
  __shared__ int s_rows[8], s_order[kMaxPairs];
  const int P = a.T * a.top_k, slot = blockIdx.y;
  if (slot >= P) return;
  const int lane = threadIdx.x & (kWave - 1);
  const int id = lane < P ? a.ids[lane] : -1 - lane;  // a lane past the pairs matches nothing
  const int e = __builtin_amdgcn_readlane(id, slot);
  const uint64_t members = __ballot(id == e);
  if (__ffsll(static_cast<unsigned long long>(members)) - 1 != slot) return;
  const int total = __popcll(members);
  if (threadIdx.x < kWave && ((members >> lane) & 1)) s_order[__popcll(members & ((1ull << lane) - 1))] = lane;
  // A group larger than the image (an expert repeated within a token) runs mt_cap pairs at a time.
  for (int first = 0; first < total; first += mt_cap) {
    const int cnt = min(mt_cap, total - first);
    __syncthreads();
    if (threadIdx.x < 8) s_rows[threadIdx.x] = static_cast<int>(threadIdx.x) < cnt ? s_order[first + threadIdx.x] / a.top_k : 0;
    __syncthreads();
    if (cnt <= 1) gate_up_rows<F, U, 1, ONE>(a, lds, e, first, cnt, s_order, s_rows);
    else if (cnt <= 2) gate_up_rows<F, U, 2, ONE>(a, lds, e, first, cnt, s_order, s_rows);
    else if (cnt <= 4) gate_up_rows<F, U, 4, ONE>(a, lds, e, first, cnt, s_order, s_rows);
    else gate_up_rows<F, U, 8, ONE>(a, lds, e, first, cnt, s_order, s_rows);
  }
}

// One workgroup per (l block, token): one output row l per wavefront. Its stream is the token's top_k
// experts' copies of row l, four at a time, each against its own slot's intermediate row, and
// out[t, l] = w0 * c0 + sum_{k >= 1} w_k * c_k in slot order (engine/cpu/moe.cpp:315-327), c_k = rowfactor * dot.
template <int F, int U>
__global__ void __launch_bounds__(kThreads) decode_down_kernel(const DecodeArgs a) {
  extern __shared__ __align__(16) float lds[];
  constexpr int R = 4;
  // Workgroup ids run over (l block / 8, token, l block % 8), the last fastest: consecutive ids land on different
  // dies, so the eight l blocks of a token spread over them while the tokens of one l block follow each other on
  // the same die, where an expert row that two tokens share is still in that die's L2.
  const int n_lblocks = (a.L + (blockDim.x / kWave) - 1) / (blockDim.x / kWave);
  const int t = (blockIdx.x >> 3) % a.T;
  const int lblock = (blockIdx.x / (8 * a.T)) * 8 + (blockIdx.x & 7);
  if (lblock >= n_lblocks) return;
  const int steps = steps_for<F>(a.I);
  const int per_row = x_row_words<F, true>(steps);  // the packed bf16 image: the intermediate rows are bf16
  const RowBase<F> base(a.dn.data, a.dn.scale, a.I);
  const int64_t rb = base.rb, scale_row = base.scale_row;
  const int chunks = base.chunks;
  const int lane = threadIdx.x & (kWave - 1), wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int top_k = a.top_k;
  const int l = lblock * (blockDim.x / kWave) + wave;
  const int lc = min(l, a.L - 1);

  // The token's experts, routing weights and row factors are asked for first: everything else hangs on the ids,
  // and the epilogue should not wait for a load of its own. Slot k's values sit in lane k.
  const int my_slot = min(lane, top_k - 1);
  const int my_e = a.ids[t * top_k + my_slot];
  const float my_weight = a.weights[t * top_k + my_slot];
  const float my_factor = stack_factor(F, a.dn, my_e, static_cast<int64_t>(my_e) * a.L + lc);
  // Group c holds slots 4c .. 4c + 3 (a slot past top_k repeats the last one and is not added).
  auto rows_fn = [&](int c, const uint8_t* (&rows)[R], const uint8_t* (&scales)[R], const float* (&x_image)[R]) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int k = min(c * R + r, top_k - 1);
      const int e = __builtin_amdgcn_readlane(my_e, k);
      const int64_t row = static_cast<int64_t>(e) * a.L + lc;
      rows[r] = base.data + row * rb;
      scales[r] = base.scale + row * scale_row;
      x_image[r] = lds + k * per_row;
    }
  };
  float o = 0.0f;
  auto done_fn = [&](int c, float (&acc)[1][R]) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int k = c * R + r;
      const float sum = wave_sum(acc[0][r]);
      if (k < top_k) {
        const float contrib = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_factor), k)) * sum;
        const float wc = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_weight), k)) * contrib;
        o = k == 0 ? wc : o + wc;
      }
    }
  };
  const int n_groups = (top_k + R - 1) / R;
  RowStreamer<F, 1, R, U, true> st(chunks, 0, steps, per_row);
  if constexpr (F == LX_W_BF16X) st.set_bf16x(a.I);
  // Ask for the intermediate rows, then for the weights, and only then wait for the rows: loads return in order.
  const uint16_t* const rows_of_t = a.inter + static_cast<int64_t>(t) * top_k * a.I;  // the token's top_k rows, in slot order
  XRowRegs xr;
  stage_rows_load<F>(xr, rows_of_t, a.I, nullptr, top_k, a.I, steps);
  st.prefetch(rows_fn, 0, 1, n_groups);
  if (xr.ready) stage_rows_store<F, 8>(xr, reinterpret_cast<uint32_t*>(lds), top_k, a.I, steps);
  else stage_x_pairs<F, 8>(reinterpret_cast<uint32_t*>(lds), rows_of_t, a.I, nullptr, top_k, a.I, steps);
  __syncthreads();
  st.run(rows_fn, done_fn, 0, 1, n_groups);
  if (lane == 0 && l < a.L) a.out[static_cast<int64_t>(t) * a.L + l] = o;
}

// Rows whose bytes cannot be streamed 16 at a time (K not a multiple of the chunk, or a misaligned stack):
// element-wise kernels with the same sums' structure (lane strides over k, one tree), one wavefront per output.
__global__ void __launch_bounds__(kThreads) decode_gate_up_plain_kernel(const DecodeArgs a, int type) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t item = static_cast<int64_t>(blockIdx.x) * kWaves + threadIdx.x / kWave;  // (pair, i)
  const int P = a.T * a.top_k;
  if (item >= static_cast<int64_t>(P) * a.I) return;
  const int pair = static_cast<int>(item / a.I), i = static_cast<int>(item % a.I);
  const int e = a.ids[pair], t = pair / a.top_k;
  const int64_t gate_row = static_cast<int64_t>(e) * 2 * a.I + i, up_row = gate_row + a.I;
  float g = 0.0f, u = 0.0f;
  for (int k = lane; k < a.L; k += kWave) {
    const float x = bf16_bits_to_f32(a.latent[static_cast<int64_t>(t) * a.L + k]);
    g = __builtin_fmaf(x, weight_element_any(type, a.gu.data, a.gu.scale, gate_row, k, a.L), g);
    u = __builtin_fmaf(x, weight_element_any(type, a.gu.data, a.gu.scale, up_row, k, a.L), u);
  }
  g = stack_factor(type, a.gu, e, gate_row) * wave_sum(g);
  u = stack_factor(type, a.gu, e, up_row) * wave_sum(u);
  if (lane == 0) a.inter[static_cast<int64_t>(pair) * a.I + i] = f32_to_bf16_bits(silu(g) * u);
}

__global__ void __launch_bounds__(kThreads) decode_down_plain_kernel(const DecodeArgs a, int type) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t item = static_cast<int64_t>(blockIdx.x) * kWaves + threadIdx.x / kWave;  // (t, l)
  if (item >= static_cast<int64_t>(a.T) * a.L) return;
  const int t = static_cast<int>(item / a.L), l = static_cast<int>(item % a.L);
  float o = 0.0f;
  for (int k = 0; k < a.top_k; ++k) {
    const int pair = t * a.top_k + k, e = a.ids[pair];
    const int64_t row = static_cast<int64_t>(e) * a.L + l;
    float s = 0.0f;
    for (int j = lane; j < a.I; j += kWave)
      s = __builtin_fmaf(bf16_bits_to_f32(a.inter[static_cast<int64_t>(pair) * a.I + j]),
                         weight_element_any(type, a.dn.data, a.dn.scale, row, j, a.I), s);
    const float wc = a.weights[pair] * (stack_factor(type, a.dn, e, row) * wave_sum(s));
    o = k == 0 ? wc : o + wc;
  }
  if (lane == 0) a.out[item] = o;
}

template <int F>
bool streamable(const Stack& s, int64_t K, int max_rows) {
  const int64_t rb = row_bytes<F>(K);
  const int steps = steps_for<F>(K);
  const bool vector_rows = F == LX_W_BF16X ? K % 8 == 0 && reinterpret_cast<uintptr_t>(s.data) % 8 == 0
                                           : rb % 16 == 0 && reinterpret_cast<uintptr_t>(s.data) % 16 == 0 &&
                                                 (F != LX_W_NVFP4 || reinterpret_cast<uintptr_t>(s.scale) % 2 == 0);
  return vector_rows &&
         static_cast<int64_t>(max_rows) * x_row_words<F, true>(steps) * 4 <= 128 * 1024;
}

template <class Kernel>
void allow_big_lds(Kernel kernel, size_t lds) {
  if (lds > 48 * 1024) allow_lds(reinterpret_cast<const void*>(kernel), 160 * 1024 - 1024);
}

template <int F, int U>
int launch_gate_up_u(const DecodeArgs& a, hipStream_t s) {
  const int P = a.T * a.top_k;
  // With distinct experts per token a group has at most T pairs; the LDS image holds that many rows.
  const int mt_cap = a.T <= 1 ? 1 : a.T <= 2 ? 2 : a.T <= 4 ? 4 : 8;
  const size_t lds = sizeof(float) * mt_cap * x_row_words<F, true>(steps_for<F>(a.L));
  auto launch = [&](auto kernel) {
    allow_big_lds(kernel, lds);
    hipLaunchKernelGGL(kernel, dim3((a.I + kWaves - 1) / kWaves, P), dim3(kThreads), lds, s, a, mt_cap);
    return status_of(hipGetLastError());
  };
  const bool one = steps_for<F>(a.L) <= U;
  if (a.T == 1) return one ? launch(decode_gate_up_kernel<F, U, true, true>) : launch(decode_gate_up_kernel<F, U, false, true>);
  return one ? launch(decode_gate_up_kernel<F, U, true, false>) : launch(decode_gate_up_kernel<F, U, false, false>);
}

template <int F>
int launch_gate_up(const DecodeArgs& a, hipStream_t s) {
  switch (batch_depth(steps_for<F>(a.L), 4)) {  // two rows a wavefront: four steps each at most
    case 4: return launch_gate_up_u<F, 4>(a, s);
    case 2: return launch_gate_up_u<F, 2>(a, s);
    default: return launch_gate_up_u<F, 1>(a, s);
  }
}

template <int F, int U>
int launch_down_u(const DecodeArgs& a, hipStream_t s) {
  const size_t lds = sizeof(float) * 8 * x_row_words<F, true>(steps_for<F>(a.I));
  auto kernel = decode_down_kernel<F, U>;
  allow_big_lds(kernel, lds);
  const int n_lblocks = (a.L + kWaves - 1) / kWaves;
  hipLaunchKernelGGL(kernel, dim3((n_lblocks + 7) / 8 * 8 * a.T), dim3(kThreads), lds, s, a);
  return status_of(hipGetLastError());
}

template <int F>
int launch_down(const DecodeArgs& a, hipStream_t s) {
  switch (batch_depth(steps_for<F>(a.I), 2)) {  // four rows a wavefront: two steps each at most
    case 2: return launch_down_u<F, 2>(a, s);
    default: return launch_down_u<F, 1>(a, s);
  }
}

int64_t round256(int64_t b) { return (b + 255) / 256 * 256; }

int gate_up_plain(const DecodeArgs& a, int type, hipStream_t s) {
  const int64_t items = static_cast<int64_t>(a.T) * a.top_k * a.I;
  hipLaunchKernelGGL(decode_gate_up_plain_kernel, dim3(static_cast<unsigned>((items + kWaves - 1) / kWaves)), dim3(kThreads), 0,
                     s, a, type);
  return status_of(hipGetLastError());
}

int down_plain(const DecodeArgs& a, int type, hipStream_t s) {
  const int64_t items = static_cast<int64_t>(a.T) * a.L;
  hipLaunchKernelGGL(decode_down_plain_kernel, dim3(static_cast<unsigned>((items + kWaves - 1) / kWaves)), dim3(kThreads), 0, s,
                     a, type);
  return status_of(hipGetLastError());
}

}  // namespace

// The decode experts on two stacks of any formats; `inter` holds bf16 [T * top_k, I].
int experts_decode(const void* latent, const int32_t* ids, const float* weights, const lx_weight& gate_up,
                   const lx_weight& down, float* out, void* inter, int T, int L, int I, int top_k, hipStream_t s) {
  DecodeArgs a{};
  a.latent = static_cast<const uint16_t*>(latent);
  a.ids = ids;
  a.weights = weights;
  a.gu = as_stack(gate_up);
  a.dn = as_stack(down);
  a.inter = static_cast<uint16_t*>(inter);
  a.out = out;
  a.T = T;
  a.L = L;
  a.I = I;
  a.top_k = top_k;
  auto can_stream = [](int type, const Stack& st, int64_t K) {
    switch (type) {
      case LX_W_BF16: return streamable<LX_W_BF16>(st, K, 8);
      case LX_W_BF16X: return streamable<LX_W_BF16X>(st, K, 8);
      case LX_W_INT8: return streamable<LX_W_INT8>(st, K, 8);
      case LX_W_FP8: return streamable<LX_W_FP8>(st, K, 8);
      default: return streamable<LX_W_NVFP4>(st, K, 8);
    }
  };
  int st;
  if (!can_stream(gate_up.type, a.gu, L)) {
    st = gate_up_plain(a, gate_up.type, s);
  } else {
    switch (gate_up.type) {
      case LX_W_BF16: st = launch_gate_up<LX_W_BF16>(a, s); break;
      case LX_W_BF16X: st = launch_gate_up<LX_W_BF16X>(a, s); break;
      case LX_W_INT8: st = launch_gate_up<LX_W_INT8>(a, s); break;
      case LX_W_FP8: st = launch_gate_up<LX_W_FP8>(a, s); break;
      default: st = launch_gate_up<LX_W_NVFP4>(a, s); break;
    }
  }
  if (st) return st;
  if (!can_stream(down.type, a.dn, I)) return down_plain(a, down.type, s);
  switch (down.type) {
    case LX_W_BF16: return launch_down<LX_W_BF16>(a, s);
    case LX_W_BF16X: return launch_down<LX_W_BF16X>(a, s);
    case LX_W_INT8: return launch_down<LX_W_INT8>(a, s);
    case LX_W_FP8: return launch_down<LX_W_FP8>(a, s);
    default: return launch_down<LX_W_NVFP4>(a, s);
  }
}

// lx_moe_route behind its validation (engine/cpu/moe.cpp:343-348).
int route(const float* logits, const float* selection_bias, int32_t* ids, float* weights, float* entropy, float* confidence, int T,
          int E, int top_k, hipStream_t s) {
  if (T <= 0) return kOk;
  if (top_k < 1 || top_k > 64 || top_k > E || !logits || !ids || !weights || !entropy || !confidence) return fail(kInvalid);
  if (E > 4096) return fail(kNotSupported);
  // One token: one wavefront, not a workgroup of sixteen of which fifteen leave at once.
  const int waves = T < kWaves ? T : kWaves;
  const dim3 grid((T + waves - 1) / waves), block(waves * kWave);
  if (E <= 64) hipLaunchKernelGGL(route_kernel<1>, grid, block, 0, s, logits, selection_bias, ids, weights, entropy, confidence, T, E, top_k);
  else if (E <= 128) hipLaunchKernelGGL(route_kernel<2>, grid, block, 0, s, logits, selection_bias, ids, weights, entropy, confidence, T, E, top_k);
  else if (E <= 256) hipLaunchKernelGGL(route_kernel<4>, grid, block, 0, s, logits, selection_bias, ids, weights, entropy, confidence, T, E, top_k);
  else if (E <= 1024) hipLaunchKernelGGL(route_kernel<16>, grid, block, 0, s, logits, selection_bias, ids, weights, entropy, confidence, T, E, top_k);
  else hipLaunchKernelGGL(route_kernel<64>, grid, block, 0, s, logits, selection_bias, ids, weights, entropy, confidence, T, E, top_k);
  return status_of(hipGetLastError());
}

int experts_plain(const DecodeArgs& a, int gu_type, int dn_type, hipStream_t s) {
  if (int st = gate_up_plain(a, gu_type, s)) return st;
  return down_plain(a, dn_type, s);
}

}  // namespace dro

using namespace dro;

extern "C" {

int lx_moe_route(const float* logits, const float* selection_bias, int32_t* ids, float* weights, float* entropy,
                 float* confidence, int T, int E, int top_k, void* stream) {
  return route(logits, selection_bias, ids, weights, entropy, confidence, T, E, top_k, as_stream(stream));
}

int lx_moe_experts_decode(const void* latent, const int32_t* ids, const float* weights, const lx_weight* gate_up,
                          const lx_weight* down, float* out, void* workspace, int T, int L, int I, int top_k, void* stream) {
  if (T <= 0) return kOk;
  if (T > 8 || top_k > 8) return fail(kInvalid);
  if (!latent || !ids || !weights || !out || L <= 0 || I <= 0 || top_k < 1) return fail(kInvalid);
  if (!gate_up || !down || !workspace) return fail(kInvalid);
  if (gate_up->type == LX_W_BF16X || down->type == LX_W_BF16X) {
    // engine/cpu/moe.cpp:528-533: both stacks encoded, or no kernel.
    if (gate_up->type != LX_W_BF16X || down->type != LX_W_BF16X) return fail(kNotSupported);
    return lx_moe_experts_bf16x(latent, ids, weights, gate_up->data, down->data, out, workspace, T, L, I, top_k, stream);
  }
  if (!valid_stack(*gate_up, L) || !valid_stack(*down, I)) return fail(kInvalid);
  return experts_decode(latent, ids, weights, *gate_up, *down, out, workspace, T, L, I, top_k, as_stream(stream));
}

int64_t lx_moe_decode_workspace_bytes(int T, int I, int top_k) {
  if (T <= 0 || I <= 0 || top_k <= 0) return 0;
  return round256(2 * static_cast<int64_t>(T) * top_k * I);  // the intermediate rows
}

int64_t lx_moe_bf16x_workspace_bytes(int T, int I, int top_k) { return lx_moe_decode_workspace_bytes(T, I, top_k); }

// The decode kernels on a pair of stacks of one format for any T, eight tokens a step (a token's output depends on
// nothing but the token, so the steps are independent).
static int experts_by_eight(const void* latent, const int32_t* ids, const float* weights, const lx_weight& gu, const lx_weight& dn,
                            float* out, void* workspace, int T, int L, int I, int top_k, void* stream) {
  hipStream_t s = as_stream(stream);
  for (int t0 = 0; t0 < T; t0 += 8) {
    const int n = T - t0 < 8 ? T - t0 : 8;
    const int st = experts_decode(static_cast<const uint16_t*>(latent) + static_cast<int64_t>(t0) * L, ids + static_cast<int64_t>(t0) * top_k,
                                  weights + static_cast<int64_t>(t0) * top_k, gu, dn, out + static_cast<int64_t>(t0) * L, workspace, n, L, I,
                                  top_k, s);
    if (st) return st;
  }
  return kOk;
}

// engine/cpu/moe.cpp:480-494. The kernels are the bf16 decode kernels with the encoded rows decoded in registers to
// the bf16 bits those load, so out equals lx_moe_experts_decode_bf16 on the original stacks to the bit.
int lx_moe_experts_bf16x(const void* latent, const int32_t* ids, const float* weights, const void* gate_up, const void* down,
                         float* out, void* workspace, int T, int L, int I, int top_k, void* stream) {
  if (T <= 0) return kOk;
  if (!latent || !ids || !weights || !out || L <= 0 || I <= 0 || top_k < 1) return fail(kInvalid);
  if (top_k > 8 || !gate_up || !down || !workspace || L >= bf16x::kMaxK || I >= bf16x::kMaxK) return fail(kInvalid);
  if ((reinterpret_cast<uintptr_t>(gate_up) | reinterpret_cast<uintptr_t>(down)) & 7) return fail(kInvalid);
  const lx_weight gu{LX_W_BF16X, gate_up, nullptr, 1.0f, nullptr}, dn{LX_W_BF16X, down, nullptr, 1.0f, nullptr};
  return experts_by_eight(latent, ids, weights, gu, dn, out, workspace, T, L, I, top_k, stream);
}

int lx_moe_experts_decode_bf16(const void* latent, const int32_t* ids, const float* weights, const void* gate_up,
                               const void* down, float* out, void* workspace, int T, int L, int I, int top_k, void* stream) {
  if (T <= 0) return kOk;
  if (top_k > 8 || !workspace) return fail(kInvalid);
  if (!latent || !ids || !weights || !out || !gate_up || !down || L <= 0 || I <= 0 || top_k < 1) return fail(kInvalid);
  const lx_weight gu{LX_W_BF16, gate_up, nullptr, 1.0f, nullptr}, dn{LX_W_BF16, down, nullptr, 1.0f, nullptr};
  return experts_by_eight(latent, ids, weights, gu, dn, out, workspace, T, L, I, top_k, stream);
}

}  // extern "C"
