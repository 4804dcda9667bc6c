// Weight quantisers and the dequantiser: lx_quantize_w8, lx_quantize_weight, lx_dequantize_weight
// (contract: engine/cuda/kernels.h:248-251,513-523; byte-exact behaviour: engine/cpu/quant.cpp:12-56,66-140,
// 250-271). Load-time work: every rounding is done in software the way the CPU reference does it (IEEE f32
// divisions, ties to even), so the bytes are identical; speed matters little here.
#include <string.h>

#include "common.h"

namespace dro {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;

// e4m3fn -> f32 by the reference's formula for all 256 codes, 0x7f / 0xff included (they read as +-480
// there): normal codes rebase the exponent, subnormals are m * 2^-9 (engine/cpu/quant.cpp:12-18).
__device__ __forceinline__ float e4m3_decode(uint32_t b) {
  const uint32_t mag = b & 0x7fu;
  const float v = mag >= 8u ? __uint_as_float((mag << 20) + (120u << 23)) : static_cast<float>(mag) * 0x1p-9f;
  return (b & 0x80u) ? -v : v;
}

// f32 -> e4m3fn, nearest even, saturating at 448, NaN -> 0x7f with the sign (engine/cpu/quant.cpp:20-39).
__device__ __forceinline__ uint32_t e4m3_encode(float f) {
  uint32_t u = __float_as_uint(f);
  const uint32_t sign = (u >> 24) & 0x80u;
  u &= 0x7fffffffu;
  if (u > 0x7f800000u) return sign | 0x7fu;
  const float a = __uint_as_float(u);
  if (a >= 448.0f) return sign | 0x7eu;
  if (a < 0x1p-6f) return sign | static_cast<uint32_t>(static_cast<int>(rintf(a * 512.0f)));
  u += 0x7ffffu + ((u >> 20) & 1u);
  const int e = static_cast<int>(u >> 23) - 127 + 7;
  const uint32_t m = (u >> 20) & 7u;
  if (e > 15 || (e == 15 && m == 7u)) return sign | 0x7eu;
  return sign | (static_cast<uint32_t>(e) << 3) | m;
}

// Nearest e2m1 code, ties to the even code, saturating at 6, zero unsigned (engine/cpu/quant.cpp:47-56).
__device__ __forceinline__ uint32_t e2m1_encode(float x) {
  const float mag = fminf(fabsf(x), 6.0f);
  uint32_t idx = 0;
  idx += mag > 0.25f;
  idx += mag > 0.75f;
  idx += mag > 1.25f;
  idx += mag > 1.75f;
  idx += mag > 2.5f;
  idx += mag > 3.5f;
  idx += mag > 5.0f;
  // On the midpoint above an odd code, the even neighbour is the next one up.
  const float mid_above = idx == 1 ? 0.75f : idx == 3 ? 1.75f : idx == 5 ? 3.5f : -1.0f;
  if (mag == mid_above) ++idx;
  return idx | ((x < 0.0f && idx > 0u) ? 8u : 0u);
}

__device__ __forceinline__ float block_max(float v, float* shared) {
  v = wave_max(v);
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  __syncthreads();
  if (lane == 0) shared[wave] = v;
  __syncthreads();
  float m = shared[0];
  for (int i = 1; i < kWaves; ++i) m = fmaxf(m, shared[i]);
  return m;
}

// Per-token activation quantisation (engine/cuda/kernels.h:479-493; engine/cpu/quant.cpp:159-203): one workgroup per
// row. Unlike the weight quantisers it multiplies by a reciprocal: inv = qmax / a and q = round(x * inv); FP4:
// g = a / 2688, s_b = e4m3(a_b / (6 g)), r = 1 / (s_b g), code = e2m1(x * r). A zero row gets scale 1 and zeros.
__global__ void __launch_bounds__(kThreads) quantize_act_kernel(const void* __restrict__ x, int x_dtype, int64_t ld_x, int math,
                                                                uint8_t* __restrict__ q, int64_t ld_q, float* __restrict__ scale,
                                                                uint8_t* __restrict__ block_scale, int64_t ld_bs, int K) {
  __shared__ float shared[kWaves];
  const int64_t m = blockIdx.x, base = m * ld_x;
  float a = 0.0f;
  for (int k = threadIdx.x; k < K; k += kThreads) a = fmaxf(a, fabsf(load_as_f32(x, x_dtype, base + k)));
  a = block_max(a, shared);
  uint8_t* const row = q + m * ld_q;
  if (math == LX_MATH_INT8 || math == LX_MATH_FP8) {
    const float qmax = math == LX_MATH_INT8 ? 127.0f : 448.0f;
    const float inv = a > 0.0f ? qmax / a : 0.0f;
    for (int k = threadIdx.x; k < K; k += kThreads) {
      const float v = load_as_f32(x, x_dtype, base + k) * inv;
      if (math == LX_MATH_INT8) row[k] = static_cast<uint8_t>(static_cast<int8_t>(static_cast<int>(fminf(fmaxf(rintf(v), -127.0f), 127.0f))));
      else row[k] = static_cast<uint8_t>(e4m3_encode(v));
    }
    if (threadIdx.x == 0) scale[m] = a > 0.0f ? a / qmax : 1.0f;
    return;
  }
  const float g = a > 0.0f ? a / 2688.0f : 1.0f;
  if (threadIdx.x == 0) scale[m] = g;
  for (int b = threadIdx.x; b < K / 16; b += kThreads) {  // a thread per block of 16
    float v[16], amax = 0.0f;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      v[j] = load_as_f32(x, x_dtype, base + 16 * b + j);
      amax = fmaxf(amax, fabsf(v[j]));
    }
    const uint32_t s8 = e4m3_encode(amax / (6.0f * g));
    block_scale[m * ld_bs + b] = static_cast<uint8_t>(s8);
    const float d = e4m3_decode(s8) * g;
    const float r = d > 0.0f ? 1.0f / d : 0.0f;
#pragma unroll
    for (int p = 0; p < 8; ++p) {
      uint32_t lo = 0, hi = 0;
      if (d > 0.0f) {
        lo = e2m1_encode(v[2 * p] * r);
        hi = e2m1_encode(v[2 * p + 1] * r);
      }
      row[8 * b + p] = static_cast<uint8_t>(lo | (hi << 4));
    }
  }
}

// The INT8 / FP8 rules of quantize_act_kernel for rows that can be read 16 bytes at a time and fit a workgroup's
// registers (K <= 8 * kActVecs * kThreads): every value is read once, eight bf16 or two times four f32 per thread
// and pass, and eight codes are stored at a time. The same operations on the same values: the same bytes.
constexpr int kActVecs = 4;

template <bool XF32>
__global__ void __launch_bounds__(kThreads) quantize_act_rows_kernel(const void* __restrict__ x, int64_t ld_x, int math,
                                                                     uint8_t* __restrict__ q, int64_t ld_q, float* __restrict__ scale,
                                                                     int K) {
  __shared__ float shared[kWaves];
  const int64_t m = blockIdx.x;
  const char* const row = static_cast<const char*>(x) + m * ld_x * (XF32 ? 4 : 2);
  const int vecs = K >> 3;
  float v[kActVecs][8];
  float a = 0.0f;
#pragma unroll
  for (int u = 0; u < kActVecs; ++u) {
    const int vi = threadIdx.x + u * kThreads;
    const int vc = min(vi, vecs - 1);  // clamped: no predicated loads; a piece past the row is not stored
    if constexpr (XF32) {
      const f32x4 lo = *reinterpret_cast<const f32x4*>(row + vc * 32), hi = *reinterpret_cast<const f32x4*>(row + vc * 32 + 16);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v[u][j] = lo[j];
        v[u][4 + j] = hi[j];
      }
    } else {
      const u32x4 w = *reinterpret_cast<const u32x4*>(row + vc * 16);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v[u][2 * j] = __uint_as_float(w[j] << 16);
        v[u][2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
      }
    }
    if (vi < vecs) {
#pragma unroll
      for (int j = 0; j < 8; ++j) a = fmaxf(a, fabsf(v[u][j]));
    }
  }
  a = block_max(a, shared);
  const float qmax = math == LX_MATH_INT8 ? 127.0f : 448.0f;
  const float inv = a > 0.0f ? qmax / a : 0.0f;
  uint8_t* const out = q + m * ld_q;
#pragma unroll
  for (int u = 0; u < kActVecs; ++u) {
    const int vi = threadIdx.x + u * kThreads;
    if (vi < vecs) {
      uint32_t packed[2] = {0u, 0u};
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float t = v[u][j] * inv;
        const uint32_t code = math == LX_MATH_INT8 ? static_cast<uint32_t>(static_cast<int>(fminf(fmaxf(rintf(t), -127.0f), 127.0f))) & 0xffu
                                                   : e4m3_encode(t);
        packed[j >> 2] |= code << (8 * (j & 3));
      }
      *reinterpret_cast<uint2*>(out + vi * 8) = uint2{packed[0], packed[1]};
    }
  }
  if (threadIdx.x == 0) scale[m] = a > 0.0f ? a / qmax : 1.0f;
}

// One workgroup per row: absmax, then the row's codes. FP8 = false is INT8.
template <bool FP8>
__global__ void __launch_bounds__(kThreads) quantize_rows_kernel(const uint16_t* __restrict__ w, uint8_t* __restrict__ q,
                                                                 float* __restrict__ scale, int64_t rows, int cols) {
  __shared__ float shared[kWaves];
  for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
    const uint16_t* src = w + r * cols;
    float m = 0.0f;
    for (int c = threadIdx.x; c < cols; c += kThreads) m = fmaxf(m, fabsf(bf16_bits_to_f32(src[c])));
    const float amax = block_max(m, shared);
    const float qmax = FP8 ? 448.0f : 127.0f;
    const float s = amax > 0.0f ? amax / qmax : 1.0f;  // a zero row keeps scale 1
    if (threadIdx.x == 0) scale[r] = s;
    uint8_t* dst = q + r * cols;
    for (int c = threadIdx.x; c < cols; c += kThreads) {
      const float v = bf16_bits_to_f32(src[c]) / s;
      if (FP8) {
        dst[c] = static_cast<uint8_t>(e4m3_encode(fminf(fmaxf(v, -448.0f), 448.0f)));
      } else {
        const float i = fminf(fmaxf(rintf(v), -127.0f), 127.0f);
        dst[c] = static_cast<uint8_t>(static_cast<int8_t>(static_cast<int>(i)));
      }
    }
  }
}

// max |w| over the matrix into *out (f32 bits; non-negative floats order as their bits do).
__global__ void __launch_bounds__(kThreads) absmax_kernel(const uint16_t* __restrict__ w, int64_t n, unsigned* out) {
  __shared__ float shared[kWaves];
  float m = 0.0f;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < n; i += static_cast<int64_t>(gridDim.x) * kThreads)
    m = fmaxf(m, fabsf(bf16_bits_to_f32(w[i])));
  const float b = block_max(m, shared);
  if (threadIdx.x == 0) atomicMax(out, __float_as_uint(b));
}

// One thread per block of 16 values: its e4m3 scale and its eight bytes of codes.
__global__ void __launch_bounds__(kThreads) quantize_nvfp4_kernel(const uint16_t* __restrict__ w, uint8_t* __restrict__ q,
                                                                  uint8_t* __restrict__ scale, float global, int64_t blocks) {
  const int64_t b = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (b >= blocks) return;
  float v[16];
  float amax = 0.0f;
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    v[j] = bf16_bits_to_f32(w[16 * b + j]);
    amax = fmaxf(amax, fabsf(v[j]));
  }
  const uint32_t sb = e4m3_encode(amax / (6.0f * global));
  scale[b] = static_cast<uint8_t>(sb);
  const float eff = e4m3_decode(sb) * global;
#pragma unroll
  for (int p = 0; p < 8; ++p) {
    uint32_t lo = 0, hi = 0;
    if (eff > 0.0f) {
      lo = e2m1_encode(v[2 * p] / eff);
      hi = e2m1_encode(v[2 * p + 1] / eff);
    }
    q[8 * b + p] = static_cast<uint8_t>(lo | (hi << 4));  // the even k in the low nibble
  }
}

// out[n, k] = bf16(element(n, k) * rowfactor[n]), one thread per element.
__global__ void __launch_bounds__(kThreads) dequantize_kernel(int type, const uint8_t* __restrict__ data,
                                                              const uint8_t* __restrict__ scale, float global,
                                                              uint16_t* __restrict__ out, int64_t rows, int cols) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i >= rows * cols) return;
  const int64_t n = i / cols, k = i % cols;
  float e, f;
  if (type == LX_W_INT8) {
    e = static_cast<float>(static_cast<int8_t>(data[i]));
    f = reinterpret_cast<const float*>(scale)[n];
  } else if (type == LX_W_FP8) {
    e = e4m3_decode(data[i]);
    f = reinterpret_cast<const float*>(scale)[n];
  } else {
    const uint32_t byte = data[n * (cols / 2) + k / 2];
    const uint32_t code = (k & 1) ? (byte >> 4) : (byte & 15u);
    e = e2m1_to_f32(code) * e4m3_decode(scale[n * (cols / 16) + k / 16]);
    f = global;
  }
  out[i] = f32_to_bf16_bits(e * f);
}

unsigned grid_for(int64_t items, int64_t cap) {
  int64_t g = items < cap ? items : cap;
  return static_cast<unsigned>(g < 1 ? 1 : g);
}

int quantize_rows(bool fp8, const void* w, void* q, float* scale, int64_t rows, int cols, hipStream_t s) {
  const unsigned grid = grid_for(rows, 65535 * 16);
  if (fp8)
    hipLaunchKernelGGL(quantize_rows_kernel<true>, dim3(grid), dim3(kThreads), 0, s, static_cast<const uint16_t*>(w),
                       static_cast<uint8_t*>(q), scale, rows, cols);
  else
    hipLaunchKernelGGL(quantize_rows_kernel<false>, dim3(grid), dim3(kThreads), 0, s, static_cast<const uint16_t*>(w),
                       static_cast<uint8_t*>(q), scale, rows, cols);
  return status_of(hipGetLastError());
}

int quantize_nvfp4(const void* w, lx_weight* out, int64_t rows, int cols, hipStream_t s) {
  // The global needs the whole matrix's absmax on the host (it is returned in out->global): one small
  // device word, one synchronisation. Load-time only.
  unsigned* d_max = nullptr;
  if (int e = status_of(hipMalloc(&d_max, sizeof(unsigned)))) return e;
  int st = status_of(hipMemsetAsync(d_max, 0, sizeof(unsigned), s));
  const int64_t n = rows * cols;
  if (!st) {
    hipLaunchKernelGGL(absmax_kernel, dim3(grid_for((n + kThreads - 1) / kThreads, 4096)), dim3(kThreads), 0, s,
                       static_cast<const uint16_t*>(w), n, d_max);
    st = status_of(hipGetLastError());
  }
  unsigned bits = 0;
  if (!st) st = status_of(hipMemcpyAsync(&bits, d_max, sizeof(unsigned), hipMemcpyDeviceToHost, s));
  if (!st) st = status_of(hipStreamSynchronize(s));
  (void)hipFree(d_max);
  if (st) return st;
  float amax;
  memcpy(&amax, &bits, 4);
  volatile float divisor = 2688.0f;  // 448 * 6; an IEEE division on the host, as on the CPU backend
  const float global = amax / divisor;
  out->global = global;
  const int64_t blocks = n / 16;
  hipLaunchKernelGGL(quantize_nvfp4_kernel, dim3(static_cast<unsigned>((blocks + kThreads - 1) / kThreads)), dim3(kThreads),
                     0, s, static_cast<const uint16_t*>(w), static_cast<uint8_t*>(const_cast<void*>(out->data)),
                     static_cast<uint8_t*>(const_cast<void*>(out->scale)), global, blocks);
  return status_of(hipGetLastError());
}

}  // namespace
}  // namespace dro

namespace dro {

// The launch behind lx_quantize_act (arguments already validated), shared with the INT8 math of lx_gemm_w.
int quantize_act_rows(const void* x, int x_dtype, int64_t ld_x, int math, void* q, int64_t ld_q, float* scale, void* block_scale,
                      int64_t ld_bs, int M, int K, hipStream_t stream) {
  const int esize = x_dtype == LX_F32 ? 4 : 2;
  const bool fast = math != LX_MATH_FP4 && K % 8 == 0 && K <= 8 * kActVecs * kThreads && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
                    (ld_x * esize) % 16 == 0 && reinterpret_cast<uintptr_t>(q) % 8 == 0 && ld_q % 8 == 0;
  if (fast && x_dtype == LX_F32)
    hipLaunchKernelGGL(quantize_act_rows_kernel<true>, dim3(static_cast<unsigned>(M)), dim3(kThreads), 0, stream, x, ld_x, math,
                       static_cast<uint8_t*>(q), ld_q, scale, K);
  else if (fast)
    hipLaunchKernelGGL(quantize_act_rows_kernel<false>, dim3(static_cast<unsigned>(M)), dim3(kThreads), 0, stream, x, ld_x, math,
                       static_cast<uint8_t*>(q), ld_q, scale, K);
  else
    hipLaunchKernelGGL(quantize_act_kernel, dim3(static_cast<unsigned>(M)), dim3(kThreads), 0, stream, x, x_dtype, ld_x, math,
                       static_cast<uint8_t*>(q), ld_q, scale, static_cast<uint8_t*>(block_scale), ld_bs, K);
  return status_of(hipGetLastError());
}

namespace {

// xhat[m, k] = the value row m holds at k after its quantisation: the int8, the e4m3 value, or the e2m1 code times its
// block's e4m3 scale, as bf16 (exact: eight, four and six significant bits). One thread per eight values.
__global__ void __launch_bounds__(kThreads) act_values_kernel(const uint8_t* __restrict__ q, int64_t ld_q, const uint8_t* __restrict__ bs,
                                                              int64_t ld_bs, int math, uint16_t* __restrict__ xhat, int64_t ld_o, int M,
                                                              int K) {
  const int per_row = (K + 7) / 8;
  const int64_t item = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (item >= static_cast<int64_t>(M) * per_row) return;
  const int64_t m = item / per_row;
  const int k0 = static_cast<int>(item - m * per_row) * 8;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int k = k0 + j;
    if (k >= K) break;
    float v;
    if (math == LX_MATH_INT8) {
      v = static_cast<float>(static_cast<int8_t>(q[m * ld_q + k]));
    } else if (math == LX_MATH_FP8) {
      v = e4m3_decode(q[m * ld_q + k]);
    } else {
      const uint32_t byte = q[m * ld_q + (k >> 1)];
      v = e2m1_to_f32((k & 1) ? (byte >> 4) : (byte & 15u)) * e4m3_decode(bs[m * ld_bs + (k >> 4)]);
    }
    xhat[m * ld_o + k] = f32_to_bf16_bits(v);
  }
}

}  // namespace

// The rows of x [M, K] as a quantised math sees them: quantised per row by lx_quantize_act's rule for `math` (bytes into
// `q`, M * (K + K / 16) of them at most; scales into scale [M]) and their values written back as bf16 rows xhat [M, K]
// (exact). The matrix-core kernels then multiply xhat as they multiply any bf16 activations and apply the scales in
// their epilogues.
int act_images(const void* x, int x_dtype, int64_t ld_x, int math, uint8_t* q, uint16_t* xhat, float* scale, int M, int K,
               hipStream_t stream) {
  const int64_t ld_q = math == LX_MATH_FP4 ? K / 2 : K, ld_bs = K / 16;
  uint8_t* const bs = q + static_cast<int64_t>(M) * ld_q;
  if (int st = quantize_act_rows(x, x_dtype, ld_x, math, q, ld_q, scale, bs, ld_bs, M, K, stream)) return st;
  const int64_t items = static_cast<int64_t>(M) * ((K + 7) / 8);
  hipLaunchKernelGGL(act_values_kernel, dim3(static_cast<unsigned>((items + kThreads - 1) / kThreads)), dim3(kThreads), 0, stream, q, ld_q,
                     bs, ld_bs, math, xhat, static_cast<int64_t>(K), M, K);
  return status_of(hipGetLastError());
}

}  // namespace dro

using namespace dro;

extern "C" {

int lx_quantize_w8(const void* w, int8_t* q, float* scale, int64_t rows, int cols, void* stream) {
  if (rows <= 0) return kOk;
  if (cols <= 0 || !w || !q || !scale) return fail(kInvalid);
  return quantize_rows(false, w, q, scale, rows, cols, as_stream(stream));
}

int lx_quantize_weight(const void* w, lx_weight* out, int64_t rows, int cols, void* stream) {
  if (!out || !w) return fail(kInvalid);
  if (rows <= 0) return kOk;
  if (cols <= 0) return fail(kInvalid);
  void* data = const_cast<void*>(out->data);
  void* scale = const_cast<void*>(out->scale);
  switch (out->type) {
    case LX_W_INT8:
      if (!data || !scale) return fail(kInvalid);
      return quantize_rows(false, w, data, static_cast<float*>(scale), rows, cols, as_stream(stream));
    case LX_W_FP8:
      if (!data || !scale) return fail(kInvalid);
      return quantize_rows(true, w, data, static_cast<float*>(scale), rows, cols, as_stream(stream));
    case LX_W_NVFP4:
      if (!data || !scale || cols % 16 != 0) return fail(kInvalid);
      return quantize_nvfp4(w, out, rows, cols, as_stream(stream));
    case LX_W_BF16X: return fail(kNotSupported);
    default: return fail(kInvalid);  // bf16 is its own quantisation
  }
}

int lx_dequantize_weight(const lx_weight* w, void* out, int64_t rows, int cols, void* stream) {
  if (!w || !w->data || !out) return fail(kInvalid);
  if (rows <= 0) return kOk;
  if (cols <= 0) return fail(kInvalid);
  if (w->type == LX_W_BF16X) return fail(kNotSupported);
  if (w->type != LX_W_BF16 && w->type != LX_W_INT8 && w->type != LX_W_FP8 && w->type != LX_W_NVFP4) return fail(kInvalid);
  if (w->type != LX_W_BF16 && !w->scale) return fail(kInvalid);
  if (w->type == LX_W_NVFP4 && cols % 16 != 0) return fail(kInvalid);
  hipStream_t s = as_stream(stream);
  if (w->type == LX_W_BF16)
    return status_of(hipMemcpyAsync(out, w->data, static_cast<size_t>(2 * rows * cols), hipMemcpyDeviceToDevice, s));
  const int64_t n = rows * cols;
  hipLaunchKernelGGL(dequantize_kernel, dim3(static_cast<unsigned>((n + kThreads - 1) / kThreads)), dim3(kThreads), 0, s,
                     static_cast<int>(w->type), static_cast<const uint8_t*>(w->data), static_cast<const uint8_t*>(w->scale),
                     w->global, static_cast<uint16_t*>(out), rows, cols);
  return status_of(hipGetLastError());
}

int lx_quantize_act(const void* x, lx_dtype x_dtype, int ld_x, lx_math math, void* q, int ld_q, float* scale, void* block_scale,
                    int ld_bs, int M, int K, void* stream) {
  if (M <= 0) return kOk;
  if (!x || !q || !scale || K <= 0 || (x_dtype != LX_F32 && x_dtype != LX_BF16) || (M > 1 && ld_x < K)) return fail(kInvalid);
  if (math != LX_MATH_INT8 && math != LX_MATH_FP8 && math != LX_MATH_FP4) return fail(kInvalid);
  if (math == LX_MATH_FP4) {
    if (K % 16 != 0 || !block_scale || (M > 1 && (ld_q < K / 2 || ld_bs < K / 16))) return fail(kInvalid);
  } else if (M > 1 && ld_q < K) {
    return fail(kInvalid);
  }
  return quantize_act_rows(x, x_dtype, ld_x, math, q, ld_q, scale, block_scale, ld_bs, M, K, as_stream(stream));
}

}  // extern "C"
