// Shared by the library's source files: status codes, the wave-level helpers, and the exact decoders of
// the four weight formats. gfx950 only (wave64, OCP e4m3fn conversions in hardware).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "dromos_hip.h"

namespace dro {

constexpr int kOk = 0;
constexpr int kInvalid = 1;   // hipErrorInvalidValue
constexpr int kNoMemory = 2;  // hipErrorOutOfMemory
constexpr int kNotSupported = LX_ERR_NOT_SUPPORTED;

// Records the status for lx_rt_last_error and returns it.
int fail(int status);
// A HIP runtime status as this ABI's status (the numbering is shared), recorded when it is an error.
int status_of(hipError_t e);
// LX_BATCH_INVARIANT, read on every call (engine/cuda/common.cuh:66-73).
bool batch_invariant();
inline hipStream_t as_stream(void* s) { return static_cast<hipStream_t>(s); }
// Compute units of the current device (cached per device).
int compute_units();
// Lets `kernel` take up to `limit` bytes of dynamic LDS on the current device. The runtime is asked once per
// (device, kernel) and thread; later calls cost a table lookup.
void allow_lds(const void* kernel, int limit);

// The variant table (runtime.hip): the K split registered for (kernel, M bucket, N, K), or -1.
int tuned_variant(const char* kernel, int M, int N, int K);

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x8 __attribute__((ext_vector_type(8)));

constexpr int kWave = 64;

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// Round to nearest even; a NaN keeps its sign and gets a quiet bit (engine/cpu/cpu.h:47-52).
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return static_cast<uint16_t>(u >> 16);
}

__device__ __forceinline__ float load_as_f32(const void* p, int dtype, int64_t i) {
  return dtype == LX_BF16 ? bf16_bits_to_f32(static_cast<const uint16_t*>(p)[i]) : static_cast<const float*>(p)[i];
}
__device__ __forceinline__ void store_from_f32(void* p, int dtype, int64_t i, float v) {
  if (dtype == LX_BF16) static_cast<uint16_t*>(p)[i] = f32_to_bf16_bits(v);
  else static_cast<float*>(p)[i] = v;
}

// e4m3fn -> f32 in hardware (exact; 0x7f / 0xff are NaN). SEL picks the byte of the word.
template <int SEL>
__device__ __forceinline__ float e4m3_byte_to_f32(uint32_t word) {
  return __builtin_amdgcn_cvt_f32_fp8(word, SEL);
}
// e2m1 code -> f32, exact: {0, .5, 1, 1.5, 2, 3, 4, 6} with bit 3 the sign.
__device__ __forceinline__ float e2m1_to_f32(uint32_t code) {
  // The magnitude's three bits are an exponent field of two bits over one mantissa bit: as the top of
  // a float they read (1 + m / 2) * 2^(e - 127), and code 1 (e = 0, m = 1) is the one subnormal, 0.5.
  const uint32_t mag = code & 7u;
  const float normal = __uint_as_float((mag << 22) + (126u << 23));  // e >= 1: exponent e - 1 + 127
  const float v = mag >= 2u ? normal : (mag ? 0.5f : 0.0f);
  return (code & 8u) ? -v : v;
}

// ---- wave reductions: one fixed tree, every lane ends with the same bits ---------------------------

template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}

// The two halves of an exchange across 16-lane rows (ROWS16: every lane gets its own value and that of the lane 16
// away) or across the halves of the wavefront (32 away), by gfx950's lane-swap instructions: vector ALU work, where a
// shuffle would go through the LDS pipeline and be waited for. In every lane {a, b} is {own, other} or {other, own}:
// callers combine them with a commutative operation.
template <bool ROWS16>
__device__ __forceinline__ void swap_halves(float v, float& a, float& b) {
  const uint32_t u = __float_as_uint(v);
  if constexpr (ROWS16) {
    const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    a = __uint_as_float(r[0]);
    b = __uint_as_float(r[1]);
  } else {
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    a = __uint_as_float(r[0]);
    b = __uint_as_float(r[1]);
  }
}

__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_move<0xB1>(v);   // quad_perm [1, 0, 3, 2]
  v += dpp_move<0x4E>(v);   // quad_perm [2, 3, 0, 1]
  v += dpp_move<0x141>(v);  // row_half_mirror: the other quad of the half row
  v += dpp_move<0x140>(v);  // row_mirror: the other half of the 16-lane row
  float a, b;
  swap_halves<true>(v, a, b);  // the lane 16 away
  v = a + b;
  swap_halves<false>(v, a, b);  // the lane 32 away
  return a + b;
}

// N wave sums at once (N = 2, 4, 8 or 16): lane l ends with the sum of v[l % N] over the wavefront, by wave_sum's
// tree. Where wave_sum adds a value and its partner's in every lane, two sums share the step: the lanes whose bit d is
// clear keep the first sum's pair, the others the second's, so the registers halve at every step and sixteen sums cost
// about fifty instructions instead of a hundred and sixty. The operands of every addition are those of wave_sum (a + b
// or b + a), so each sum has wave_sum's bits. (Partners are true xor partners here: lane ^ 4 through the LDS crossbar,
// lane ^ 8 by a rotation of the 16-lane row; wave_sum's mirrors pair the same partial sums only while every lane of a
// quad holds the same one.)
template <int N>
__device__ __forceinline__ float wave_sum_many(const float (&in)[N]) {
  static_assert(N == 2 || N == 4 || N == 8 || N == 16, "a power of two up to 16");
  const unsigned lane = threadIdx.x & (kWave - 1);
  float v[N];
#pragma unroll
  for (int i = 0; i < N; ++i) v[i] = in[i];
  auto xor1 = [](float x) { return dpp_move<0xB1>(x); };
  auto xor2 = [](float x) { return dpp_move<0x4E>(x); };
  auto xor4 = [](float x) { return __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(x), 0x101F)); };
  auto xor8 = [](float x) { return dpp_move<0x128>(x); };  // row_ror:8
  int n = N;
  auto step = [&](bool upper, auto partner) {
    if (n > 1) {
      // v[i] <- the pair sums of v[2 i] (lanes with the bit clear) and of v[2 i + 1] (lanes with it set)
#pragma unroll
      for (int i = 0; i < N / 2; ++i) {
        if (i < n / 2) {
          const float keep = upper ? v[2 * i + 1] : v[2 * i], send = upper ? v[2 * i] : v[2 * i + 1];
          v[i] = keep + partner(send);
        }
      }
      n /= 2;
    } else {
      v[0] += partner(v[0]);
    }
  };
  step((lane & 1u) != 0, xor1);
  step((lane & 2u) != 0, xor2);
  step((lane & 4u) != 0, xor4);
  step((lane & 8u) != 0, xor8);
  float a, b;
  swap_halves<true>(v[0], a, b);
  const float w = a + b;
  swap_halves<false>(w, a, b);
  return a + b;
}

__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_move<0xB1>(v));
  v = fmaxf(v, dpp_move<0x4E>(v));
  v = fmaxf(v, dpp_move<0x141>(v));
  v = fmaxf(v, dpp_move<0x140>(v));
  float a, b;
  swap_halves<true>(v, a, b);
  v = fmaxf(a, b);
  swap_halves<false>(v, a, b);
  return fmaxf(a, b);
}

// ---- the weight formats as a wave streams them --------------------------------------------------------
// A lane reads 16 bytes of a row at a time (one 128-bit load): kElems consecutive k. The decoders hand the
// values on as f32, exactly, without the row factor; NVFP4's block scale is applied to a block's partial sum
// by the caller (a block's 16 codes sit in two consecutive dwords of the lane's 16 bytes).

template <int F>
struct Fmt;
template <>
struct Fmt<LX_W_BF16> {
  static constexpr int kElems = 8;     // k per 16-byte chunk
  static constexpr int kBitsPerK = 16;
};
template <>
struct Fmt<LX_W_INT8> {
  static constexpr int kElems = 16;
  static constexpr int kBitsPerK = 8;
};
template <>
struct Fmt<LX_W_FP8> {
  static constexpr int kElems = 16;
  static constexpr int kBitsPerK = 8;
};
template <>
struct Fmt<LX_W_NVFP4> {
  static constexpr int kElems = 32;
  static constexpr int kBitsPerK = 4;
};

// LX_W_BF16X: eight values a lane and step, as bf16; a row record is a header and 192-byte blocks of 128 values
// (bf16x.h). A lane's loads are 8 bytes of sign|mantissa, 4 bytes of codes and the block's base exponent.
template <>
struct Fmt<LX_W_BF16X> {
  static constexpr int kElems = 8;
  static constexpr int kBitsPerK = 16;  // once decoded: the products are bf16's
};

// A dword as two bf16 (low half first). Taking the dword by value matters: a bit cast written directly on an
// element of a vector, `__builtin_bit_cast(bf16x2, v[i])`, has compiled to element 0 for every i.
__device__ __forceinline__ bf16x2 as_bf16x2(uint32_t d) { return __builtin_bit_cast(bf16x2, d); }

// The values of one dword of a row: 2 (bf16), 4 (int8, fp8) or 8 (nvfp4 codes, unscaled).
template <int F>
struct DwordVals {
  static constexpr int kCount = 32 / Fmt<F>::kBitsPerK;
};

template <int F>
__device__ __forceinline__ void decode_dword(uint32_t d, float* out);

template <>
__device__ __forceinline__ void decode_dword<LX_W_BF16>(uint32_t d, float* out) {
  out[0] = __uint_as_float(d << 16);
  out[1] = __uint_as_float(d & 0xffff0000u);
}
template <>
__device__ __forceinline__ void decode_dword<LX_W_INT8>(uint32_t d, float* out) {
  out[0] = static_cast<float>(static_cast<int>(static_cast<int8_t>(d)));
  out[1] = static_cast<float>(static_cast<int>(static_cast<int8_t>(d >> 8)));
  out[2] = static_cast<float>(static_cast<int>(static_cast<int8_t>(d >> 16)));
  out[3] = static_cast<float>(static_cast<int>(d) >> 24);
}
template <>
__device__ __forceinline__ void decode_dword<LX_W_FP8>(uint32_t d, float* out) {
  const f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8(d, false);
  const f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8(d, true);
  out[0] = lo.x;
  out[1] = lo.y;
  out[2] = hi.x;
  out[3] = hi.y;
}
template <>
__device__ __forceinline__ void decode_dword<LX_W_NVFP4>(uint32_t d, float* out) {
  // Two codes a byte, the low nibble first. The conversion's scale operand only takes a power of two, so
  // it is 1 here and the e4m3 block scale is applied by the caller.
  const f32x2 a = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(d, 1.0f, 0);
  const f32x2 b = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(d, 1.0f, 1);
  const f32x2 c = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(d, 1.0f, 2);
  const f32x2 e = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(d, 1.0f, 3);
  out[0] = a.x;
  out[1] = a.y;
  out[2] = b.x;
  out[3] = b.y;
  out[4] = c.x;
  out[5] = c.y;
  out[6] = e.x;
  out[7] = e.y;
}

// Bytes of one row of K values.
template <int F>
__host__ __device__ inline int64_t row_bytes(int64_t K) {
  return K * Fmt<F>::kBitsPerK / 8;
}
template <>
__host__ __device__ inline int64_t row_bytes<LX_W_BF16X>(int64_t K) {
  const int64_t blocks = (K + 127) / 128;
  return (4 * (2 + K / 2048) + blocks + 7) / 8 * 8 + 192 * blocks;
}
// The 16-byte (BF16X: eight-value) chunks a lane may take of a row of K values.
template <int F>
__host__ __device__ inline int chunks_of(int64_t K) {
  return static_cast<int>(F == LX_W_BF16X ? K / 8 : row_bytes<F>(K) / 16);
}
__host__ __device__ inline int64_t row_bytes_of(int type, int64_t K) {
  return type == LX_W_BF16 ? 2 * K : type == LX_W_NVFP4 ? K / 2 : K;
}

// The row factor of output row n: the row scale (INT8 / FP8), the global (NVFP4), or 1.
__device__ __forceinline__ float row_factor(int type, const void* scale, float global, int64_t n) {
  if (type == LX_W_INT8 || type == LX_W_FP8) return static_cast<const float*>(scale)[n];
  return type == LX_W_NVFP4 ? global : 1.0f;
}

// Element (n, k) of an [N, K] weight, exact, without the row factor (engine/cpu/quant.cpp:143-154).
__device__ __forceinline__ float weight_element(int type, const void* data, const void* scale, int64_t n, int64_t k,
                                                int64_t K) {
  switch (type) {
    case LX_W_BF16: return bf16_bits_to_f32(static_cast<const uint16_t*>(data)[n * K + k]);
    case LX_W_INT8: return static_cast<float>(static_cast<const int8_t*>(data)[n * K + k]);
    case LX_W_FP8: return e4m3_byte_to_f32<0>(static_cast<const uint8_t*>(data)[n * K + k]);
    default: {
      const uint32_t byte = static_cast<const uint8_t*>(data)[n * (K / 2) + k / 2];
      const uint32_t code = (k & 1) ? (byte >> 4) : (byte & 15u);
      return e2m1_to_f32(code) * e4m3_byte_to_f32<0>(static_cast<const uint8_t*>(scale)[n * (K / 16) + k / 16]);
    }
  }
}

// silu as the reference's CPU computes it (engine/cpu/cpu.h:68), with the device's exp.
__device__ __forceinline__ float silu(float v) { return v / (1.0f + expf(-v)); }

// quant.hip: the launch behind lx_quantize_act, arguments already validated.
int quantize_act_rows(const void* x, int x_dtype, int64_t ld_x, int math, void* q, int64_t ld_q, float* scale, void* block_scale,
                      int64_t ld_bs, int M, int K, hipStream_t stream);

// quant.hip: the rows of x as a quantised math sees them (quantised per row, their exact values back as bf16 rows
// xhat [M, K], the per-row scales apart); q is scratch of M * (K + K / 16) bytes.
int act_images(const void* x, int x_dtype, int64_t ld_x, int math, uint8_t* q, uint16_t* xhat, float* scale, int M, int K,
               hipStream_t stream);

}  // namespace dro
