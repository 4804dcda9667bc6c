// LX_W_BF16X: bf16 weights stored in 12 bits a value, every bit recoverable (the format and its entry points:
// engine/cuda/kernels.h:567-611; byte layout: engine/cuda/bf16x.cuh:13-27; CPU codec: engine/cpu/bf16x.cpp).
// This header holds the geometry of a row record and the device code that turns stored bytes back into bf16 bits.
//
// Why it works: the 8 exponent bits of neighbouring trained weights cluster. Take a span of 128 consecutive k of one
// row and call its largest exponent the span's top; nearly every value's exponent is top - c with 0 <= c <= 15. Such a
// value is stored as one byte (sign bit above the 7 mantissa bits) plus the nibble c. A value further than 15 below
// the top is an exception: its nibble is 0 and its true exponent is listed in the row's header.
//
// One row record, all rows of a matrix the same size (a multiple of 8 bytes), row r at r * row_bytes(K):
//   [0, 4S)            S exception words in ascending k, each k << 8 | exponent; unused words are kVacant. When a row
//                      has more than S exceptions, word 0 is 0x80000000 | q and the list lives in a spill record at
//                      q * 8 bytes from the row's first byte (behind all rows): u32 n, n words, kVacant.
//   [4S, 4S + B)       the tops of the B = ceil(K / 128) spans, one byte each; zero bytes up to the header size H
//   B spans of 192 bytes: bytes [0, 128) the sign|mantissa bytes of the span's values in k order; bytes [128, 192)
//                      sixteen u32 of nibbles: word g, byte b = value 8g + b (low nibble) and value 8g + 4 + b (high).
//                      Positions at or past K hold zero bytes and zero nibbles.
//   H = 4 * (2 + K / 2048) + B rounded up to 8; S = (H - B) / 4.
#pragma once

#include "common.h"

namespace dro {
namespace bf16x {

constexpr int kSpan = 128;
constexpr int kSpanBytes = 192;
constexpr int kNibbles = 128;  // where a span's nibble words start
constexpr uint32_t kVacant = 0xffffffffu;
constexpr uint32_t kSpilled = 0x80000000u;
constexpr int kMaxK = 1 << 23;  // an exception word keeps k in 23 bits

// The sizes that follow from K.
struct Geometry {
  int spans, header, slots;
  __host__ __device__ constexpr explicit Geometry(int K)
      : spans((K + kSpan - 1) / kSpan), header((4 * (2 + K / 2048) + spans + 7) & ~7), slots((header - spans) / 4) {}
  __host__ __device__ constexpr int tops_at() const { return 4 * slots; }
  __host__ __device__ constexpr int64_t row_bytes() const { return header + static_cast<int64_t>(kSpanBytes) * spans; }
};

__host__ __device__ constexpr int64_t row_bytes(int K) { return Geometry(K).row_bytes(); }
// A spill record of n exceptions: count word, the words, a kVacant terminator; a multiple of 8 bytes.
__host__ __device__ constexpr int64_t spill_bytes(int64_t n) { return ((n + 2) * 4 + 7) & ~int64_t{7}; }

// The exception list of the row record at `rec`: its words and how many to look at at most (a kVacant ends it early).
struct Exceptions {
  const uint32_t* words;
  uint32_t limit;
  __device__ __forceinline__ Exceptions(const uint8_t* rec, int slots) {
    const uint32_t* head = reinterpret_cast<const uint32_t*>(rec);
    const uint32_t first = head[0];
    if (first != kVacant && (first & kSpilled)) {
      const uint32_t* spill = reinterpret_cast<const uint32_t*>(rec + static_cast<int64_t>(first & ~kSpilled) * 8);
      words = spill + 1;
      limit = spill[0];
    } else {
      words = head;
      limit = static_cast<uint32_t>(slots);
    }
  }
  // e holds the exponents of values k0 .. k0 + 3, one a byte: those of them that are exceptions get theirs.
  __device__ __forceinline__ uint32_t fix(uint32_t e, uint32_t k0) const {
    for (uint32_t i = 0; i < limit; ++i) {
      const uint32_t word = words[i];
      if (word == kVacant) break;
      const uint32_t off = (word >> 8) - k0;
      if (off < 4u) {
        const uint32_t sh = off * 8u;
        e ^= (e ^ (word << sh)) & (0xffu << sh);
      }
    }
    return e;
  }
};

// bf16 bits of four values: `sm` their sign|mantissa bytes, `e` their exponents, one a byte (a span's top in every
// byte minus the values' nibbles: a nibble never exceeds the top it was taken from, so bytes do not borrow). A bf16's upper byte is the sign over
// exponent bits 7..1, its lower byte exponent bit 0 over the mantissa; v_perm_b32 zips the two byte rows (selectors
// 0..3 name bytes of the second operand, 4..7 of the first). Values 0, 1 land in .x, 2, 3 in .y, lower k in the low half.
__device__ __forceinline__ u32x2 quad_bits(uint32_t sm, uint32_t e) {
  // Each a bit-field insert: the mask's bits from sm, the others from the shifted exponents.
  const uint32_t upper = (sm & 0x80808080u) | ((e >> 1) & ~0x80808080u);
  const uint32_t lower = (sm & 0x7f7f7f7fu) | ((e << 7) & ~0x7f7f7f7fu);
  return u32x2{__builtin_amdgcn_perm(upper, lower, 0x05010400u), __builtin_amdgcn_perm(upper, lower, 0x07030602u)};
}

// One value (any k < K) of the row record at `rec`: its bf16 bits.
__device__ __forceinline__ uint16_t value_bits(const uint8_t* rec, int K, int k) {
  const Geometry g(K);
  const int span = k / kSpan, i = k % kSpan;
  const uint8_t* sp = rec + g.header + static_cast<int64_t>(span) * kSpanBytes;
  const uint32_t pair = sp[kNibbles + (i >> 3) * 4 + (i & 3)];
  const uint32_t nib = (i & 4) ? pair >> 4 : pair & 15u;
  const int lane = k & 3;
  uint32_t e = ((rec[g.tops_at() + span] - nib) & 0xffu) << (8 * lane);
  e = (Exceptions(rec, g.slots).fix(e, static_cast<uint32_t>(k - lane)) >> (8 * lane)) & 0xffu;
  const uint32_t sm = sp[i];
  return static_cast<uint16_t>((sm & 0x80u) << 8 | e << 7 | (sm & 0x7fu));
}

}  // namespace bf16x

// weight_element for every format, LX_W_BF16X included (data: the first row record).
__device__ __forceinline__ float weight_element_any(int type, const void* data, const void* scale, int64_t n, int64_t k, int64_t K) {
  if (type == LX_W_BF16X) {
    const int k_len = static_cast<int>(K);
    return bf16_bits_to_f32(bf16x::value_bits(static_cast<const uint8_t*>(data) + n * bf16x::row_bytes(k_len), k_len, static_cast<int>(k)));
  }
  return weight_element(type, data, scale, n, k, K);
}

}  // namespace dro
