/*
 * CPU oracle for the decode matrix-product path. TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain scalar C, the arithmetic of the reference's CPU backend for the
 * decode products: number formats, weight quantisers, the weight-streaming GEMV / skinny GEMM and the
 * routed experts. It is the checker that the GPU library's results are compared with. Nothing that
 * ships may call it: only the tests, the smoke check and the bench's cpu_baseline leg load it.
 *
 * It exports the same lx_* C ABI as the GPU library (include/dromos_hip.h), on host pointers, so one
 * test harness drives the GPU library, this oracle and (where it was built) the reference's own CPU
 * backend. Every function cites the reference file:line whose behaviour it follows. The code is
 * single-threaded unless built with -fopenmp (the loops over output rows carry pragmas).
 *
 * Parity status of each function (what pins it besides the compiled reference backend):
 *   bf16 / e4m3 / e2m1 codecs        pinned: exhaustive tables against torch.float8_e4m3fn and closed forms
 *   lx_quantize_w8 / _weight         pinned: known-answer ties/zero rows + torch IEEE-division references
 *   lx_dequantize_weight             pinned: closed-form dense values from the stored bytes
 *   lx_quantize_act                  pinned: the per-token rules in torch with IEEE f32 operations, FP4 tie / underflow cases
 *   lx_gemv* / lx_gemm_w / _skinny   pinned: float64 x @ W^T on the decoded values
 *   lx_gemm_w INT8 / FP8 / FP4 maths pinned: exact integer / float64 products of the quantised values, bit for bit
 *   lx_gemm_bf16, lx_spec_gemv_f32   pinned: float64 x @ W^T + bias
 *   lx_router_route                  pinned: equals lx_spec_gemv_f32 followed by lx_moe_route, word for word
 *   lx_moe_summary(_history)         pinned: float64 weighted sums of the expert embeddings, the history's closed form
 *   lx_moe_route                     pinned: stable sort of -(logit + bias) + float64 softmax, tie cases
 *   lx_moe_experts* (every math)     pinned: float64 experts with the bf16-rounded intermediate (quantised maths: on the
 *                                    quantised rows' exact values)
 *   lx_bf16x_* / *_bf16x             pinned: decode(encode(w)) == w over every exponent pattern incl. spilled rows, sizes
 *                                    by closed form, hand-built records; the products equal the bf16 products' bits
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))

enum { LX_F32 = 0, LX_BF16 = 1 };
enum { LX_W_BF16 = 0, LX_W_INT8 = 1, LX_W_FP8 = 2, LX_W_NVFP4 = 3, LX_W_BF16X = 4 };
enum { LX_MATH_BF16 = 0, LX_MATH_INT8 = 1, LX_MATH_FP8 = 2, LX_MATH_FP4 = 3 };
enum { ORC_OK = 0, ORC_INVALID = 1, ORC_NOMEM = 2, ORC_UNSUPPORTED = 801 };

/* The weight descriptor of engine/cuda/kernels.h:411-417. */
typedef struct {
  int type;
  const void* data;
  const void* scale;
  float global;
  const float* expert_global;
} lx_weight;

static __thread int g_last_error = 0;
static int fail(int status) {
  g_last_error = status;
  return status;
}

/* ---- number formats -------------------------------------------------------------------------- */

static float bits_to_f32(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static uint32_t f32_to_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}

/* bf16 is the top half of an f32 (engine/cpu/cpu.h:44). */
static float bf16_value(uint16_t h) { return bits_to_f32((uint32_t)h << 16); }

/* f32 -> bf16, nearest even; a NaN keeps its sign and gets a quiet payload bit (engine/cpu/cpu.h:47-52). */
static uint16_t bf16_round(float f) {
  uint32_t u = f32_to_bits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  uint32_t lsb = (u >> 16) & 1u;
  u += 0x7fffu + lsb;
  return (uint16_t)(u >> 16);
}

/* e4m3 "fn": bias 7, no infinities, subnormals m * 2^-9 (engine/cpu/quant.cpp:12-18). The two NaN
 * codes 0x7f / 0xff decode by the same formula (to +-480), as the reference's table does
 * (engine/cpu/kern/simd.h:77-85); no valid weight holds them. */
ORC_API float orc_e4m3_to_f32(uint8_t b) {
  int e = (b >> 3) & 15, m = b & 7;
  float v = e == 0 ? ldexpf((float)m, -9) : ldexpf(1.0f + (float)m / 8.0f, e - 7);
  return (b & 0x80) ? -v : v;
}

/* f32 -> e4m3, nearest even, saturating at 448, NaN -> 0x7f with the sign (engine/cpu/quant.cpp:20-39). */
ORC_API uint8_t orc_f32_to_e4m3(float f) {
  uint32_t u = f32_to_bits(f);
  uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
  u &= 0x7fffffffu;
  if (u > 0x7f800000u) return sign | 0x7f;
  float a = bits_to_f32(u);
  if (a >= 448.0f) return sign | 0x7e;
  if (a < 0.015625f) { /* below 2^-6: the subnormal grid, steps of 2^-9; 8 steps is the first normal */
    int steps = (int)rintf(a * 512.0f);
    return sign | (uint8_t)steps;
  }
  /* keep 3 mantissa bits: add half of the dropped field, plus the kept lsb for ties to even */
  u += 0x7ffffu + ((u >> 20) & 1u);
  int e = (int)(u >> 23) - 127 + 7;
  int m = (int)((u >> 20) & 7u);
  if (e > 15 || (e == 15 && m == 7)) return sign | 0x7e;
  return sign | (uint8_t)(e << 3) | (uint8_t)m;
}

static const float kE2m1[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};

/* e2m1 code (bit 3 = sign) -> f32 (engine/cpu/quant.cpp:41-45). */
ORC_API float orc_e2m1_to_f32(uint32_t code) {
  float v = kE2m1[code & 7u];
  return (code & 8u) ? -v : v;
}

/* Nearest e2m1 code: ties go to the even code, saturates at 6, zero carries no sign
 * (engine/cpu/quant.cpp:47-56). */
ORC_API uint32_t orc_f32_to_e2m1(float x) {
  float mag = fabsf(x);
  if (mag > 6.0f) mag = 6.0f;
  uint32_t idx = 0;
  for (int i = 0; i < 7; ++i) {
    float mid = 0.5f * (kE2m1[i] + kE2m1[i + 1]);
    if (mag > mid) idx = (uint32_t)i + 1;
    else if (mag == mid) { idx = (i & 1) ? (uint32_t)i + 1 : (uint32_t)i; break; }
    else break;
  }
  /* NaN compares false everywhere: idx stays 0, as in the reference */
  return idx | ((x < 0.0f && idx > 0) ? 8u : 0u);
}

static float load_f32(const void* p, int dtype, int64_t i) {
  return dtype == LX_BF16 ? bf16_value(((const uint16_t*)p)[i]) : ((const float*)p)[i];
}
static void store_f32(void* p, int dtype, int64_t i, float v) {
  if (dtype == LX_BF16) ((uint16_t*)p)[i] = bf16_round(v);
  else ((float*)p)[i] = v;
}
static int dtype_ok(int d) { return d == LX_F32 || d == LX_BF16; }

/* ---- weight quantisers (engine/cpu/quant.cpp:66-140, contract engine/cuda/kernels.h:248-251,513-518) ---- */

static float row_amax(const uint16_t* w, int64_t cols) {
  float m = 0.0f;
  for (int64_t c = 0; c < cols; ++c) m = fmaxf(m, fabsf(bf16_value(w[c])));
  return m;
}

static void quant_int8(const uint16_t* w, int8_t* q, float* scale, int64_t rows, int64_t cols) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    const uint16_t* src = w + r * cols;
    float amax = row_amax(src, cols);
    float s = amax > 0.0f ? amax / 127.0f : 1.0f; /* IEEE division; a zero row keeps scale 1 */
    scale[r] = s;
    for (int64_t c = 0; c < cols; ++c) {
      float v = rintf(bf16_value(src[c]) / s);
      v = fminf(fmaxf(v, -127.0f), 127.0f);
      q[r * cols + c] = (int8_t)(int)v;
    }
  }
}

static void quant_fp8(const uint16_t* w, uint8_t* q, float* scale, int64_t rows, int64_t cols) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    const uint16_t* src = w + r * cols;
    float amax = row_amax(src, cols);
    float s = amax > 0.0f ? amax / 448.0f : 1.0f;
    scale[r] = s;
    for (int64_t c = 0; c < cols; ++c) {
      float v = bf16_value(src[c]) / s;
      q[r * cols + c] = orc_f32_to_e4m3(fminf(fmaxf(v, -448.0f), 448.0f));
    }
  }
}

static void quant_nvfp4(const uint16_t* w, uint8_t* q, uint8_t* scale, float* global_out, int64_t rows, int64_t cols) {
  float amax = 0.0f;
  for (int64_t r = 0; r < rows; ++r) amax = fmaxf(amax, row_amax(w + r * cols, cols));
  const float global = amax / 2688.0f; /* 448 * 6 */
  *global_out = global;
  const int64_t blocks = cols / 16;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    for (int64_t b = 0; b < blocks; ++b) {
      float v[16], bmax = 0.0f;
      for (int j = 0; j < 16; ++j) {
        v[j] = bf16_value(w[r * cols + 16 * b + j]);
        bmax = fmaxf(bmax, fabsf(v[j]));
      }
      uint8_t sb = orc_f32_to_e4m3(bmax / (6.0f * global));
      scale[r * blocks + b] = sb;
      float eff = orc_e4m3_to_f32(sb) * global;
      for (int p = 0; p < 8; ++p) {
        uint32_t lo = 0, hi = 0;
        if (eff > 0.0f) {
          lo = orc_f32_to_e2m1(v[2 * p] / eff);
          hi = orc_f32_to_e2m1(v[2 * p + 1] / eff);
        }
        q[r * (cols / 2) + 8 * b + p] = (uint8_t)(lo | (hi << 4)); /* even k in the low nibble */
      }
    }
  }
}

ORC_API int lx_quantize_w8(const void* w, int8_t* q, float* scale, int64_t rows, int cols, void* stream) {
  (void)stream;
  if (rows <= 0) return ORC_OK;
  if (cols <= 0 || !w || !q || !scale) return fail(ORC_INVALID);
  quant_int8((const uint16_t*)w, q, scale, rows, cols);
  return ORC_OK;
}

ORC_API int lx_quantize_weight(const void* w, lx_weight* out, int64_t rows, int cols, void* stream) {
  (void)stream;
  if (!out || !w) return fail(ORC_INVALID);
  if (rows <= 0) return ORC_OK;
  if (cols <= 0) return fail(ORC_INVALID);
  void* data = (void*)out->data;
  void* scale = (void*)out->scale;
  switch (out->type) {
    case LX_W_INT8:
      if (!data || !scale) return fail(ORC_INVALID);
      quant_int8((const uint16_t*)w, (int8_t*)data, (float*)scale, rows, cols);
      return ORC_OK;
    case LX_W_FP8:
      if (!data || !scale) return fail(ORC_INVALID);
      quant_fp8((const uint16_t*)w, (uint8_t*)data, (float*)scale, rows, cols);
      return ORC_OK;
    case LX_W_NVFP4:
      if (!data || !scale || cols % 16 != 0) return fail(ORC_INVALID);
      quant_nvfp4((const uint16_t*)w, (uint8_t*)data, (uint8_t*)scale, &out->global, rows, cols);
      return ORC_OK;
    default: return fail(ORC_INVALID); /* bf16 is its own quantisation */
  }
}

/* Per-token activation quantisation (contract engine/cuda/kernels.h:479-493; engine/cpu/quant.cpp:159-203,273-292).
 * Unlike the weight quantisers it multiplies by a reciprocal: inv = qmax / a, q = round(x * inv); FP4 r = 1 / (s_b g).
 * Pinned bit for bit against oracle/_ref and the golden vectors (tests/test_oracle_quant.py, tests/test_golden.py). */
static void quant_act_row(const void* x, int x_dtype, int64_t base, int math, int K, uint8_t* q, float* scale, uint8_t* block_scale) {
  float a = 0.0f;
  for (int k = 0; k < K; ++k) a = fmaxf(a, fabsf(load_f32(x, x_dtype, base + k)));
  if (math == LX_MATH_INT8 || math == LX_MATH_FP8) {
    const float qmax = math == LX_MATH_INT8 ? 127.0f : 448.0f;
    const float inv = a > 0.0f ? qmax / a : 0.0f;
    for (int k = 0; k < K; ++k) {
      const float v = load_f32(x, x_dtype, base + k) * inv;
      if (math == LX_MATH_INT8) ((int8_t*)q)[k] = (int8_t)(int)fminf(fmaxf(rintf(v), -127.0f), 127.0f);
      else q[k] = orc_f32_to_e4m3(v);
    }
    *scale = a > 0.0f ? a / qmax : 1.0f;
    return;
  }
  const float g = a > 0.0f ? a / 2688.0f : 1.0f;
  *scale = g;
  for (int b = 0; b < K / 16; ++b) {
    float v[16], amax = 0.0f;
    for (int j = 0; j < 16; ++j) {
      v[j] = load_f32(x, x_dtype, base + 16 * b + j);
      amax = fmaxf(amax, fabsf(v[j]));
    }
    const uint8_t s8 = orc_f32_to_e4m3(amax / (6.0f * g));
    block_scale[b] = s8;
    const float d = orc_e4m3_to_f32(s8) * g;
    const float r = d > 0.0f ? 1.0f / d : 0.0f;
    for (int p = 0; p < 8; ++p) {
      uint32_t lo = 0, hi = 0;
      if (d > 0.0f) {
        lo = orc_f32_to_e2m1(v[2 * p] * r);
        hi = orc_f32_to_e2m1(v[2 * p + 1] * r);
      }
      q[8 * b + p] = (uint8_t)(lo | (hi << 4));
    }
  }
}

ORC_API int lx_quantize_act(const void* x, int x_dtype, int ld_x, int math, void* q, int ld_q, float* scale, void* block_scale,
                            int ld_bs, int M, int K, void* stream) {
  (void)stream;
  if (M <= 0) return ORC_OK;
  if (!x || !q || !scale || K <= 0 || !dtype_ok(x_dtype) || (M > 1 && ld_x < K)) return fail(ORC_INVALID);
  if (math != LX_MATH_INT8 && math != LX_MATH_FP8 && math != LX_MATH_FP4) return fail(ORC_INVALID);
  if (math == LX_MATH_FP4) {
    if (K % 16 != 0 || !block_scale || (M > 1 && (ld_q < K / 2 || ld_bs < K / 16))) return fail(ORC_INVALID);
  } else if (M > 1 && ld_q < K) {
    return fail(ORC_INVALID);
  }
  for (int64_t m = 0; m < M; ++m)
    quant_act_row(x, x_dtype, m * ld_x, math, K, (uint8_t*)q + m * ld_q, scale + m,
                  block_scale ? (uint8_t*)block_scale + m * ld_bs : NULL);
  return ORC_OK;
}

/* ---- LX_W_BF16X: bf16 in 12 bits a value (layout: engine/cuda/bf16x.cuh:13-27; codec: engine/cpu/bf16x.cpp) ----
 * A row record is S exception words, one top exponent per span of 128 values, zero bytes up to the header size,
 * then 192 bytes a span: 128 sign|mantissa bytes and 16 words of 4-bit codes (top - exponent). */
#define BX_SPAN 128
#define BX_SPAN_BYTES 192
#define BX_VACANT 0xffffffffu
#define BX_MAX_K (1 << 23)

static int bx_spans(int K) { return (K + BX_SPAN - 1) / BX_SPAN; }
static int bx_header(int K) { return (4 * (2 + K / 2048) + bx_spans(K) + 7) / 8 * 8; } /* bf16x.cuh:46 */
static int bx_slots(int K) { return (bx_header(K) - bx_spans(K)) / 4; }                 /* bf16x.cuh:47 */
static int64_t bx_row_bytes(int K) { return bx_header(K) + (int64_t)BX_SPAN_BYTES * bx_spans(K); }
static int64_t bx_spill_bytes(int64_t n) { return (4 * (n + 2) + 7) / 8 * 8; } /* bf16x.cpp:48 */
static int bx_k_ok(int K) { return K > 0 && K < BX_MAX_K; }

static uint32_t bx_get(const uint8_t* p) {
  uint32_t v;
  memcpy(&v, p, 4);
  return v;
}
static void bx_put(uint8_t* p, uint32_t v) { memcpy(p, &v, 4); }
static int bx_exponent(uint16_t v) { return (v >> 7) & 0xff; }

/* The largest exponent among values [k0, k0 + 128) of a row of K (bf16x.cpp:25-32). */
static int bx_top(const uint16_t* row, int K, int k0) {
  int top = 0;
  for (int k = k0; k < K && k < k0 + BX_SPAN; ++k)
    if (bx_exponent(row[k]) > top) top = bx_exponent(row[k]);
  return top;
}

/* Values whose exponent is more than 15 below their span's top (bf16x.cpp:35-46). */
static int64_t bx_exceptions(const uint16_t* row, int K) {
  int64_t n = 0;
  for (int k0 = 0; k0 < K; k0 += BX_SPAN) {
    int top = bx_top(row, K, k0);
    for (int k = k0; k < K && k < k0 + BX_SPAN; ++k) n += top - bx_exponent(row[k]) > 15;
  }
  return n;
}

/* Where byte and nibble of value i of a span live: the nibble of value i is in code byte 4 * (i / 8) + i % 4, the
 * low half for i % 8 < 4 (bf16x.cuh:22-25). */
static uint8_t* bx_code_byte(uint8_t* span, int i) { return span + 128 + 4 * (i / 8) + (i % 4); }

/* One row record at rec; its spill record (when n exceeds the slots) at rec + spill_off (bf16x.cpp:58-104). */
static void bx_encode_row(const uint16_t* row, int K, uint8_t* rec, int64_t n, int64_t spill_off) {
  const int S = bx_slots(K), H = bx_header(K), B = bx_spans(K);
  memset(rec, 0, (size_t)bx_row_bytes(K));
  for (int s = 0; s < S; ++s) bx_put(rec + 4 * s, BX_VACANT);
  uint8_t* list = rec;
  if (n > S) {
    uint8_t* sp = rec + spill_off;
    memset(sp, 0, (size_t)bx_spill_bytes(n));
    bx_put(rec, 0x80000000u | (uint32_t)(spill_off / 8));
    bx_put(sp, (uint32_t)n);
    bx_put(sp + 4 * (n + 1), BX_VACANT);
    list = sp + 4;
  }
  int64_t listed = 0;
  for (int b = 0; b < B; ++b) {
    uint8_t* span = rec + H + (int64_t)b * BX_SPAN_BYTES;
    const int top = bx_top(row, K, b * BX_SPAN);
    rec[4 * S + b] = (uint8_t)top;
    for (int i = 0; i < BX_SPAN && b * BX_SPAN + i < K; ++i) {
      const int k = b * BX_SPAN + i;
      const uint16_t v = row[k];
      span[i] = (uint8_t)(((v >> 8) & 0x80) | (v & 0x7f));
      int code = top - bx_exponent(v);
      if (code > 15) {
        bx_put(list + 4 * listed++, ((uint32_t)k << 8) | (uint32_t)bx_exponent(v));
        code = 0;
      }
      *bx_code_byte(span, i) |= (uint8_t)((i % 8) < 4 ? code : code << 4);
    }
  }
}

/* bf16 bits of value k of the row record at rec: the coded exponent unless an exception word names k (bf16x.cpp:162-193). */
static uint16_t bx_value(const uint8_t* rec, int K, int k) {
  const int S = bx_slots(K), b = k / BX_SPAN, i = k % BX_SPAN;
  const uint8_t* span = rec + bx_header(K) + (int64_t)b * BX_SPAN_BYTES;
  const uint8_t pair = *bx_code_byte((uint8_t*)span, i);
  uint32_t e = (uint32_t)(rec[4 * S + b] - ((i % 8) < 4 ? pair & 15 : pair >> 4)) & 0xffu;
  const uint8_t* list = rec;
  int64_t n = S;
  const uint32_t first = bx_get(rec);
  if (first != BX_VACANT && (first & 0x80000000u)) {
    const uint8_t* sp = rec + (int64_t)(first & 0x7fffffffu) * 8;
    n = bx_get(sp);
    list = sp + 4;
  }
  for (int64_t q = 0; q < n; ++q) {
    const uint32_t word = bx_get(list + 4 * q);
    if (word == BX_VACANT) break;
    if ((word >> 8) == (uint32_t)k) e = word & 0xffu;
  }
  return (uint16_t)(((span[i] & 0x80u) << 8) | (e << 7) | (span[i] & 0x7fu));
}

/* engine/cpu/bf16x.cpp:129 */
ORC_API int64_t lx_bf16x_row_bytes(int K) { return bx_k_ok(K) ? bx_row_bytes(K) : -1; }

/* The spill area: records in row order (bf16x.cpp:107-123). at (optional): each row's offset in it, -1 for none. */
static int64_t bx_layout(const uint16_t* w, int64_t rows, int K, int64_t* counts, int64_t* at) {
  int64_t area = 0;
  for (int64_t r = 0; r < rows; ++r) {
    const int64_t n = bx_exceptions(w + r * K, K);
    if (counts) counts[r] = n;
    if (at) at[r] = -1;
    if (n <= bx_slots(K)) continue;
    if (at) at[r] = area;
    area += bx_spill_bytes(n);
  }
  return area;
}

/* engine/cpu/bf16x.cpp:131-138 */
ORC_API int64_t lx_bf16x_bytes(const void* w, int64_t rows, int K, void* stream) {
  (void)stream;
  if (rows <= 0 || !bx_k_ok(K) || !w) return -(int64_t)fail(ORC_INVALID);
  return rows * bx_row_bytes(K) + bx_layout((const uint16_t*)w, rows, K, NULL, NULL);
}

/* engine/cpu/bf16x.cpp:140-160 */
ORC_API int lx_bf16x_encode(const void* w, int64_t rows, int K, void* out, int64_t out_bytes, void* stream) {
  (void)stream;
  if (rows <= 0) return ORC_OK;
  const int64_t rb = bx_k_ok(K) ? bx_row_bytes(K) : 0;
  if (!rb || !w || !out || ((uintptr_t)out & 7) != 0 || out_bytes < rows * rb) return fail(ORC_INVALID);
  int64_t* counts = (int64_t*)malloc(sizeof(int64_t) * (size_t)rows * 2);
  if (!counts) return fail(ORC_NOMEM);
  int64_t* at = counts + rows;
  const int64_t area = bx_layout((const uint16_t*)w, rows, K, counts, at);
  int st = ORC_OK;
  if (rows * rb + area > out_bytes) st = fail(ORC_INVALID);
  for (int64_t r = 0; r < rows && !st; ++r)
    bx_encode_row((const uint16_t*)w + r * K, K, (uint8_t*)out + r * rb, counts[r], at[r] < 0 ? 0 : rows * rb + at[r] - r * rb);
  free(counts);
  return st;
}

/* engine/cpu/bf16x.cpp:162-197 */
ORC_API int lx_bf16x_decode(const void* data, int64_t rows, int K, void* w, void* stream) {
  (void)stream;
  if (rows <= 0) return ORC_OK;
  if (!bx_k_ok(K) || !data || !w) return fail(ORC_INVALID);
  for (int64_t r = 0; r < rows; ++r)
    for (int k = 0; k < K; ++k) ((uint16_t*)w)[r * K + k] = bx_value((const uint8_t*)data + r * bx_row_bytes(K), K, k);
  return ORC_OK;
}

/* Element (n, k) of an [N, K] weight, exact, without its row factor (engine/cpu/quant.cpp:143-154). */
static float weight_element(int type, const void* data, const void* scale, int64_t n, int64_t k, int64_t K) {
  switch (type) {
    case LX_W_BF16: return bf16_value(((const uint16_t*)data)[n * K + k]);
    case LX_W_INT8: return (float)((const int8_t*)data)[n * K + k];
    case LX_W_FP8: return orc_e4m3_to_f32(((const uint8_t*)data)[n * K + k]);
    case LX_W_BF16X: return bf16_value(bx_value((const uint8_t*)data + n * bx_row_bytes((int)K), (int)K, (int)k));
    default: {
      uint8_t byte = ((const uint8_t*)data)[n * (K / 2) + k / 2];
      uint32_t code = (k & 1) ? (uint32_t)(byte >> 4) : (uint32_t)(byte & 15);
      return orc_e2m1_to_f32(code) * orc_e4m3_to_f32(((const uint8_t*)scale)[n * (K / 16) + k / 16]);
    }
  }
}

/* out[n, k] = bf16(element * row factor) (engine/cpu/quant.cpp:250-271). */
ORC_API int lx_dequantize_weight(const lx_weight* w, void* out, int64_t rows, int cols, void* stream) {
  (void)stream;
  if (!w || !w->data || !out) return fail(ORC_INVALID);
  if (rows <= 0) return ORC_OK;
  if (cols <= 0) return fail(ORC_INVALID);
  if (w->type < LX_W_BF16 || w->type > LX_W_NVFP4) return fail(ORC_INVALID);
  if (w->type != LX_W_BF16 && !w->scale) return fail(ORC_INVALID);
  if (w->type == LX_W_NVFP4 && cols % 16 != 0) return fail(ORC_INVALID);
  uint16_t* o = (uint16_t*)out;
  if (w->type == LX_W_BF16) {
    memcpy(o, w->data, (size_t)(2 * rows * cols));
    return ORC_OK;
  }
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < rows; ++n) {
    float f = w->type == LX_W_NVFP4 ? w->global : ((const float*)w->scale)[n];
    for (int64_t k = 0; k < cols; ++k) o[n * cols + k] = bf16_round(weight_element(w->type, w->data, w->scale, n, k, cols) * f);
  }
  return ORC_OK;
}

/* ---- the product ------------------------------------------------------------------------------ */

/* One weight row decoded to f32 without its row factor: what the reference's Row<F> hands the dot
 * (engine/cpu/kern/isa.cpp:26-91; the NVFP4 block scale is applied per element, :78-90). */
static void decode_row(int type, const void* data, const void* scale, int64_t n, int64_t K, float* out) {
  for (int64_t k = 0; k < K; ++k) out[k] = weight_element(type, data, scale, n, k, K);
}

/* sum_k x[k] * w[k] in f32: four lane accumulators over ascending k (a separate multiply and add per
 * step), one horizontal sum (0 + 2) + (1 + 3), then a fused scalar tail. This is the reference's tile at
 * its generic level (vector width 4): engine/cpu/kern/isa.cpp:205-270 with vfma / vhsum of
 * engine/cpu/kern/simd.h:144-157 and the fused tail of simd.h:467-476. Built with -ffp-contract=off so
 * the lane step stays two roundings; the sums then equal that level's bit for bit. */
static float dot_f32(const float* x, const float* w, int64_t K) {
  float lane[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  int64_t k = 0;
  for (; k + 4 <= K; k += 4)
    for (int j = 0; j < 4; ++j) {
      float prod = x[k + j] * w[k + j];
      lane[j] = lane[j] + prod;
    }
  float s = (lane[0] + lane[2]) + (lane[1] + lane[3]);
  for (; k < K; ++k) s = fmaf(x[k], w[k], s);
  return s;
}

/* The epilogue's exact operation order (engine/cpu/gemm.cpp:21-34). */
static void epilogue(float sum, float rf, const void* bias, int bias_dtype, void* y, int y_dtype, int64_t at, int64_t n,
                     float alpha, float beta) {
  float t = rf * 1.0f * sum;
  if (bias) t += load_f32(bias, bias_dtype, n);
  float v = alpha * t;
  if (beta != 0.0f) v = beta * load_f32(y, y_dtype, at) + v;
  store_f32(y, y_dtype, at, v);
}

static int weight_ok(const lx_weight* w, int64_t K) {
  if (!w || !w->data) return 0;
  switch (w->type) {
    case LX_W_BF16: return 1;
    case LX_W_INT8:
    case LX_W_FP8: return w->scale != NULL;
    case LX_W_NVFP4: return w->scale != NULL && K % 16 == 0;
    case LX_W_BF16X: return K < BX_MAX_K; /* only through the *_bf16x entries (engine/cpu/gemm.cpp:165) */
    default: return 0;
  }
}

/* y = alpha * (rf * (x @ W^T) + bias) + beta * y on f32 activation rows xs [M, K] (already in the
 * form the math sees them). Shared by the GEMV and the GEMM (engine/cpu/gemm.cpp:74-124). */
static int product(const float* xs, int64_t M, const lx_weight* w, const void* bias, int bias_dtype, void* y, int y_dtype,
                   int64_t ld_y, int64_t N, int64_t K, float alpha, float beta) {
  int err = 0;
#pragma omp parallel
  {
    float* row = (float*)malloc(sizeof(float) * (size_t)K);
    if (!row) {
#pragma omp atomic write
      err = 1;
    } else {
#pragma omp for schedule(static)
      for (int64_t n = 0; n < N; ++n) {
        decode_row(w->type, w->data, w->scale, n, K, row);
        float rf = 1.0f;
        if (w->type == LX_W_INT8 || w->type == LX_W_FP8) rf = ((const float*)w->scale)[n];
        else if (w->type == LX_W_NVFP4) rf = w->global;
        for (int64_t m = 0; m < M; ++m)
          epilogue(dot_f32(xs + m * K, row, K), rf, bias, bias_dtype, y, y_dtype, m * ld_y + n, n, alpha, beta);
      }
      free(row);
    }
  }
  return err ? fail(ORC_NOMEM) : ORC_OK;
}

/* The decode GEMV of every format: weight-only, f32 math on x as given (engine/cpu/gemm.cpp:160-183). */
static int gemv_any(const void* x, int x_dtype, int ld_x, const lx_weight* w, const void* bias, int bias_dtype, void* y,
                    int y_dtype, int ld_y, int M, int N, int K, float alpha, float beta) {
  if (M == 0 || N == 0) return ORC_OK;
  if (M < 0 || M > 8 || K <= 0 || ld_x < K || ld_y < N) return fail(ORC_INVALID);
  if (!dtype_ok(x_dtype) || !dtype_ok(y_dtype) || !dtype_ok(bias_dtype)) return fail(ORC_INVALID);
  if (!x || !y || !weight_ok(w, K)) return fail(ORC_INVALID);
  float* xs = (float*)malloc(sizeof(float) * (size_t)M * (size_t)K);
  if (!xs) return fail(ORC_NOMEM);
  for (int64_t m = 0; m < M; ++m)
    for (int64_t k = 0; k < K; ++k) xs[m * K + k] = load_f32(x, x_dtype, m * (int64_t)ld_x + k);
  int st = product(xs, M, w, bias, bias_dtype, y, y_dtype, ld_y, N, K, alpha, beta);
  free(xs);
  return st;
}

/* engine/cpu/gemm.cpp:339-348 */
ORC_API int lx_gemv(const void* x, int x_dtype, int ld_x, const void* w, int w_type, const float* w_scale, const void* bias,
                    int bias_dtype, void* y, int y_dtype, int ld_y, int M, int N, int K, float alpha, float beta,
                    void* stream) {
  (void)stream;
  if (w_type != LX_W_BF16 && w_type != LX_W_INT8) return fail(ORC_INVALID);
  if (w_type == LX_W_INT8 && !w_scale && M > 0 && N > 0) return fail(ORC_INVALID);
  lx_weight wt = {w_type, w, w_scale, 1.0f, NULL};
  return gemv_any(x, x_dtype, ld_x, &wt, bias, bias_dtype, y, y_dtype, ld_y, M, N, K, alpha, beta);
}

/* engine/cpu/gemm.cpp:364-371: the f32 product on the rows the encoding decodes to, so y is the bf16 weights' to the bit. */
ORC_API int lx_gemv_bf16x(const void* x, int x_dtype, int ld_x, const void* w, const void* bias, int bias_dtype, void* y,
                          int y_dtype, int ld_y, int M, int N, int K, float alpha, float beta, void* stream) {
  (void)stream;
  if (M != 0 && N != 0 && ((uintptr_t)w & 7) != 0) return fail(ORC_INVALID);
  lx_weight wt = {LX_W_BF16X, w, NULL, 1.0f, NULL};
  return gemv_any(x, x_dtype, ld_x, &wt, bias, bias_dtype, y, y_dtype, ld_y, M, N, K, alpha, beta);
}

/* engine/cpu/gemm.cpp:350-359 */
ORC_API int lx_gemv_w(const void* x, int x_dtype, int ld_x, const lx_weight* w, const void* bias, int bias_dtype, void* y,
                      int y_dtype, int ld_y, int M, int N, int K, float alpha, float beta, void* stream) {
  (void)stream;
  if (!w) return fail(ORC_INVALID);
  if (w->type == LX_W_BF16X)
    return lx_gemv_bf16x(x, x_dtype, ld_x, w->data, bias, bias_dtype, y, y_dtype, ld_y, M, N, K, alpha, beta, stream);
  return gemv_any(x, x_dtype, ld_x, w, bias, bias_dtype, y, y_dtype, ld_y, M, N, K, alpha, beta);
}

/* engine/cpu/gemm.cpp:373-381 */
ORC_API int lx_gemv_decode_bf16(const void* x, int x_dtype, int ld_x, const void* w, const void* bias, int bias_dtype,
                                void* y, int y_dtype, int ld_y, int M, int N, int K, float alpha, float beta,
                                void* stream) {
  (void)stream;
  lx_weight wt = {LX_W_BF16, w, NULL, 1.0f, NULL};
  return gemv_any(x, x_dtype, ld_x, &wt, bias, bias_dtype, y, y_dtype, ld_y, M, N, K, alpha, beta);
}

/* Any M, weight-only BF16 math: x is rounded to bf16 (a bf16 x is used as it is) and the weights are
 * expanded exactly, f32 accumulation (engine/cpu/gemm.cpp:189-296, the LX_MATH_BF16 branch :253-262).
 * The low-precision maths are outside this build's path and answer 801. */
static int gemm_bf16_math(const void* x, int x_dtype, int64_t ld_x, const lx_weight* w, const void* bias, int bias_dtype,
                          void* y, int y_dtype, int64_t ld_y, int64_t M, int64_t N, int64_t K, float alpha, float beta) {
  if (M == 0 || N == 0) return ORC_OK;
  if (M < 0 || N < 0 || K <= 0 || ld_x < K || ld_y < N) return fail(ORC_INVALID);
  if (!dtype_ok(x_dtype) || !dtype_ok(y_dtype) || (bias && !dtype_ok(bias_dtype))) return fail(ORC_INVALID);
  if (!x || !y || !weight_ok(w, K)) return fail(ORC_INVALID);
  float* xs = (float*)malloc(sizeof(float) * (size_t)M * (size_t)K);
  if (!xs) return fail(ORC_NOMEM);
  for (int64_t m = 0; m < M; ++m)
    for (int64_t k = 0; k < K; ++k) {
      uint16_t b = x_dtype == LX_BF16 ? ((const uint16_t*)x)[m * ld_x + k] : bf16_round(((const float*)x)[m * ld_x + k]);
      xs[m * K + k] = bf16_value(b);
    }
  int st = product(xs, M, w, bias, bias_dtype, y, y_dtype, ld_y, N, K, alpha, beta);
  free(xs);
  return st;
}

/* The INT8 math (engine/cpu/gemm.cpp:203-206,231-243, kern/isa.cpp:728-757, Epilogue::apply :21-34): int8 weights
 * only (else 801); the activations are quantised per token (lx_quantize_act's INT8 rule), the dot is an exact int32
 * sum converted to f32, and t = (rowscale * xscale) * sum before bias, alpha and beta. Pinned bit for bit against
 * oracle/_ref (tests/test_oracle_products.py) and by a float64 statement on the quantised values. */
static int gemm_int8_math(const void* x, int x_dtype, int64_t ld_x, const lx_weight* w, const void* bias, int bias_dtype,
                          void* y, int y_dtype, int64_t ld_y, int64_t M, int64_t N, int64_t K, float alpha, float beta) {
  if (M == 0 || N == 0) return ORC_OK;
  if (M < 0 || N < 0 || K <= 0 || ld_x < K || ld_y < N) return fail(ORC_INVALID);
  if (!dtype_ok(x_dtype) || !dtype_ok(y_dtype) || (bias && !dtype_ok(bias_dtype))) return fail(ORC_INVALID);
  if (!x || !y || !weight_ok(w, K)) return fail(ORC_INVALID);
  if (w->type != LX_W_INT8) return fail(ORC_UNSUPPORTED);
  int8_t* q = (int8_t*)malloc((size_t)M * (size_t)K);
  float* xs = (float*)malloc(sizeof(float) * (size_t)M);
  if (!q || !xs) {
    free(q);
    free(xs);
    return fail(ORC_NOMEM);
  }
  for (int64_t m = 0; m < M; ++m) quant_act_row(x, x_dtype, m * ld_x, LX_MATH_INT8, (int)K, (uint8_t*)(q + m * K), xs + m, NULL);
  const int8_t* wq = (const int8_t*)w->data;
  const float* rs = (const float*)w->scale;
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; ++n)
    for (int64_t m = 0; m < M; ++m) {
      int32_t sum = 0;
      for (int64_t k = 0; k < K; ++k) sum += (int32_t)q[m * K + k] * (int32_t)wq[n * K + k];
      float t = rs[n] * xs[m] * (float)sum;
      if (bias) t += load_f32(bias, bias_dtype, n);
      float v = alpha * t;
      if (beta != 0.0f) v = beta * load_f32(y, y_dtype, m * ld_y + n) + v;
      store_f32(y, y_dtype, m * ld_y + n, v);
    }
  free(q);
  free(xs);
  return ORC_OK;
}

/* The value an activation row holds under the FP8 or FP4 math at element k: the e4m3 value, or the e2m1 code times
 * its block's e4m3 scale (engine/cpu/gemm.cpp:270-277; exact in f32). */
static float act_value(int math, const uint8_t* q, const uint8_t* bs, int64_t k) {
  if (math == LX_MATH_FP8) return orc_e4m3_to_f32(q[k]);
  const uint8_t b = q[k >> 1];
  return orc_e2m1_to_f32((k & 1) ? (uint32_t)(b >> 4) : (uint32_t)(b & 15u)) * orc_e4m3_to_f32(bs[k >> 4]);
}

/* The FP8 math (fp8 or NVFP4 weights) and the FP4 math (NVFP4 weights) (engine/cpu/gemm.cpp:207-212,246-288,
 * Epilogue::apply_d :36-50): the activations are quantised per token (lx_quantize_act's rule for the math); the
 * products of the quantised activation values and the exact weight elements are summed in double (exactly), and
 * t = float(rowfactor * xscale * sum) with the products in double, before bias, alpha and beta in f32. Pinned bit for
 * bit against oracle/_ref (tests/test_oracle_products.py). */
static int gemm_exact_math(int math, const void* x, int x_dtype, int64_t ld_x, const lx_weight* w, const void* bias, int bias_dtype,
                           void* y, int y_dtype, int64_t ld_y, int64_t M, int64_t N, int64_t K, float alpha, float beta) {
  if (M == 0 || N == 0) return ORC_OK;
  if (M < 0 || N < 0 || K <= 0 || ld_x < K || ld_y < N) return fail(ORC_INVALID);
  if (!dtype_ok(x_dtype) || !dtype_ok(y_dtype) || (bias && !dtype_ok(bias_dtype))) return fail(ORC_INVALID);
  if (!x || !y || !weight_ok(w, K)) return fail(ORC_INVALID);
  if (math == LX_MATH_FP8 && w->type != LX_W_FP8 && w->type != LX_W_NVFP4) return fail(ORC_UNSUPPORTED);
  if (math == LX_MATH_FP4 && (w->type != LX_W_NVFP4 || K % 16 != 0)) return fail(ORC_UNSUPPORTED);
  float* xv = (float*)malloc(sizeof(float) * (size_t)M * (size_t)K);
  float* xs = (float*)malloc(sizeof(float) * (size_t)M);
  uint8_t* q = (uint8_t*)malloc((size_t)K + (size_t)K / 16 + 64);
  if (!xv || !xs || !q) {
    free(xv);
    free(xs);
    free(q);
    return fail(ORC_NOMEM);
  }
  for (int64_t m = 0; m < M; ++m) {
    quant_act_row(x, x_dtype, m * ld_x, math, (int)K, q, xs + m, q + K);
    for (int64_t k = 0; k < K; ++k) xv[m * K + k] = act_value(math, q, q + K, k);
  }
  int err = 0;
#pragma omp parallel
  {
    float* row = (float*)malloc(sizeof(float) * (size_t)K);
    if (!row) {
#pragma omp atomic write
      err = 1;
    } else {
#pragma omp for schedule(static)
      for (int64_t n = 0; n < N; ++n) {
        decode_row(w->type, w->data, w->scale, n, K, row);
        const double rf = w->type == LX_W_NVFP4 ? (double)w->global : (double)((const float*)w->scale)[n];
        for (int64_t m = 0; m < M; ++m) {
          double sum = 0.0;
          for (int64_t k = 0; k < K; ++k) sum += (double)xv[m * K + k] * (double)row[k];
          float t = (float)(rf * (double)xs[m] * sum);
          if (bias) t += load_f32(bias, bias_dtype, n);
          float v = alpha * t;
          if (beta != 0.0f) v = beta * load_f32(y, y_dtype, m * ld_y + n) + v;
          store_f32(y, y_dtype, m * ld_y + n, v);
        }
      }
      free(row);
    }
  }
  free(xv);
  free(xs);
  free(q);
  return err ? fail(ORC_NOMEM) : ORC_OK;
}

ORC_API int lx_gemm_w(const void* x, int x_dtype, int ld_x, const lx_weight* w, int math, const void* bias, int bias_dtype,
                      void* y, int y_dtype, int ld_y, int M, int N, int K, float alpha, float beta, void* workspace,
                      void* stream) {
  (void)stream;
  (void)workspace;
  if (!w) return fail(ORC_INVALID);
  if (math < LX_MATH_BF16 || math > LX_MATH_FP4) return fail(ORC_INVALID);
  if (math == LX_MATH_INT8) return gemm_int8_math(x, x_dtype, ld_x, w, bias, bias_dtype, y, y_dtype, ld_y, M, N, K, alpha, beta);
  if (math == LX_MATH_FP8 || math == LX_MATH_FP4)
    return gemm_exact_math(math, x, x_dtype, ld_x, w, bias, bias_dtype, y, y_dtype, ld_y, M, N, K, alpha, beta);
  return gemm_bf16_math(x, x_dtype, ld_x, w, bias, bias_dtype, y, y_dtype, ld_y, M, N, K, alpha, beta);
}

/* engine/cpu/gemm.cpp:290-296 */
ORC_API int64_t lx_gemm_workspace_bytes(int M, int K, int math) {
  if (M <= 0 || K <= 0) return 0;
  int64_t elem = math == LX_MATH_INT8 ? 1 : 4;
  int64_t bytes = ((int64_t)M * 4 + 63) / 64 * 64 + (int64_t)M * K * elem;
  return (bytes + 255) / 256 * 256;
}

/* The skinny decode GEMM's contract (engine/cuda/kernels.h:453-477): bf16 x, exact bf16 products,
 * f32 sums, f32 epilogue v = alpha * (sum + bias) + beta * y. The reference has it on CUDA only
 * (bf16 weights); the contract text is what this restates, for every format. */
ORC_API int lx_gemm_skinny(const void* x, int x_dtype, int ld_x, const lx_weight* w, const void* bias, int bias_dtype,
                           void* y, int y_dtype, int ld_y, int M, int N, int K, float alpha, float beta, void* stream) {
  (void)stream;
  if (!w) return fail(ORC_INVALID);
  if (x_dtype != LX_BF16 && M > 0 && N > 0) return fail(ORC_UNSUPPORTED);
  return gemm_bf16_math(x, x_dtype, ld_x, w, bias, bias_dtype, y, y_dtype, ld_y, M, N, K, alpha, beta);
}

/* ---- routing (engine/cpu/moe.cpp:343-397, contract engine/cuda/kernels.h:203-209) ----------------- */

ORC_API int lx_moe_route(const float* logits, const float* selection_bias, int32_t* ids, float* weights, float* entropy,
                         float* confidence, int T, int E, int top_k, void* stream) {
  (void)stream;
  if (T <= 0) return ORC_OK;
  if (top_k < 1 || top_k > 64 || top_k > E || !logits || !ids || !weights || !entropy || !confidence)
    return fail(ORC_INVALID);
  for (int64_t t = 0; t < T; ++t) {
    const float* row = logits + t * E;
    float m = -INFINITY;
    for (int i = 0; i < E; ++i)
      if (row[i] > m) m = row[i];
    float z = 0.0f;
    for (int i = 0; i < E; ++i) z += expf(row[i] - m);
    float h = 0.0f;
    for (int i = 0; i < E; ++i) {
      float p = expf(row[i] - m) / z;
      h -= p * logf(p > 1e-9f ? p : 1e-9f);
    }
    entropy[t] = h;
    confidence[t] = 1.0f / z; /* the largest probability is exp(0) / z */
    int picked[64];
    for (int r = 0; r < top_k; ++r) {
      float best = -INFINITY;
      int best_i = E;
      for (int i = 0; i < E; ++i) {
        int taken = 0;
        for (int q = 0; q < r; ++q) taken |= picked[q] == i;
        if (taken) continue;
        float v = row[i] + (selection_bias ? selection_bias[i] : 0.0f); /* one f32 add */
        if (v > best || (v == best && i < best_i)) {
          best = v;
          best_i = i;
        }
      }
      picked[r] = best_i;
    }
    float lmax = -INFINITY;
    for (int r = 0; r < top_k; ++r)
      if (row[picked[r]] > lmax) lmax = row[picked[r]];
    float e[64], esum = 0.0f;
    for (int r = 0; r < top_k; ++r) {
      e[r] = expf(row[picked[r]] - lmax);
      esum += e[r];
    }
    for (int r = 0; r < top_k; ++r) {
      ids[t * top_k + r] = picked[r];
      weights[t * top_k + r] = e[r] / esum;
    }
  }
  return ORC_OK;
}

/* ---- routed experts (engine/cpu/moe.cpp:163-329) -------------------------------------------------- */

static float silu(float v) { return v / (1.0f + expf(-v)); } /* engine/cpu/cpu.h:68 */

/* Expert e of an [E, N, K] stack as a plain [N, K] weight, with the expert's own NVFP4 global when the
 * stack carries them (engine/cpu/moe.cpp:36-64). */
static lx_weight expert_slice(const lx_weight* s, int64_t e, int64_t N, int64_t K) {
  lx_weight o = {s->type, NULL, NULL, 1.0f, NULL};
  int64_t rows = e * N;
  switch (s->type) {
    case LX_W_BF16: o.data = (const uint16_t*)s->data + rows * K; break;
    case LX_W_BF16X: o.data = (const uint8_t*)s->data + rows * bx_row_bytes((int)K); break; /* moe.cpp:44-45 */
    case LX_W_INT8:
    case LX_W_FP8:
      o.data = (const uint8_t*)s->data + rows * K;
      o.scale = (const float*)s->scale + rows;
      break;
    default:
      o.data = (const uint8_t*)s->data + rows * (K / 2);
      o.scale = (const uint8_t*)s->scale + rows * (K / 16);
      o.global = s->expert_global ? s->expert_global[e] : s->global;
      break;
  }
  return o;
}

static float row_factor(const lx_weight* w, int64_t n) {
  if (w->type == LX_W_INT8 || w->type == LX_W_FP8) return ((const float*)w->scale)[n];
  if (w->type == LX_W_NVFP4) return w->global;
  return 1.0f;
}

#define ORC_WEIGHT_ONLY (-1) /* the decode and legacy entries: f32 math on the activations as given */

/* One pass's activation rows under a math (engine/cpu/moe.cpp:82-121): weight-only and BF16: the bf16 values; INT8:
 * per-row int8 and a scale; FP8 / FP4: the quantised rows' exact values as f32 and a scale. */
typedef struct {
  float* f;     /* [rows, K] values (all maths but INT8) */
  int8_t* i;    /* [rows, K] (INT8) */
  float* scale; /* [rows], or NULL */
  int64_t K;
} orc_acts;

static void acts_fill(orc_acts* a, int64_t r, const uint16_t* src, int math, uint8_t* tmp) {
  const int64_t K = a->K;
  if (math == ORC_WEIGHT_ONLY || math == LX_MATH_BF16) {
    for (int64_t k = 0; k < K; ++k) a->f[r * K + k] = bf16_value(src[k]);
    return;
  }
  if (math == LX_MATH_INT8) {
    quant_act_row(src, LX_BF16, 0, LX_MATH_INT8, (int)K, (uint8_t*)(a->i + r * K), a->scale + r, NULL);
    return;
  }
  quant_act_row(src, LX_BF16, 0, math, (int)K, tmp, a->scale + r, tmp + K);
  for (int64_t k = 0; k < K; ++k) a->f[r * K + k] = act_value(math, tmp, tmp + K, k);
}

/* The dot of activation row r with a decoded weight row (wrow: f32 values; wq: the int8 bytes under the INT8 math):
 * f32 lanes (weight-only, BF16), an exact int32 sum as f32 (INT8), or an exact double sum (FP8 / FP4)
 * (engine/cpu/moe.cpp:125-154). */
static double acts_dot(const orc_acts* a, int64_t r, const float* wrow, const int8_t* wq, int math) {
  const int64_t K = a->K;
  if (math == LX_MATH_INT8) {
    int32_t sum = 0;
    for (int64_t k = 0; k < K; ++k) sum += (int32_t)a->i[r * K + k] * (int32_t)wq[k];
    return (double)(float)sum;
  }
  if (math == LX_MATH_FP8 || math == LX_MATH_FP4) {
    double sum = 0.0;
    for (int64_t k = 0; k < K; ++k) sum += (double)a->f[r * K + k] * (double)wrow[k];
    return sum;
  }
  return (double)dot_f32(a->f + r * K, wrow, K);
}

/* The routed experts under a math (engine/cpu/moe.cpp:163-329): for each (token, slot) pair, inter =
 * bf16(silu(s_g * (xs * g)) * (s_u * (xs * u))) with g = gate_e . x, u = up_e . x on the pair's activation row (the
 * token's latent row, quantised per row under the INT8 / FP8 / FP4 maths: xs is its scale; :241-279, rounding point
 * :267-270; under the FP8 / FP4 maths the whole SwiGLU is in double on the exact dots, :259-265); the intermediate row
 * is quantised again per row once it is complete (:281-286); contribution = s_l * (xs2 * down_e . inter) (:292-312),
 * and out[t] = w0 * c0 + sum_{k >= 1} w_k * c_k in slot order (:315-327). */
static int experts(const uint16_t* latent, const int32_t* ids, const float* weights, const lx_weight* gu,
                   const lx_weight* dn, float* out, int64_t T, int64_t L, int64_t I, int64_t top_k, int64_t E, int math) {
  const int64_t P = T * top_k;
  if (E <= 0) {
    for (int64_t p = 0; p < P; ++p)
      if (ids[p] + 1 > E) E = ids[p] + 1;
  }
  for (int64_t p = 0; p < P; ++p)
    if (ids[p] < 0 || ids[p] >= E) return fail(ORC_INVALID);
  const int quantised = math == LX_MATH_INT8 || math == LX_MATH_FP8 || math == LX_MATH_FP4;
  const int exact = math == LX_MATH_FP8 || math == LX_MATH_FP4;
  const int int8 = math == LX_MATH_INT8;
  float* contrib = (float*)malloc(sizeof(float) * (size_t)P * (size_t)L);
  orc_acts x1 = {NULL, NULL, NULL, L}, x2 = {NULL, NULL, NULL, I};
  x1.f = int8 ? NULL : (float*)malloc(sizeof(float) * (size_t)P * (size_t)L);
  x1.i = int8 ? (int8_t*)malloc((size_t)P * (size_t)L) : NULL;
  x2.f = int8 ? NULL : (float*)malloc(sizeof(float) * (size_t)P * (size_t)I);
  x2.i = int8 ? (int8_t*)malloc((size_t)P * (size_t)I) : NULL;
  x1.scale = quantised ? (float*)malloc(sizeof(float) * (size_t)P) : NULL;
  x2.scale = quantised ? (float*)malloc(sizeof(float) * (size_t)P) : NULL;
  uint16_t* staged = (uint16_t*)malloc(sizeof(uint16_t) * (size_t)P * (size_t)I); /* the bf16 intermediate, by pair */
  const int64_t kmax = L > I ? L : I;
  uint8_t* tmp = (uint8_t*)malloc((size_t)kmax + (size_t)kmax / 16 + 64);
  int err = !contrib || !staged || !tmp || (int8 ? !x1.i || !x2.i : !x1.f || !x2.f) || (quantised && (!x1.scale || !x2.scale));
  if (!err) {
    /* Rows are kept by pair (the reference keeps them in grouped order; a row's content is the same). */
    for (int64_t p = 0; p < P; ++p) acts_fill(&x1, p, latent + (p / top_k) * L, math, tmp);
    /* Gate/up: experts in turn; each expert's rows are decoded once for all the pairs that chose it. */
#pragma omp parallel for schedule(dynamic, 1)
    for (int64_t e = 0; e < E; ++e) {
      int64_t cnt = 0;
      for (int64_t p = 0; p < P; ++p) cnt += ids[p] == e;
      if (!cnt) continue;
      lx_weight g = expert_slice(gu, e, 2 * I, L);
      float* wg = (float*)malloc(sizeof(float) * (size_t)L);
      float* wu = (float*)malloc(sizeof(float) * (size_t)L);
      if (!wg || !wu) {
#pragma omp atomic write
        err = 1;
      } else {
        for (int64_t i = 0; i < I; ++i) {
          decode_row(g.type, g.data, g.scale, i, L, wg);
          decode_row(g.type, g.data, g.scale, I + i, L, wu);
          const int8_t* qg = int8 ? (const int8_t*)g.data + i * L : NULL;
          const int8_t* qu = int8 ? (const int8_t*)g.data + (I + i) * L : NULL;
          const float sg = row_factor(&g, i), su = row_factor(&g, I + i);
          for (int64_t p = 0; p < P; ++p) {
            if (ids[p] != e) continue;
            const float xs = x1.scale ? x1.scale[p] : 1.0f;
            const double dg = acts_dot(&x1, p, wg, qg, math), du = acts_dot(&x1, p, wu, qu, math);
            if (exact) {
              const double gg = sg * ((double)xs * dg), uu = su * ((double)xs * du);
              staged[p * I + i] = bf16_round((float)(gg / (1.0 + exp(-gg)) * uu));
            } else {
              const float gg = sg * (xs * (float)dg), uu = su * (xs * (float)du);
              staged[p * I + i] = bf16_round(silu(gg) * uu);
            }
          }
        }
      }
      free(wg);
      free(wu);
    }
  }
  if (!err) {
    for (int64_t p = 0; p < P; ++p) acts_fill(&x2, p, staged + p * I, math, tmp);
#pragma omp parallel for schedule(dynamic, 1)
    for (int64_t e = 0; e < E; ++e) {
      int64_t cnt = 0;
      for (int64_t p = 0; p < P; ++p) cnt += ids[p] == e;
      if (!cnt) continue;
      lx_weight d = expert_slice(dn, e, L, I);
      float* wrow = (float*)malloc(sizeof(float) * (size_t)I);
      if (!wrow) {
#pragma omp atomic write
        err = 1;
      } else {
        for (int64_t l = 0; l < L; ++l) {
          decode_row(d.type, d.data, d.scale, l, I, wrow);
          const int8_t* qd = int8 ? (const int8_t*)d.data + l * I : NULL;
          const float rf = row_factor(&d, l);
          for (int64_t p = 0; p < P; ++p) {
            if (ids[p] != e) continue;
            const float xs = x2.scale ? x2.scale[p] : 1.0f;
            const double dd = acts_dot(&x2, p, wrow, qd, math);
            contrib[p * L + l] = exact ? (float)(rf * ((double)xs * dd)) : rf * (xs * (float)dd);
          }
        }
      }
      free(wrow);
    }
  }
  if (!err) {
    for (int64_t t = 0; t < T; ++t) {
      float* o = out + t * L;
      const float w0 = weights[t * top_k];
      for (int64_t l = 0; l < L; ++l) o[l] = w0 * contrib[(t * top_k) * L + l];
      for (int64_t k = 1; k < top_k; ++k) {
        const float wk = weights[t * top_k + k];
        for (int64_t l = 0; l < L; ++l) o[l] += wk * contrib[(t * top_k + k) * L + l];
      }
    }
  }
  free(contrib);
  free(x1.f);
  free(x1.i);
  free(x2.f);
  free(x2.i);
  free(x1.scale);
  free(x2.scale);
  free(staged);
  free(tmp);
  return err ? fail(ORC_NOMEM) : ORC_OK;
}

static int stack_ok(const lx_weight* w, int64_t K) { return weight_ok(w, K); }

static int experts_args(const void* latent, const int32_t* ids, const float* weights, float* out, int L, int I, int top_k) {
  if (!latent || !ids || !weights || !out || L <= 0 || I <= 0 || top_k < 1) return fail(ORC_INVALID);
  return ORC_OK;
}

/* engine/cpu/moe.cpp:444-458 */
ORC_API int lx_moe_experts(const void* latent, const int32_t* ids, const float* weights, const void* gate_up,
                           const void* down, float* out, int T, int L, int I, int top_k, void* stream) {
  (void)stream;
  if (T <= 0) return ORC_OK;
  int st = experts_args(latent, ids, weights, out, L, I, top_k);
  if (st) return st;
  if (!gate_up || !down) return fail(ORC_INVALID);
  lx_weight gu = {LX_W_BF16, gate_up, NULL, 1.0f, NULL}, dn = {LX_W_BF16, down, NULL, 1.0f, NULL};
  return experts((const uint16_t*)latent, ids, weights, &gu, &dn, out, T, L, I, top_k, 0, ORC_WEIGHT_ONLY);
}

/* engine/cpu/moe.cpp:496-503 */
ORC_API int lx_moe_experts_decode_bf16(const void* latent, const int32_t* ids, const float* weights, const void* gate_up,
                                       const void* down, float* out, void* workspace, int T, int L, int I, int top_k,
                                       void* stream) {
  if (T <= 0) return ORC_OK;
  if (top_k > 8 || !workspace) return fail(ORC_INVALID);
  return lx_moe_experts(latent, ids, weights, gate_up, down, out, T, L, I, top_k, stream);
}

/* engine/cpu/moe.cpp:480-494: lx_moe_experts with the rows read from the encoding. */
ORC_API int lx_moe_experts_bf16x(const void* latent, const int32_t* ids, const float* weights, const void* gate_up,
                                 const void* down, float* out, void* workspace, int T, int L, int I, int top_k, void* stream) {
  (void)stream;
  if (T <= 0) return ORC_OK;
  int st = experts_args(latent, ids, weights, out, L, I, top_k);
  if (st) return st;
  if (top_k > 8 || !gate_up || !down || !workspace || L >= BX_MAX_K || I >= BX_MAX_K) return fail(ORC_INVALID);
  lx_weight gu = {LX_W_BF16X, gate_up, NULL, 1.0f, NULL}, dn = {LX_W_BF16X, down, NULL, 1.0f, NULL};
  return experts((const uint16_t*)latent, ids, weights, &gu, &dn, out, T, L, I, top_k, 0, ORC_WEIGHT_ONLY);
}

/* engine/cpu/moe.cpp:519-538 */
ORC_API int lx_moe_experts_decode(const void* latent, const int32_t* ids, const float* weights, const lx_weight* gate_up,
                                  const lx_weight* down, float* out, void* workspace, int T, int L, int I, int top_k,
                                  void* stream) {
  (void)stream;
  (void)workspace;
  if (T <= 0) return ORC_OK;
  if (T > 8 || top_k > 8) return fail(ORC_INVALID);
  int st = experts_args(latent, ids, weights, out, L, I, top_k);
  if (st) return st;
  if (!gate_up || !down) return fail(ORC_INVALID);
  if (gate_up->type == LX_W_BF16X || down->type == LX_W_BF16X) {
    if (gate_up->type != LX_W_BF16X || down->type != LX_W_BF16X) return fail(ORC_UNSUPPORTED);
    return lx_moe_experts_bf16x(latent, ids, weights, gate_up->data, down->data, out, workspace, T, L, I, top_k, stream);
  }
  if (!stack_ok(gate_up, L) || !stack_ok(down, I)) return fail(ORC_INVALID);
  return experts((const uint16_t*)latent, ids, weights, gate_up, down, out, T, L, I, top_k, 0, ORC_WEIGHT_ONLY);
}

/* engine/cpu/moe.cpp:546-572 */
ORC_API int lx_moe_experts_grouped(const void* latent, const int32_t* ids, const float* weights, const lx_weight* gate_up,
                                   const lx_weight* down, int math, float* out, void* workspace, int T, int L, int I, int E,
                                   int top_k, void* stream) {
  (void)stream;
  (void)workspace;
  if (T <= 0) return ORC_OK;
  int st = experts_args(latent, ids, weights, out, L, I, top_k);
  if (st) return st;
  if (E <= 0 || !gate_up || !down || !stack_ok(gate_up, L) || !stack_ok(down, I)) return fail(ORC_INVALID);
  switch (math) {
    case LX_MATH_BF16: break;
    case LX_MATH_INT8:
      if (gate_up->type != LX_W_INT8 || down->type != LX_W_INT8) return fail(ORC_UNSUPPORTED);
      break;
    case LX_MATH_FP8:
      if ((gate_up->type != LX_W_FP8 && gate_up->type != LX_W_NVFP4) || (down->type != LX_W_FP8 && down->type != LX_W_NVFP4))
        return fail(ORC_UNSUPPORTED);
      break;
    case LX_MATH_FP4:
      if (gate_up->type != LX_W_NVFP4 || down->type != LX_W_NVFP4 || L % 16 || I % 16) return fail(ORC_UNSUPPORTED);
      break;
    default: return fail(ORC_INVALID);
  }
  return experts((const uint16_t*)latent, ids, weights, gate_up, down, out, T, L, I, top_k, E, math);
}

static int64_t round256(int64_t b) { return (b + 255) / 256 * 256; }

/* engine/cpu/moe.cpp:540-544 */
ORC_API int64_t lx_moe_decode_workspace_bytes(int T, int I, int top_k) {
  if (T <= 0 || I <= 0 || top_k <= 0) return 0;
  return round256(2 * (int64_t)T * top_k * I);
}
/* engine/cpu/moe.cpp:506-509 */
ORC_API int64_t lx_moe_bf16x_workspace_bytes(int T, int I, int top_k) { return lx_moe_decode_workspace_bytes(T, I, top_k); }
/* engine/cpu/moe.cpp:574-581 */
ORC_API int64_t lx_moe_grouped_workspace_bytes(int T, int L, int I, int E, int top_k, int math) {
  (void)E;
  (void)math;
  if (T <= 0 || L <= 0 || I <= 0 || top_k <= 0) return 0;
  return round256(2 * (int64_t)T * top_k * I);
}

/* ---- the calls either side of the experts in a decode layer, and the legacy product forms ------------ */

/* engine/cpu/gemm.cpp:304-314: bf16 x and weights under the BF16 math, bias bf16 or null. */
ORC_API int lx_gemm_bf16(const void* x, int ld_x, const void* w, const void* bias, void* y, int y_dtype, int ld_y, int M, int N,
                         int K, float alpha, float beta, void* stream) {
  (void)stream;
  if (y_dtype != LX_F32 && y_dtype != LX_BF16) return fail(ORC_INVALID);
  if (M < 0 || N < 0 || K <= 0 || ld_x < K || ld_y < N) return fail(ORC_INVALID);
  if (M == 0 || N == 0) return ORC_OK;
  if (!x || !w || !y) return fail(ORC_INVALID);
  lx_weight wt = {LX_W_BF16, w, NULL, 1.0f, NULL};
  return gemm_bf16_math(x, LX_BF16, ld_x, &wt, bias, LX_BF16, y, y_dtype, ld_y, M, N, K, alpha, beta);
}

/* engine/cpu/gemm.cpp:316-337: f32 x and weights, the same dot and epilogue (row factor 1, alpha 1, beta 0). */
ORC_API int lx_gemm_f32(const float* x, int ld_x, const float* w, const float* bias, float* y, int ld_y, int M, int N, int K,
                        void* stream) {
  (void)stream;
  if (M < 0 || N < 0 || K <= 0 || ld_x < K || ld_y < N) return fail(ORC_INVALID);
  if (M == 0 || N == 0) return ORC_OK;
  if (!x || !w || !y) return fail(ORC_INVALID);
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; ++n)
    for (int64_t m = 0; m < M; ++m)
      epilogue(dot_f32(x + m * (int64_t)ld_x, w + n * (int64_t)K, K), 1.0f, bias, LX_F32, y, LX_F32, m * (int64_t)ld_y + n, n, 1.0f, 0.0f);
  return ORC_OK;
}

/* engine/cpu/spec.cpp:21-28: lx_gemm_f32 limited to decode-sized steps. */
ORC_API int lx_spec_gemv_f32(const float* x, int ld_x, const float* w, const float* bias, float* y, int ld_y, int M, int N, int K,
                             void* stream) {
  if (M == 0 || N == 0) return ORC_OK;
  if (M < 0 || M > 8 || K <= 0 || ld_x < K || ld_y < N || !x || !w || !y) return fail(ORC_INVALID);
  return lx_gemm_f32(x, ld_x, w, bias, y, ld_y, M, N, K, stream);
}

ORC_API int lx_moe_route(const float* logits, const float* selection_bias, int32_t* ids, float* weights, float* entropy,
                         float* confidence, int T, int E, int top_k, void* stream);

/* engine/cuda/kernels.h:211-219: the two calls in one (the reference's CPU backend leaves it out; by its contract every
 * output has the bits of lx_spec_gemv_f32 followed by lx_moe_route, which is what this is). */
ORC_API int lx_router_route(const float* x, int ld_x, const float* w, const float* bias, float* logits, const float* selection_bias,
                            int32_t* ids, float* weights, float* entropy, float* confidence, int32_t* ticket, int M, int E, int K,
                            int top_k, void* stream) {
  if (M <= 0) return ORC_OK;
  if (M > 8 || E <= 0 || E > 1024 || K <= 0 || K > 2048 || ld_x < K || top_k < 1 || top_k > 32 || top_k > E || !x || !w || !logits ||
      !ids || !weights || !entropy || !confidence || !ticket)
    return fail(ORC_INVALID);
  int st = lx_spec_gemv_f32(x, ld_x, w, bias, logits, E, M, E, K, stream);
  if (st) return st;
  return lx_moe_route(logits, selection_bias, ids, weights, entropy, confidence, M, E, top_k, stream);
}

/* engine/cpu/moe.cpp:399-418 (history == NULL) and :420-442. */
static int summary(const int32_t* ids, const float* weights, const void* expert_emb, float* sum, float* history, float a, float b,
                   int T, int R, int top_k, int with_history) {
  if (T <= 0 || R <= 0) return ORC_OK;
  if (!ids || !weights || !expert_emb || !sum || top_k < 1 || (with_history && !history)) return fail(ORC_INVALID);
  const uint16_t* emb = (const uint16_t*)expert_emb;
  for (int64_t t = 0; t < T; ++t) {
    float* s = sum + t * R;
    for (int r = 0; r < R; ++r) s[r] = 0.0f;
    for (int k = 0; k < top_k; ++k) {
      const float w = weights[t * top_k + k];
      const uint16_t* row = emb + (int64_t)ids[t * top_k + k] * R;
      for (int r = 0; r < R; ++r) s[r] += w * bf16_value(row[r]);
    }
    if (with_history) {
      float* h = history + t * R;
      for (int r = 0; r < R; ++r) h[r] = a * h[r] + b * s[r];
    }
  }
  return ORC_OK;
}
ORC_API int lx_moe_summary(const int32_t* ids, const float* weights, const void* expert_emb, float* sum, int T, int R, int top_k,
                           void* stream) {
  (void)stream;
  return summary(ids, weights, expert_emb, sum, NULL, 0.0f, 0.0f, T, R, top_k, 0);
}
ORC_API int lx_moe_summary_history(const int32_t* ids, const float* weights, const void* expert_emb, float* sum, float* history,
                                   float a, float b, int T, int R, int top_k, void* stream) {
  (void)stream;
  return summary(ids, weights, expert_emb, sum, history, a, b, T, R, top_k, 1);
}

/* engine/cpu/moe.cpp:460-476: the weight-only experts on int8 stacks with per-row scales, any T. */
ORC_API int lx_moe_experts_w8(const void* latent, const int32_t* ids, const float* weights, const int8_t* gate_up,
                              const float* gate_up_scale, const int8_t* down, const float* down_scale, float* out, void* workspace,
                              int T, int L, int I, int top_k, void* stream) {
  (void)stream;
  (void)workspace;
  if (T <= 0) return ORC_OK;
  int st = experts_args(latent, ids, weights, out, L, I, top_k);
  if (st) return st;
  if (!gate_up || !gate_up_scale || !down || !down_scale) return fail(ORC_INVALID);
  lx_weight gu = {LX_W_INT8, gate_up, gate_up_scale, 1.0f, NULL}, dn = {LX_W_INT8, down, down_scale, 1.0f, NULL};
  return experts((const uint16_t*)latent, ids, weights, &gu, &dn, out, T, L, I, top_k, 0, ORC_WEIGHT_ONLY);
}
/* engine/cpu/moe.cpp:512-517 */
ORC_API int64_t lx_moe_workspace_bytes(int T, int I, int top_k) {
  if (T <= 0 || I <= 0 || top_k <= 0) return 0;
  const int64_t pairs = (int64_t)T * top_k;
  return round256((2 * pairs * I + 15) / 16 * 16 + 8 * pairs);
}

/* ---- the few runtime calls a host-memory harness needs (engine/cuda/kernels.h:308-339) ------------- */

ORC_API int lx_rt_backend(void) { return 3; /* LX_BACKEND_CPU */ }
ORC_API int lx_rt_device_count(void) { return 1; }
ORC_API int lx_rt_stream_sync(void* stream) {
  (void)stream;
  return ORC_OK;
}
ORC_API int lx_rt_device_sync(void) { return ORC_OK; }
ORC_API int lx_rt_last_error(void) {
  int e = g_last_error;
  g_last_error = 0;
  return e;
}
