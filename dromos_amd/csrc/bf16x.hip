// The LX_W_BF16X codec: lx_bf16x_row_bytes, lx_bf16x_bytes, lx_bf16x_encode, lx_bf16x_decode
// (contract: engine/cuda/kernels.h:573-586; the bytes written are those of engine/cpu/bf16x.cpp:58-140).
//
// Load-time work, one wavefront per row. A row's bytes depend on that row alone except for where its spill record
// lies (rows with more exceptions than header slots keep their list behind all rows, in row order), so the encoder
// runs in two launches around one host step: count every row's exceptions, lay the spill records out on the host from
// the counts, encode. Rows that spill are rare in trained weights; without any the host step is a sum of zeros.
#include <vector>

#include "bf16x.h"
#include "common.h"

namespace dro {
namespace {

constexpr int kThreads = 256;
constexpr int kRowsPerWg = kThreads / kWave;

__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) v = max(v, static_cast<uint32_t>(__shfl_xor(static_cast<int>(v), off)));
  return v;
}

// What a lane sees of one span: values 2 * lane and 2 * lane + 1 of it (zero past the row's end), their exponents,
// and the span's top.
struct SpanView {
  uint32_t v0, v1, e0, e1, top;
  bool in0, in1;
  int k0;
  __device__ __forceinline__ SpanView(const uint16_t* row, int K, int span, int lane) {
    k0 = span * bf16x::kSpan + 2 * lane;
    in0 = k0 < K;
    in1 = k0 + 1 < K;
    v0 = in0 ? row[k0] : 0u;
    v1 = in1 ? row[k0 + 1] : 0u;
    e0 = (v0 >> 7) & 0xffu;
    e1 = (v1 >> 7) & 0xffu;
    top = wave_max_u32(max(e0, e1));
  }
  // A value whose exponent lies more than 15 below the top cannot be coded in a nibble.
  __device__ __forceinline__ bool out0() const { return in0 && top - e0 > 15u; }
  __device__ __forceinline__ bool out1() const { return in1 && top - e1 > 15u; }
};

__global__ void __launch_bounds__(kThreads) bf16x_count_kernel(const uint16_t* __restrict__ w, int64_t rows, int K, int* __restrict__ counts) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t r = static_cast<int64_t>(blockIdx.x) * kRowsPerWg + threadIdx.x / kWave;
  if (r >= rows) return;
  const uint16_t* row = w + r * K;
  const int spans = bf16x::Geometry(K).spans;
  int n = 0;
  for (int b = 0; b < spans; ++b) {
    const SpanView s(row, K, b, lane);
    n += __popcll(__ballot(s.out0())) + __popcll(__ballot(s.out1()));
  }
  if (lane == 0) counts[r] = n;
}

// spill_at: per row, the offset of its spill record from the end of the rows (null when no row spills).
__global__ void __launch_bounds__(kThreads) bf16x_encode_kernel(const uint16_t* __restrict__ w, int64_t rows, int K, uint8_t* __restrict__ out,
                                                                const int* __restrict__ counts, const int64_t* __restrict__ spill_at) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t r = static_cast<int64_t>(blockIdx.x) * kRowsPerWg + threadIdx.x / kWave;
  if (r >= rows) return;
  const bf16x::Geometry g(K);
  const int64_t rb = g.row_bytes();
  const uint16_t* row = w + r * K;
  uint8_t* rec = out + r * rb;
  uint32_t* slots = reinterpret_cast<uint32_t*>(rec);
  const int n = counts[r];
  const bool spilled = n > g.slots;
  uint32_t* list = slots;
  if (spilled) {
    // A record's address is kept relative to its own row, in 8-byte units.
    const int64_t off = rows * rb + spill_at[r] - r * rb;
    uint32_t* spill = reinterpret_cast<uint32_t*>(rec + off);
    if (lane == 0) {
      slots[0] = bf16x::kSpilled | static_cast<uint32_t>(off / 8);
      spill[0] = static_cast<uint32_t>(n);
      spill[1 + n] = bf16x::kVacant;
      if (bf16x::spill_bytes(n) > 4 * (static_cast<int64_t>(n) + 2)) spill[2 + n] = 0u;
    }
    list = spill + 1;
  }
  // The slots no exception word goes to, and the zero bytes between the tops and the first span.
  for (int i = (spilled ? 1 : n) + lane; i < g.slots; i += kWave) slots[i] = bf16x::kVacant;
  for (int i = g.tops_at() + g.spans + lane; i < g.header; i += kWave) rec[i] = 0;

  const uint64_t below = (1ull << lane) - 1;
  int at = 0;  // exception words written so far: the same in every lane
  for (int b = 0; b < g.spans; ++b) {
    const SpanView s(row, K, b, lane);
    uint8_t* sp = rec + g.header + static_cast<int64_t>(b) * bf16x::kSpanBytes;
    if (lane == 0) rec[g.tops_at() + b] = static_cast<uint8_t>(s.top);
    // Exceptions go to the list in ascending k: lane-major, the even value first.
    const bool x0 = s.out0(), x1 = s.out1();
    const uint64_t m0 = __ballot(x0), m1 = __ballot(x1);
    const int before = at + __popcll(m0 & below) + __popcll(m1 & below);
    if (x0) list[before] = static_cast<uint32_t>(s.k0) << 8 | s.e0;
    if (x1) list[before + (x0 ? 1 : 0)] = static_cast<uint32_t>(s.k0 + 1) << 8 | s.e1;
    at += __popcll(m0) + __popcll(m1);
    // Nibbles: zero for exceptions and past the row's end.
    const uint32_t c0 = s.in0 && !x0 ? s.top - s.e0 : 0u, c1 = s.in1 && !x1 ? s.top - s.e1 : 0u;
    *reinterpret_cast<uint16_t*>(sp + 2 * lane) =
        static_cast<uint16_t>(((s.v0 >> 8) & 0x80u) | (s.v0 & 0x7fu) | (((s.v1 >> 8) & 0x80u) | (s.v1 & 0x7fu)) << 8);
    // Nibble word q = lane / 4 covers values 8q .. 8q + 7; this lane holds values i and i + 1 of them, i = 2 * (lane % 4):
    // value j sits in byte j % 4, the low half for j < 4, the high half otherwise. The four lanes' parts are or-ed.
    const int i = 2 * (lane & 3);
    const int shift = 8 * (i & 3) + (i & 4);
    uint32_t word = c0 << shift | c1 << (shift + 8);
    word |= static_cast<uint32_t>(__shfl_xor(static_cast<int>(word), 1));
    word |= static_cast<uint32_t>(__shfl_xor(static_cast<int>(word), 2));
    if ((lane & 3) == 0) reinterpret_cast<uint32_t*>(sp + bf16x::kNibbles)[lane >> 2] = word;
  }
}

__global__ void __launch_bounds__(kThreads) bf16x_decode_kernel(const uint8_t* __restrict__ data, int64_t rows, int K, uint16_t* __restrict__ w) {
  const int64_t item = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (item >= rows * K) return;
  const int64_t r = item / K;
  w[item] = bf16x::value_bits(data + r * bf16x::row_bytes(K), K, static_cast<int>(item - r * K));
}

bool valid_k(int K) { return K > 0 && K < bf16x::kMaxK; }

// Every row's exception count on the device (*d_counts, from hipMallocAsync: the caller frees it) and on the host.
int count_rows(const void* w, int64_t rows, int K, hipStream_t s, int** d_counts, std::vector<int>& counts) {
  if (int st = status_of(hipMallocAsync(reinterpret_cast<void**>(d_counts), sizeof(int) * rows, s))) return st;
  const unsigned grid = static_cast<unsigned>((rows + kRowsPerWg - 1) / kRowsPerWg);
  hipLaunchKernelGGL(bf16x_count_kernel, dim3(grid), dim3(kThreads), 0, s, static_cast<const uint16_t*>(w), rows, K, *d_counts);
  int st = status_of(hipGetLastError());
  counts.resize(static_cast<size_t>(rows));
  if (!st) st = status_of(hipMemcpyAsync(counts.data(), *d_counts, sizeof(int) * rows, hipMemcpyDeviceToHost, s));
  if (!st) st = status_of(hipStreamSynchronize(s));
  if (st) {
    (void)hipFreeAsync(*d_counts, s);
    *d_counts = nullptr;
  }
  return st;
}

// The spill area the counts give (engine/cpu/bf16x.cpp:107-123): records in row order; at[r] = row r's offset in it.
int64_t spill_layout(const std::vector<int>& counts, int K, std::vector<int64_t>* at) {
  const int slots = bf16x::Geometry(K).slots;
  int64_t area = 0;
  for (size_t r = 0; r < counts.size(); ++r) {
    if (counts[r] <= slots) continue;
    if (at) {
      if (at->empty()) at->assign(counts.size(), -1);
      (*at)[r] = area;
    }
    area += bf16x::spill_bytes(counts[r]);
  }
  return area;
}

}  // namespace
}  // namespace dro

using namespace dro;

extern "C" {

int64_t lx_bf16x_row_bytes(int K) { return valid_k(K) ? bf16x::row_bytes(K) : -1; }

int64_t lx_bf16x_bytes(const void* w, int64_t rows, int K, void* stream) {
  if (rows <= 0 || !valid_k(K) || !w) return -static_cast<int64_t>(fail(kInvalid));
  hipStream_t s = as_stream(stream);
  int* d_counts = nullptr;
  std::vector<int> counts;
  if (int st = count_rows(w, rows, K, s, &d_counts, counts)) return -static_cast<int64_t>(st);
  (void)hipFreeAsync(d_counts, s);
  return rows * bf16x::row_bytes(K) + spill_layout(counts, K, nullptr);
}

int lx_bf16x_encode(const void* w, int64_t rows, int K, void* out, int64_t out_bytes, void* stream) {
  if (rows <= 0) return kOk;
  const int64_t rb = valid_k(K) ? bf16x::row_bytes(K) : 0;
  if (!rb || !w || !out || (reinterpret_cast<uintptr_t>(out) & 7) != 0 || out_bytes < rows * rb) return fail(kInvalid);
  hipStream_t s = as_stream(stream);
  int* d_counts = nullptr;
  std::vector<int> counts;
  if (int st = count_rows(w, rows, K, s, &d_counts, counts)) return st;
  std::vector<int64_t> at;
  const int64_t area = spill_layout(counts, K, &at);
  int st = kOk;
  int64_t* d_at = nullptr;
  if (rows * rb + area > out_bytes) st = fail(kInvalid);
  if (!st && area > 0) {
    st = status_of(hipMallocAsync(reinterpret_cast<void**>(&d_at), sizeof(int64_t) * rows, s));
    if (!st) st = status_of(hipMemcpyAsync(d_at, at.data(), sizeof(int64_t) * rows, hipMemcpyHostToDevice, s));
  }
  if (!st) {
    const unsigned grid = static_cast<unsigned>((rows + kRowsPerWg - 1) / kRowsPerWg);
    hipLaunchKernelGGL(bf16x_encode_kernel, dim3(grid), dim3(kThreads), 0, s, static_cast<const uint16_t*>(w), rows, K,
                       static_cast<uint8_t*>(out), d_counts, d_at);
    st = status_of(hipGetLastError());
  }
  if (d_at) {
    // The offsets were copied from this call's host memory: they must have left it before it goes.
    const int st2 = status_of(hipStreamSynchronize(s));
    if (!st) st = st2;
    (void)hipFreeAsync(d_at, s);
  }
  (void)hipFreeAsync(d_counts, s);
  return st;
}

int lx_bf16x_decode(const void* data, int64_t rows, int K, void* w, void* stream) {
  if (rows <= 0) return kOk;
  if (!valid_k(K) || !data || !w) return fail(kInvalid);
  const int64_t items = rows * K;
  hipLaunchKernelGGL(bf16x_decode_kernel, dim3(static_cast<unsigned>((items + kThreads - 1) / kThreads)), dim3(kThreads), 0,
                     as_stream(stream), static_cast<const uint8_t*>(data), rows, K, static_cast<uint16_t*>(w));
  return status_of(hipGetLastError());
}

}  // extern "C"
