// The runtime half of the backend ABI on the HIP runtime (engine/cuda/kernels.h:294-381), lx_arch and the
// kernel variant table (engine/cuda/tunable.h:37-55), and the measured read bandwidth probe.
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <map>
#include <mutex>
#include <string>
#include <tuple>
#include <vector>

#include "common.h"

namespace dro {

namespace {
thread_local int g_last_error = 0;
}

int fail(int status) {
  if (status != kOk) g_last_error = status;
  return status;
}

int status_of(hipError_t e) {
  if (e == hipSuccess) return kOk;
  (void)hipGetLastError();  // the runtime's sticky copy
  return fail(static_cast<int>(e));
}

bool batch_invariant() {
  const char* v = getenv("LX_BATCH_INVARIANT");
  return v && *v && v[0] != '0';
}

int compute_units() {
  static thread_local int cached_dev = -1, cached = 0;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 256;
  if (dev != cached_dev) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached = n;
    cached_dev = dev;
  }
  return cached;
}

void allow_lds(const void* kernel, int limit) {
  static thread_local std::vector<std::tuple<int, const void*, int>> raised;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) (void)hipGetLastError();
  for (const auto& r : raised)
    if (std::get<0>(r) == dev && std::get<1>(r) == kernel && std::get<2>(r) >= limit) return;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, limit) != hipSuccess) (void)hipGetLastError();
  raised.emplace_back(dev, kernel, limit);
}

// gemm.hip: the per-stream buffer of the slab kernel's partial tiles.
int slab_reserve(hipStream_t stream);
int slab_release(hipStream_t stream);

// Admission rule of the GEMV's variants (gemv.hip).
bool gemv_admits(int wtype, int variant, int N, int K);

namespace {

std::mutex& table_lock() {
  static std::mutex m;
  return m;
}
int g_arch_override = -1;

struct Registered {
  std::vector<std::string> variants;
  int gemv_format;  // the lx_wtype whose order class admits a variant, or -1 for no rule
};

// The kernels with variants. The GEMV of each format has three: its K split of 1, 2 or 4 wavefronts (admitted where the
// split is the shape's order class). The matrix-core product of each format (9 .. 64 activation rows) has four: the tile
// kernels by their own rule, the walk kernel with 1, 2 or 4 tiles a workgroup, the tile kernels without or with the slab
// kernel; none changes a sum, so all are admitted.
const std::map<std::string, Registered>& registry() {
  static const auto* r = new std::map<std::string, Registered>{
      {"gemv_w_bf16", {{"s1", "s2", "s4"}, LX_W_BF16}},
      {"gemv_w_int8", {{"s1", "s2", "s4"}, LX_W_INT8}},
      {"gemv_w_fp8", {{"s1", "s2", "s4"}, LX_W_FP8}},
      {"gemv_w_nvfp4", {{"s1", "s2", "s4"}, LX_W_NVFP4}},
      {"gemm_w_bf16", {{"tiles", "walk1", "walk2", "walk4", "window", "slab", "walkparts", "walksplit"}, -1}},
      {"gemm_w_int8", {{"tiles", "walk1", "walk2", "walk4", "window", "slab", "walkparts", "walksplit"}, -1}},
      {"gemm_w_fp8", {{"tiles", "walk1", "walk2", "walk4", "window", "slab", "walkparts", "walksplit"}, -1}},
      {"gemm_w_nvfp4", {{"tiles", "walk1", "walk2", "walk4", "window", "slab", "walkparts", "walksplit"}, -1}},
  };
  return *r;
}

using Key = std::tuple<std::string, int, int, int>;
std::map<Key, int>& table() {
  static auto* t = new std::map<Key, int>;
  return *t;
}

int bucket(int m) {
  int b = 1;
  while (b < m) b <<= 1;
  return b;
}

int real_arch() {
  // gfx950 reports 9.5: the same major * 10 + minor form the CUDA backend uses for its cards.
  static thread_local int cached_dev = -1, cached = 95;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 95;
  if (dev != cached_dev) {
    int major = 9, minor = 5;
    if (hipDeviceGetAttribute(&major, hipDeviceAttributeComputeCapabilityMajor, dev) != hipSuccess) major = 9;
    if (hipDeviceGetAttribute(&minor, hipDeviceAttributeComputeCapabilityMinor, dev) != hipSuccess) minor = 5;
    cached = major * 10 + minor;
    cached_dev = dev;
  }
  return cached;
}

__global__ void __launch_bounds__(256) read_probe_kernel(const u32x4* __restrict__ p, int64_t n16, unsigned* sink) {
  int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
  unsigned acc = 0;
  for (; i + 7 * stride < n16; i += 8 * stride) {
    u32x4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(p + i + u * stride);
#pragma unroll
    for (int u = 0; u < 8; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  for (; i < n16; i += stride) {
    const u32x4 v = __builtin_nontemporal_load(p + i);
    acc ^= v.x ^ v.y ^ v.z ^ v.w;
  }
  if (acc == 0x9e3779b9u) *sink = acc;  // keeps the loads alive; pseudo-random data never matches
}

// The measurement floor of a streamed product: 16-byte non-temporal loads, eight in flight per lane, every wavefront's
// loads asked for at once, 1 KB contiguous per instruction: what the decode GEMV does, without the product.
__global__ void __launch_bounds__(256) stream_read_kernel(const u32x4* __restrict__ p, int64_t n16, unsigned* sink) {
  const int64_t base = (static_cast<int64_t>(blockIdx.x) * 4 + threadIdx.x / kWave) * (8 * kWave) + (threadIdx.x & (kWave - 1));
  u32x4 v[8];
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    const int64_t i = base + u * kWave;
    v[u] = __builtin_nontemporal_load(p + (i < n16 ? i : n16 - 1));
  }
  unsigned acc = 0;
#pragma unroll
  for (int u = 0; u < 8; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  if (acc == 0x9e3779b9u && sink) *sink = acc;
}

__global__ void empty_kernel() {}

__global__ void fill_random_kernel(unsigned* p, int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) {
    unsigned x = static_cast<unsigned>(i) * 2654435761u + 0x9e3779b9u;
    x ^= x >> 16;
    x *= 0x85ebca6bu;
    x ^= x >> 13;
    p[i] = x;
  }
}

}  // namespace

namespace {
// lx_tune_run's choice for the launches it makes on this thread: it goes before the table.
thread_local const char* g_run_kernel = nullptr;
thread_local int g_run_variant = -1;
// bf16 values spread evenly over (-scale, scale), a fixed function of the index and the seed.
__global__ void fill_bf16_kernel(uint16_t* p, int64_t n, unsigned seed, float scale) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  unsigned x = (static_cast<unsigned>(i) + seed) * 2654435761u + 0x9e3779b9u;
  x ^= x >> 16;
  x *= 0x85ebca6bu;
  x ^= x >> 13;
  const float v = (static_cast<float>(x >> 8) * (1.0f / 8388608.0f) - 1.0f) * scale;
  p[i] = f32_to_bf16_bits(v);
}

}  // namespace

int tuned_variant(const char* kernel, int M, int N, int K) {
  if (g_run_kernel && strcmp(g_run_kernel, kernel) == 0) return g_run_variant;
  std::lock_guard<std::mutex> g(table_lock());
  if (table().empty()) return -1;
  auto it = table().find(Key{kernel, bucket(M), N, K});
  return it == table().end() ? -1 : it->second;
}

}  // namespace dro

using namespace dro;

extern "C" {

int lx_rt_backend(void) { return LX_BACKEND_HIP; }

int lx_rt_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return n;
}

int lx_rt_set_device(int ordinal) { return status_of(hipSetDevice(ordinal)); }

int lx_rt_alloc(void** ptr, int64_t bytes) {
  if (!ptr) return fail(kInvalid);
  *ptr = nullptr;
  if (bytes <= 0) return kOk;
  if (int e = status_of(hipMalloc(ptr, static_cast<size_t>(bytes)))) return e;
  return status_of(hipMemset(*ptr, 0, static_cast<size_t>(bytes)));
}

int lx_rt_free(void* ptr) { return status_of(hipFree(ptr)); }

int lx_rt_host_alloc(void** ptr, int64_t bytes) {
  if (!ptr) return fail(kInvalid);
  *ptr = nullptr;
  return bytes <= 0 ? kOk : status_of(hipHostMalloc(ptr, static_cast<size_t>(bytes), hipHostMallocDefault));
}

int lx_rt_host_free(void* ptr) { return status_of(hipHostFree(ptr)); }

int lx_rt_memset(void* ptr, int value, int64_t bytes, void* stream) {
  return bytes <= 0 ? kOk : status_of(hipMemsetAsync(ptr, value, static_cast<size_t>(bytes), as_stream(stream)));
}

int lx_rt_copy(void* dst, const void* src, int64_t bytes, lx_copy_kind kind, void* stream) {
  if (bytes <= 0) return kOk;
  const hipMemcpyKind k = kind == LX_COPY_H2D       ? hipMemcpyHostToDevice
                          : kind == LX_COPY_D2H     ? hipMemcpyDeviceToHost
                          : kind == LX_COPY_DEFAULT ? hipMemcpyDefault
                                                    : hipMemcpyDeviceToDevice;
  return status_of(hipMemcpyAsync(dst, src, static_cast<size_t>(bytes), k, as_stream(stream)));
}

int lx_rt_stream_create(void** stream) {
  if (!stream) return fail(kInvalid);
  hipStream_t s = nullptr;
  const int e = status_of(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));  // default priority
  *stream = s;
  // What the products keep per stream is made here, so that no product ever allocates; a stream that cannot have it
  // still works (those products take another kernel).
  if (!e) (void)slab_reserve(s);
  return e;
}
int lx_rt_stream_destroy(void* stream) {
  (void)slab_release(as_stream(stream));
  return status_of(hipStreamDestroy(as_stream(stream)));
}
int lx_rt_stream_reserve(void* stream) { return slab_reserve(as_stream(stream)); }
int lx_rt_stream_release(void* stream) { return slab_release(as_stream(stream)); }
int lx_rt_stream_sync(void* stream) { return status_of(hipStreamSynchronize(as_stream(stream))); }

int lx_rt_event_create(void** event) {
  if (!event) return fail(kInvalid);
  hipEvent_t e = nullptr;
  const int r = status_of(hipEventCreateWithFlags(&e, hipEventDisableTiming));
  *event = e;
  return r;
}
int lx_rt_event_create_timed(void** event) {
  if (!event) return fail(kInvalid);
  hipEvent_t e = nullptr;
  const int r = status_of(hipEventCreate(&e));
  *event = e;
  return r;
}
int lx_rt_event_destroy(void* event) { return status_of(hipEventDestroy(static_cast<hipEvent_t>(event))); }
int lx_rt_event_record(void* event, void* stream) {
  return status_of(hipEventRecord(static_cast<hipEvent_t>(event), as_stream(stream)));
}
int lx_rt_event_sync(void* event) { return status_of(hipEventSynchronize(static_cast<hipEvent_t>(event))); }
int lx_rt_event_elapsed(void* start, void* stop, float* ms) {
  return status_of(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
}

int lx_rt_capture_begin(void* stream) {
  return status_of(hipStreamBeginCapture(as_stream(stream), hipStreamCaptureModeThreadLocal));
}
int lx_rt_capture_end(void* stream, void** graph) {
  if (!graph) return fail(kInvalid);
  *graph = nullptr;
  hipGraph_t g = nullptr;
  if (int e = status_of(hipStreamEndCapture(as_stream(stream), &g))) return e;
  hipGraphExec_t exec = nullptr;
  const int e = status_of(hipGraphInstantiate(&exec, g, nullptr, nullptr, 0));
  (void)hipGraphDestroy(g);
  *graph = exec;
  return e;
}
int lx_rt_graph_launch(void* graph, void* stream) {
  return status_of(hipGraphLaunch(static_cast<hipGraphExec_t>(graph), as_stream(stream)));
}
int lx_rt_graph_destroy(void* graph) { return status_of(hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph))); }

int lx_rt_device_sync(void) { return status_of(hipDeviceSynchronize()); }

int lx_rt_last_error(void) {
  const int e = g_last_error;
  g_last_error = 0;
  return e;
}

const char* lx_rt_error_string(int status) {
  switch (status) {
    case 0: return "success";
    case LX_ERR_NOT_SUPPORTED: return "operation not supported";
    case LX_ERR_TUNE_REJECTED: return "variant rejected by the kernel's order class";
    case LX_ERR_TUNE_VARIANT: return "no such variant";
    default: return hipGetErrorString(static_cast<hipError_t>(status));
  }
}

int lx_rt_is_host_memory(const void* ptr) {
  hipPointerAttribute_t attr;
  if (!ptr || hipPointerGetAttributes(&attr, ptr) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return attr.type == hipMemoryTypeHost ? 1 : 0;
}

int lx_rt_device_props(int ordinal, lx_device_props* props) {
  if (!props) return fail(kInvalid);
  hipDeviceProp_t p;
  if (int e = status_of(hipGetDeviceProperties(&p, ordinal))) return e;
  memset(props, 0, sizeof(*props));
  snprintf(props->name, sizeof(props->name), "%s", p.name);
  props->cc_major = p.major;
  props->cc_minor = p.minor;
  props->sms = p.multiProcessorCount;
  props->l2_bytes = p.l2CacheSize;
  props->mem_clock_khz = p.memoryClockRate;
  props->bus_bits = p.memoryBusWidth;
  int v = 0;
  if (hipDriverGetVersion(&v) == hipSuccess) props->driver_version = v;
  if (hipRuntimeGetVersion(&v) == hipSuccess) props->runtime_version = v;
  snprintf(props->isa, sizeof(props->isa), "%s", p.gcnArchName);
  // The maths lx_gemm_w and lx_moe_experts_grouped run on the matrix cores' own types (engine/runtime/plan.cpp:79,358
  // reads these bits): bf16, int8 (v_mfma_i32_16x16x64_i8) and e4m3 (v_mfma_f32_16x16x32_fp8_fp8) operands.
  props->native_math = (1 << LX_MATH_BF16) | (1 << LX_MATH_INT8) | (1 << LX_MATH_FP8);
  return kOk;
}

int lx_rt_mem_info(int64_t* free_bytes, int64_t* total_bytes) {
  size_t f = 0, t = 0;
  if (int e = status_of(hipMemGetInfo(&f, &t))) return e;
  if (free_bytes) *free_bytes = static_cast<int64_t>(f);
  if (total_bytes) *total_bytes = static_cast<int64_t>(t);
  return kOk;
}

// engine/cuda/kernels.h:371-381: a read-only kernel over every compute unit, 16-byte loads, eight in flight
// per thread, best of `reps` after a warm-up. The spec figure is memory clock x 2 x bus width / 8.
int lx_bandwidth_probe(int64_t bytes, int reps, double* read_gbps, double* spec_gbps, void* stream) {
  if (!read_gbps || !spec_gbps || bytes < 64 * 1024 || bytes % 16 != 0) return fail(kInvalid);
  if (reps < 1) reps = 1;
  hipStream_t s = as_stream(stream);
  int dev = 0;
  if (int e = status_of(hipGetDevice(&dev))) return e;
  hipDeviceProp_t p;
  if (int e = status_of(hipGetDeviceProperties(&p, dev))) return e;
  *spec_gbps = static_cast<double>(p.memoryClockRate) * 1e3 * 2.0 * p.memoryBusWidth / 8.0 / 1e9;
  void* buf = nullptr;
  unsigned* sink = nullptr;
  if (int e = status_of(hipMalloc(&buf, static_cast<size_t>(bytes)))) return e;
  if (int e = status_of(hipMalloc(&sink, sizeof(unsigned)))) {
    (void)hipFree(buf);
    return e;
  }
  const int64_t words = bytes / 4;
  hipLaunchKernelGGL(fill_random_kernel, dim3(static_cast<unsigned>((words + 255) / 256)), dim3(256), 0, s,
                     static_cast<unsigned*>(buf), words);
  hipEvent_t a = nullptr, b = nullptr;
  int st = status_of(hipEventCreate(&a));
  if (!st) st = status_of(hipEventCreate(&b));
  double best = 0.0;
  const unsigned grid = static_cast<unsigned>(compute_units());
  for (int r = 0; r <= reps && !st; ++r) {  // r == 0 warms up
    st = status_of(hipEventRecord(a, s));
    hipLaunchKernelGGL(read_probe_kernel, dim3(grid), dim3(256), 0, s, static_cast<const u32x4*>(buf), bytes / 16, sink);
    if (!st) st = status_of(hipEventRecord(b, s));
    if (!st) st = status_of(hipEventSynchronize(b));
    float ms = 0.0f;
    if (!st) st = status_of(hipEventElapsedTime(&ms, a, b));
    if (!st && r > 0 && ms > 0.0f) {
      const double gbps = static_cast<double>(bytes) / (ms * 1e-3) / 1e9;
      if (gbps > best) best = gbps;
    }
  }
  if (getenv("LX_BANDWIDTH_TRACE")) fprintf(stderr, "lx_bandwidth_probe: %.1f GB/s read, %.1f GB/s spec\n", best, *spec_gbps);
  *read_gbps = best;
  if (a) (void)hipEventDestroy(a);
  if (b) (void)hipEventDestroy(b);
  (void)hipFree(sink);
  (void)hipFree(buf);
  return st;
}

int lx_probe_read(const void* data, int64_t bytes, void* stream) {
  if (!data || bytes < 16 || reinterpret_cast<uintptr_t>(data) % 16 != 0) return fail(kInvalid);
  const int64_t n16 = bytes / 16, per_wg = 4 * 8 * kWave;
  hipLaunchKernelGGL(stream_read_kernel, dim3(static_cast<unsigned>((n16 + per_wg - 1) / per_wg)), dim3(256), 0, as_stream(stream),
                     static_cast<const u32x4*>(data), n16, static_cast<unsigned*>(nullptr));
  return status_of(hipGetLastError());
}

int lx_probe_empty(void* stream) {
  hipLaunchKernelGGL(empty_kernel, dim3(1), dim3(kWave), 0, as_stream(stream));
  return status_of(hipGetLastError());
}

// ---- architecture and variants ------------------------------------------------------------------------

int lx_arch(void) {
  const int real = real_arch();
  int over;
  {
    std::lock_guard<std::mutex> g(table_lock());
    if (g_arch_override < 0) {
      const char* env = getenv("LX_ARCH_OVERRIDE");
      g_arch_override = env ? atoi(env) : 0;
    }
    over = g_arch_override;
  }
  return over > 0 && over < real ? over : real;
}

int lx_set_arch_override(int arch) {
  {
    std::lock_guard<std::mutex> g(table_lock());
    g_arch_override = arch > 0 ? arch : 0;
  }
  return lx_arch();
}

int lx_tune_get(const char* kernel, int M, int N, int K) { return kernel ? tuned_variant(kernel, M, N, K) : -1; }

int lx_tune_set(const char* kernel, int M, int N, int K, int variant) {
  if (!kernel) return kInvalid;
  auto reg = registry().find(kernel);
  if (reg != registry().end()) {
    if (variant < 0 || variant >= static_cast<int>(reg->second.variants.size())) return LX_ERR_TUNE_VARIANT;
    if (reg->second.gemv_format >= 0 && !gemv_admits(reg->second.gemv_format, variant, N, K)) return LX_ERR_TUNE_REJECTED;
  }
  std::lock_guard<std::mutex> g(table_lock());
  table()[Key{kernel, bucket(M), N, K}] = variant;
  return kOk;
}

int lx_tune_force(const char* kernel, int M, int N, int K, int variant) {
  if (!kernel) return kInvalid;
  auto reg = registry().find(kernel);
  if (reg != registry().end() && (variant < 0 || variant >= static_cast<int>(reg->second.variants.size())))
    return LX_ERR_TUNE_VARIANT;
  std::lock_guard<std::mutex> g(table_lock());
  table()[Key{kernel, bucket(M), N, K}] = variant;
  return kOk;
}

void lx_tune_clear(void) {
  std::lock_guard<std::mutex> g(table_lock());
  table().clear();
}

int lx_tune_kernels(const char** names, int capacity) {
  int i = 0;
  for (const auto& kv : registry()) {
    if (names && i < capacity) names[i] = kv.first.c_str();
    ++i;
  }
  return i;
}

int lx_tune_variants(const char* kernel) {
  if (!kernel) return 0;
  auto reg = registry().find(kernel);
  return reg == registry().end() ? 0 : static_cast<int>(reg->second.variants.size());
}

const char* lx_tune_variant_name(const char* kernel, int variant) {
  if (!kernel) return "";
  auto reg = registry().find(kernel);
  if (reg == registry().end() || variant < 0 || variant >= static_cast<int>(reg->second.variants.size())) return "";
  return reg->second.variants[variant].c_str();
}


// ---- the autotuner's entry points (engine/cuda/tunable.h:57-75, engine/cuda/tunable.cu:158-185) --------------------

namespace {

// What a runnable kernel is timed on: weights of its format made from seeded bf16 values by the library's own quantiser,
// bf16 activations; kept per problem for the life of the process (the tuner asks for each many times).
struct TuneInputs {
  void* w = nullptr;
  void* scale = nullptr;
  void* x = nullptr;
  float global = 1.0f;
};

int format_of_kernel(const std::string& kernel, bool* gemv) {
  static const char* const kNames[4] = {"bf16", "int8", "fp8", "nvfp4"};
  for (int f = 0; f < 4; ++f) {
    if (kernel == std::string("gemv_w_") + kNames[f]) return *gemv = true, f;
    if (kernel == std::string("gemm_w_") + kNames[f]) return *gemv = false, f;
  }
  return -1;
}

int tune_inputs(int format, int M, int N, int K, hipStream_t s, TuneInputs* out) {
  static std::mutex lock;
  static std::map<std::tuple<int, int, int, int, int>, TuneInputs> cache;
  int dev = 0;
  if (int e = status_of(hipGetDevice(&dev))) return e;
  std::lock_guard<std::mutex> g(lock);
  auto it = cache.find({dev, format, M, N, K});
  if (it != cache.end()) return *out = it->second, kOk;
  TuneInputs in;
  void* master = nullptr;
  const int64_t wn = static_cast<int64_t>(N) * K, xn = static_cast<int64_t>(M) * K;
  auto release = [&] {
    (void)hipFree(master);
    (void)hipFree(in.w);
    (void)hipFree(in.scale);
    (void)hipFree(in.x);
  };
  if (hipMalloc(&master, wn * 2) != hipSuccess || hipMalloc(&in.x, xn * 2) != hipSuccess) return release(), fail(kNoMemory);
  hipLaunchKernelGGL(fill_bf16_kernel, dim3(static_cast<unsigned>((wn + 255) / 256)), dim3(256), 0, s, static_cast<uint16_t*>(master), wn, 17u, 0.04f);
  hipLaunchKernelGGL(fill_bf16_kernel, dim3(static_cast<unsigned>((xn + 255) / 256)), dim3(256), 0, s, static_cast<uint16_t*>(in.x), xn, 91u, 1.0f);
  int st = status_of(hipGetLastError());
  if (!st && format == LX_W_BF16) {
    in.w = master;
    master = nullptr;
  } else if (!st) {
    const int64_t data_bytes = format == LX_W_NVFP4 ? wn / 2 : wn;
    const int64_t scale_bytes = format == LX_W_NVFP4 ? wn / 16 : static_cast<int64_t>(N) * 4;
    if (hipMalloc(&in.w, data_bytes) != hipSuccess || hipMalloc(&in.scale, scale_bytes) != hipSuccess) return release(), fail(kNoMemory);
    lx_weight q{static_cast<lx_wtype>(format), in.w, in.scale, 1.0f, nullptr};
    st = lx_quantize_weight(master, &q, N, K, s);
    in.global = q.global;
  }
  if (!st) st = status_of(hipStreamSynchronize(s));
  (void)hipFree(master);
  master = nullptr;
  if (st) return release(), st;
  cache[{dev, format, M, N, K}] = in;
  *out = in;
  return kOk;
}

}  // namespace

int lx_tune_runnable(const char* kernel) {
  bool gemv;
  return kernel && format_of_kernel(kernel, &gemv) >= 0 ? 1 : 0;
}

int lx_tune_key(const char* kernel, const lx_tune_problem* problem, char* out, int capacity) {
  if (!kernel || !problem) return 0;
  std::string key = kernel;
  if (problem->weight != 0 || problem->math != 0) key += "@w" + std::to_string(problem->weight) + "m" + std::to_string(problem->math);
  if (problem->experts != 1) key += "@e" + std::to_string(problem->experts);
  if (out && capacity > 0) {
    const size_t n = key.size() < static_cast<size_t>(capacity - 1) ? key.size() : static_cast<size_t>(capacity - 1);
    memcpy(out, key.data(), n);
    out[n] = '\0';
  }
  return static_cast<int>(key.size());
}

// Runs one variant of a registered product on inputs of its own and writes y as f32 [M, N] to `out` (device memory).
// The kernels' names carry their weight format, so a problem names it again or leaves it 0; the BF16 math and single
// weights only.
int lx_tune_run(const char* kernel, int variant, const lx_tune_problem* problem, float* out, void* stream) {
  if (!kernel || !problem || !out) return fail(kInvalid);
  bool gemv = false;
  const int format = format_of_kernel(kernel, &gemv);
  if (format < 0) return kNotSupported;
  if (variant < 0 || variant >= lx_tune_variants(kernel)) return kNotSupported;
  const int M = problem->M, N = problem->N, K = problem->K;
  if (M <= 0 || N <= 0 || K <= 0) return fail(kInvalid);
  if (problem->experts != 1 || problem->math != LX_MATH_BF16 || (problem->weight != 0 && problem->weight != format)) return kNotSupported;
  if ((gemv && M > 8) || (format == LX_W_NVFP4 && K % 16 != 0)) return kNotSupported;
  TuneInputs in;
  if (int e = tune_inputs(format, M, N, K, as_stream(stream), &in)) return e;
  const lx_weight w{static_cast<lx_wtype>(format), in.w, in.scale, in.global, nullptr};
  g_run_kernel = kernel;
  g_run_variant = variant;
  const int st = gemv ? lx_gemv_w(in.x, LX_BF16, K, &w, nullptr, LX_F32, out, LX_F32, N, M, N, K, 1.0f, 0.0f, stream)
                      : lx_gemm_w(in.x, LX_BF16, K, &w, LX_MATH_BF16, nullptr, LX_F32, out, LX_F32, N, M, N, K, 1.0f, 0.0f, nullptr, stream);
  g_run_kernel = nullptr;
  g_run_variant = -1;
  return st;
}

}  // extern "C"
