// Test infrastructure, not part of the product: drives the REFERENCE's model-folder loader (engine/core/checkpoint.cpp,
// ModelWeights::load, compiled from the reference's own sources by `make ckptref`) over the reference's CPU backend
// and writes down what it holds, so that the golden fixtures under tests/golden/ can record the format and the bytes of
// every projection the reference makes from a folder. With the CPU backend "device" memory is host memory
// (engine/cpu/runtime.cpp), read here through lx_rt_copy as the reference's own test does
// (tests/unit/checkpoint_test.cpp:41-54).
//
//   ckptref_dump DIR TARGET SKIP_EXPERTS VOCAB HIDDEN EXPERTS INTERMEDIATE LATENT BLOB [plain tensor names ...] [--skipped stack names ...]
//
// prints one line per item to stdout and appends the items' bytes to BLOB:
//   stored <lx_wtype>                                       ModelWeights::stored_format()
//   format <lx_wtype>                                       ModelWeights::format()
//   device_bytes <n>
//   projection <name> <type> <E> <N> <K> <stack> <data off> <data len> <scale off> <scale len> <global bits>
//              <globals off> <globals len> <expert data bytes> <expert scale bytes>
//   skipped <name> <E> <N> <K> <stack> <expert data bytes> <expert scale bytes> <whether projection() is non-null>
//   plain <name> <lx_dtype> <rank> <dims ...> <off> <len>
//   error <text>                                            what ModelWeights::load threw
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

#include "core/checkpoint.h"
#include "core/config.h"
#include "cuda/kernels.h"

namespace {

FILE* g_blob = nullptr;
long g_at = 0;

// Copies `bytes` of the backend's memory behind the blob; returns where they start.
long dump(const void* device, size_t bytes) {
  const long at = g_at;
  if (!bytes) return at;
  std::vector<char> host(bytes);
  if (lx_rt_copy(host.data(), device, static_cast<int64_t>(bytes), LX_COPY_D2H, nullptr) != 0 || lx_rt_stream_sync(nullptr) != 0)
    throw std::runtime_error("lx_rt_copy failed");
  if (std::fwrite(host.data(), 1, bytes, g_blob) != bytes) throw std::runtime_error("short write to the blob");
  g_at += static_cast<long>(bytes);
  return at;
}

size_t scale_bytes(const lx_weight& w, int64_t rows, int64_t K) {
  switch (w.type) {
    case LX_W_INT8:
    case LX_W_FP8: return static_cast<size_t>(rows) * 4;
    case LX_W_NVFP4: return static_cast<size_t>(rows) * static_cast<size_t>(K / 16);
    default: return 0;
  }
}

}  // namespace

int main(int argc, char** argv) {
  if (argc < 10) {
    std::fprintf(stderr, "usage: %s DIR TARGET SKIP VOCAB HIDDEN EXPERTS INTERMEDIATE LATENT BLOB [plain names]\n", argv[0]);
    return 2;
  }
  const std::string dir = argv[1];
  lx::LoadOptions options;
  options.target = static_cast<lx_wtype>(std::atoi(argv[2]));
  options.skip_experts = std::atoi(argv[3]) != 0;
  lx::MetisConfig config;  // the loader reads these five (engine/core/checkpoint.cpp:318-332)
  config.vocab_size = std::atoi(argv[4]);
  config.hidden_size = std::atoi(argv[5]);
  config.n_routed_experts = std::atoi(argv[6]);
  config.expert_intermediate_size = std::atoi(argv[7]);
  config.latent_dim = std::atoi(argv[8]);
  // The family stays empty, as for a loader that reads no config.json: the NVFP4 refusal then names no repository.
  g_blob = std::fopen(argv[9], "wb");
  if (!g_blob) {
    std::fprintf(stderr, "cannot write %s\n", argv[9]);
    return 2;
  }
  try {
    std::printf("stored %d\n", static_cast<int>(lx::ModelWeights::stored_format(dir)));
    const lx::ModelWeights m = lx::ModelWeights::load(dir, config, options);
    std::printf("format %d\n", static_cast<int>(m.format()));
    std::printf("device_bytes %zu\n", m.device_bytes());
    for (const std::string& name : m.projection_names()) {
      const lx_weight* w = m.projection(name);
      const lx::ModelWeights::Shape s = m.projection_shape(name);
      const auto per_expert = m.expert_bytes(name);
      const size_t data = static_cast<size_t>(s.E) * per_expert.first;
      const size_t scale = w->scale ? scale_bytes(*w, s.E * s.N, s.K) : 0;
      const size_t globals = w->expert_global ? static_cast<size_t>(s.E) * 4 : 0;
      uint32_t bits;
      std::memcpy(&bits, &w->global, 4);
      const long d = dump(w->data, data), sc = dump(w->scale, scale), g = dump(w->expert_global, globals);
      std::printf("projection %s %d %lld %lld %lld %d %ld %zu %ld %zu %u %ld %zu %zu %zu\n", name.c_str(), static_cast<int>(w->type),
                  static_cast<long long>(s.E), static_cast<long long>(s.N), static_cast<long long>(s.K), s.stack ? 1 : 0, d, data, sc,
                  scale, bits, g, globals, per_expert.first, per_expert.second);
    }
    // Names behind "--skipped" are stacks that skip_experts left off the device: their shapes and sizes stay readable.
    bool skipped = false;
    for (int i = 10; i < argc; ++i) {
      const std::string name = argv[i];
      if (name == "--skipped") {
        skipped = true;
        continue;
      }
      if (skipped) {
        const lx::ModelWeights::Shape s = m.projection_shape(name);
        const auto per_expert = m.expert_bytes(name);
        std::printf("skipped %s %lld %lld %lld %d %zu %zu %d\n", name.c_str(), static_cast<long long>(s.E), static_cast<long long>(s.N),
                    static_cast<long long>(s.K), s.stack ? 1 : 0, per_expert.first, per_expert.second, m.projection(name) ? 1 : 0);
        continue;
      }
      const lx::WeightView v = m.find(name);
      size_t n = v.dtype == LX_BF16 ? 2 : 4;
      for (int64_t d : v.shape) n *= static_cast<size_t>(d);
      std::printf("plain %s %d %zu", name.c_str(), v.dtype, v.shape.size());
      for (int64_t d : v.shape) std::printf(" %lld", static_cast<long long>(d));
      const long at = dump(v.data, n);
      std::printf(" %ld %zu\n", at, n);
    }
  } catch (const std::exception& e) {
    std::printf("error %s\n", e.what());
  }
  std::fclose(g_blob);
  return 0;
}
