// A model folder -> the weights on the device in the formats the products take: lx_ckpt_* (host code; the C form of the
// reference's loader interface, engine/core/checkpoint.h:24-101, whose behaviour engine/core/checkpoint.cpp states).
//
// A folder is safetensors: model.safetensors, or the shards model.safetensors.index.json names. A tensor's dtype names
// its format: BF16; F8_E4M3 with an F32 weight_scale per row (compressed-tensors FP8); U8 nibble pairs with an e4m3
// weight_scale per 16 values and an F32 weight_scale_2 per expert (GPTQ NVFP4). Projections are the matrices the engine
// multiplies by; each is held in the file's own format when the target is the folder's format, else in the format the
// target's recipe gives it, converted on the device by the library's own entry points (lx_dequantize_weight to bf16,
// lx_quantize_weight to the format, lx_bf16x_encode for the lossless target), one expert at a time. Every other BF16 or
// F32 tensor is uploaded as it is. Load-time code: it synchronises freely.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cstring>
#include <fstream>
#include <map>
#include <memory>
#include <sstream>
#include <stdexcept>
#include <string>
#include <string_view>
#include <vector>

#include "common.h"

namespace dro {
namespace ckpt {

[[noreturn]] void refuse(const std::string& why) { throw std::runtime_error(why); }

// ---- the little JSON a safetensors header and index need: objects, arrays, strings, numbers, literals ----------------

struct Json {
  enum Kind { kNull, kBool, kNumber, kString, kArray, kObject } kind = kNull;
  double number = 0;
  bool boolean = false;
  std::string text;
  std::vector<Json> items;
  std::vector<std::pair<std::string, Json>> members;

  const Json* get(std::string_view key) const {
    for (const auto& m : members)
      if (m.first == key) return &m.second;
    return nullptr;
  }
};

class JsonReader {
 public:
  JsonReader(const char* p, size_t n, std::string what) : p_(p), end_(p + n), what_(std::move(what)) {}
  Json document() {
    Json v = value();
    space();
    if (p_ != end_) bad("text after the document");
    return v;
  }

 private:
  // The files this reads nest three deep (header, tensor entry, shape); a value nested deeper than this is refused
  // before the recursion that reads it can run the thread out of stack.
  static constexpr int kMaxDepth = 64;
  const char* p_;
  const char* end_;
  std::string what_;
  int depth_ = 0;

  [[noreturn]] void bad(const char* why) const { refuse(what_ + ": not valid JSON (" + why + ")"); }
  void space() {
    while (p_ < end_ && (*p_ == ' ' || *p_ == '\n' || *p_ == '\t' || *p_ == '\r')) ++p_;
  }
  bool take(char c) {
    space();
    if (p_ < end_ && *p_ == c) {
      ++p_;
      return true;
    }
    return false;
  }
  std::string string() {
    if (!take('"')) bad("a string was expected");
    std::string s;
    while (p_ < end_ && *p_ != '"') {
      char c = *p_++;
      if (c == '\\') {
        if (p_ == end_) bad("a string ends in a backslash");
        const char e = *p_++;
        switch (e) {
          case 'n': c = '\n'; break;
          case 't': c = '\t'; break;
          case 'r': c = '\r'; break;
          case 'b': c = '\b'; break;
          case 'f': c = '\f'; break;
          case 'u': {
            if (end_ - p_ < 4) bad("a short \\u escape");
            const unsigned code = static_cast<unsigned>(std::stoul(std::string(p_, 4), nullptr, 16));
            p_ += 4;
            // Names in these files are ASCII; anything else is kept as UTF-8 of the code unit.
            if (code < 0x80) {
              c = static_cast<char>(code);
            } else if (code < 0x800) {
              s += static_cast<char>(0xc0 | (code >> 6));
              c = static_cast<char>(0x80 | (code & 0x3f));
            } else {
              s += static_cast<char>(0xe0 | (code >> 12));
              s += static_cast<char>(0x80 | ((code >> 6) & 0x3f));
              c = static_cast<char>(0x80 | (code & 0x3f));
            }
            break;
          }
          default: c = e;  // \" \\ \/
        }
      }
      s += c;
    }
    if (p_ == end_) bad("a string does not end");
    ++p_;
    return s;
  }
  Json value() {
    space();
    if (p_ == end_) bad("the text ends early");
    if (*p_ == '{' || *p_ == '[') {
      if (depth_ >= kMaxDepth) bad("objects or arrays nested more than 64 deep");
      ++depth_;
      Json v = nested();
      --depth_;
      return v;
    }
    return scalar();
  }
  Json nested() {
    Json v;
    if (*p_ == '{') {
      ++p_;
      v.kind = Json::kObject;
      if (take('}')) return v;
      do {
        space();
        std::string key = string();
        if (!take(':')) bad("a ':' was expected");
        v.members.emplace_back(std::move(key), value());
      } while (take(','));
      if (!take('}')) bad("a '}' was expected");
    } else if (*p_ == '[') {
      ++p_;
      v.kind = Json::kArray;
      if (take(']')) return v;
      do v.items.push_back(value());
      while (take(','));
      if (!take(']')) bad("a ']' was expected");
    }
    return v;
  }
  Json scalar() {
    Json v;
    if (*p_ == '"') {
      v.kind = Json::kString;
      v.text = string();
    } else if (end_ - p_ >= 4 && !std::strncmp(p_, "true", 4)) {
      v.kind = Json::kBool, v.boolean = true, p_ += 4;
    } else if (end_ - p_ >= 5 && !std::strncmp(p_, "false", 5)) {
      v.kind = Json::kBool, p_ += 5;
    } else if (end_ - p_ >= 4 && !std::strncmp(p_, "null", 4)) {
      p_ += 4;
    } else {
      const char* q = p_;
      while (q < end_ && (std::strchr("+-.eE", *q) || (*q >= '0' && *q <= '9'))) ++q;
      if (q == p_) bad("a value was expected");
      v.kind = Json::kNumber;
      v.number = std::stod(std::string(p_, q));
      p_ = q;
    }
    return v;
  }
};

// ---- the folder --------------------------------------------------------------------------------------------------------

enum class Stored { kBf16, kF32, kFp8, kU8, kI8, kOther };

struct Tensor {
  std::string name, dtype;
  Stored stored = Stored::kOther;
  std::vector<int64_t> shape;
  const uint8_t* data = nullptr;
  size_t bytes = 0;
  int64_t numel() const {
    int64_t n = 1;
    for (int64_t d : shape) n *= d;
    return n;
  }
};

// Bytes per element of a safetensors dtype name; 0 for a name the format does not define.
size_t element_bytes(std::string_view dtype) {
  static const std::pair<const char*, size_t> table[] = {{"F64", 8}, {"F32", 4}, {"F16", 2},  {"BF16", 2}, {"F8_E4M3", 1}, {"F8_E5M2", 1},
                                                         {"I64", 8}, {"I32", 4}, {"I16", 2},  {"I8", 1},   {"U8", 1},      {"BOOL", 1},
                                                         {"U16", 2}, {"U32", 4}, {"U64", 8}};
  for (const auto& e : table)
    if (dtype == e.first) return e.second;
  return 0;
}

class Mapping {
 public:
  explicit Mapping(const std::string& path) {
    const int fd = ::open(path.c_str(), O_RDONLY);
    if (fd < 0) refuse("cannot open " + path + ": " + std::strerror(errno));
    struct stat st {};
    if (::fstat(fd, &st) != 0 || st.st_size < 8) {
      ::close(fd);
      refuse(path + ": too short to be a safetensors file");
    }
    size_ = static_cast<size_t>(st.st_size);
    void* p = ::mmap(nullptr, size_, PROT_READ, MAP_PRIVATE, fd, 0);
    ::close(fd);
    if (p == MAP_FAILED) refuse("cannot map " + path + ": " + std::strerror(errno));
    data_ = static_cast<const uint8_t*>(p);
  }
  Mapping(const Mapping&) = delete;
  Mapping& operator=(const Mapping&) = delete;
  ~Mapping() {
    if (data_) ::munmap(const_cast<uint8_t*>(data_), size_);
  }
  const uint8_t* data() const { return data_; }
  size_t size() const { return size_; }

 private:
  const uint8_t* data_ = nullptr;
  size_t size_ = 0;
};

class Folder {
 public:
  explicit Folder(const std::string& dir) {
    const std::string index = dir + "/model.safetensors.index.json";
    std::ifstream in(index, std::ios::binary);
    if (!in) {
      shard(dir + "/model.safetensors", nullptr);
      return;
    }
    std::stringstream text;
    text << in.rdbuf();
    const std::string body = text.str();
    const Json doc = JsonReader(body.data(), body.size(), index).document();
    const Json* map = doc.get("weight_map");
    if (!map || map->kind != Json::kObject) refuse(index + ": missing \"weight_map\" object");
    // Every shard once, in name order; afterwards every listed tensor must have turned up where the index says.
    std::map<std::string, std::vector<std::string>> by_shard;
    for (const auto& m : map->members) {
      if (m.second.kind != Json::kString) refuse(index + ": shard for \"" + m.first + "\" is not a file name");
      by_shard[m.second.text].push_back(m.first);
    }
    for (const auto& s : by_shard) shard(dir + "/" + s.first, &s.second);
  }

  const std::map<std::string, Tensor>& tensors() const { return tensors_; }
  const Tensor* find(const std::string& name) const {
    const auto it = tensors_.find(name);
    return it == tensors_.end() ? nullptr : &it->second;
  }

 private:
  std::vector<std::unique_ptr<Mapping>> files_;
  std::map<std::string, Tensor> tensors_;

  void shard(const std::string& path, const std::vector<std::string>* listed) {
    files_.push_back(std::make_unique<Mapping>(path));
    const Mapping& f = *files_.back();
    uint64_t header = 0;
    std::memcpy(&header, f.data(), 8);
    if (header > f.size() - 8) refuse(path + ": the header is longer than the file");
    // The format's own limit on a header (100 MB): a longer one is no model's table of tensors.
    if (header > 100u * 1000u * 1000u) refuse(path + ": the header is longer than 100 MB");
    const Json doc = JsonReader(reinterpret_cast<const char*>(f.data()) + 8, static_cast<size_t>(header), path).document();
    if (doc.kind != Json::kObject) refuse(path + ": the header is not an object");
    const uint8_t* base = f.data() + 8 + header;
    const size_t room = f.size() - 8 - static_cast<size_t>(header);
    for (const auto& m : doc.members) {
      if (m.first == "__metadata__") continue;
      const Json *dt = m.second.get("dtype"), *sh = m.second.get("shape"), *off = m.second.get("data_offsets");
      if (!dt || dt->kind != Json::kString || !sh || sh->kind != Json::kArray || !off || off->kind != Json::kArray || off->items.size() != 2)
        refuse(path + ": tensor \"" + m.first + "\" lacks dtype, shape or data_offsets");
      Tensor t;
      t.name = m.first;
      t.dtype = dt->text;
      const size_t esize = element_bytes(t.dtype);
      if (!esize) refuse(path + ": tensor \"" + m.first + "\" has the unknown dtype " + t.dtype);
      t.stored = t.dtype == "BF16" ? Stored::kBf16 : t.dtype == "F32" ? Stored::kF32 : t.dtype == "F8_E4M3" ? Stored::kFp8
                 : t.dtype == "U8" ? Stored::kU8 : t.dtype == "I8" ? Stored::kI8 : Stored::kOther;
      double count = 1;
      for (const Json& d : sh->items) {
        // A dimension is a whole number, and the element count stays far inside what an int64 (and a double) holds exactly.
        if (d.kind != Json::kNumber || !(d.number >= 0) || d.number > 1e15 || d.number != static_cast<double>(static_cast<int64_t>(d.number)))
          refuse(path + ": tensor \"" + m.first + "\" has a bad shape");
        count *= d.number;
        if (count > 1e15) refuse(path + ": tensor \"" + m.first + "\" has a bad shape");
        t.shape.push_back(static_cast<int64_t>(d.number));
      }
      const double b = off->items[0].number, e = off->items[1].number;
      if (off->items[0].kind != Json::kNumber || off->items[1].kind != Json::kNumber || !(b >= 0) || !(e >= b) || e > static_cast<double>(room)) refuse(path + ": tensor \"" + m.first + "\" lies outside the file");
      t.data = base + static_cast<size_t>(b);
      t.bytes = static_cast<size_t>(e - b);
      if (t.bytes != static_cast<size_t>(t.numel()) * esize) refuse(path + ": tensor \"" + m.first + "\" has " + std::to_string(t.bytes) + " bytes, its shape says otherwise");
      if (!tensors_.emplace(t.name, t).second) refuse("tensor \"" + t.name + "\" appears in two shards");
    }
    if (listed)
      for (const std::string& name : *listed) {
        const Tensor* t = find(name);
        if (!t || t->data < f.data() || t->data >= f.data() + f.size()) refuse("index lists \"" + name + "\" in " + path + ", which does not hold it");
      }
  }
};

// ---- names and the recipe ----------------------------------------------------------------------------------------------

// Whether `name` ends with the dotted component(s) `part` ("layers.4.mixer.qkv" ends with "mixer.qkv").
bool ends_with(std::string_view name, std::string_view part) {
  if (name.size() < part.size() || name.substr(name.size() - part.size()) != part) return false;
  return name.size() == part.size() || name[name.size() - part.size() - 1] == '.';
}
bool has(std::string_view s, std::string_view part) { return s.find(part) != std::string_view::npos; }
bool is_expert(std::string_view key) { return has(key, "local_experts."); }
bool is_scale(std::string_view name) { return ends_with(name, "weight_scale") || ends_with(name, "weight_scale_2") || ends_with(name, "input_scale"); }

// The matrices the engine multiplies by, named without ".weight" (engine/core/checkpoint.cpp:99-116); the tied head is
// "embedding".
bool is_projection(std::string_view key) {
  static const char* const parts[] = {"mixer.impl.mixer.in_proj", "mixer.impl.mixer.out_proj", "mixer.qkv", "mixer.out", "mixer.pass_lora_down",
                                      "mixer.pass_lora_up", "moe.latent_down", "moe.latent_up", "moe.shared_expert.gate_up",
                                      "moe.shared_expert.down", "moe.local_experts.gate_up", "moe.local_experts.down", "depth_memory.query",
                                      "depth_memory.state_write", "depth_memory.output", "depth_memory.route_projection", "depth_memory.key",
                                      "depth_memory.value", "depth_memory.metadata_write"};
  if (key == "embedding") return true;
  for (const char* p : parts)
    if (ends_with(key, p)) return true;
  return false;
}

std::string key_of(const std::string& name) {
  return name.size() > 7 && name.compare(name.size() - 7, 7, ".weight") == 0 ? name.substr(0, name.size() - 7) : name;
}

// The format a projection is held in for a target (engine/core/checkpoint.cpp:124-166). In words: the Mamba out_proj, the
// pass LoRA and the depth memory's metadata write stay bf16 everywhere; the depth memory's key and value are FP8 only
// under the NVFP4 target; the tied head is FP8 under NVFP4, bf16 under FP8, the target otherwise; FP8 quantises the
// experts, the Mamba in_proj and the attention qkv and out; NVFP4 the experts (the rest FP8, the MoE latent_up bf16);
// INT8 and BF16X everything else.
int recipe(int target, std::string_view key) {
  if (key == "embedding") return target == LX_W_NVFP4 ? LX_W_FP8 : target == LX_W_FP8 ? LX_W_BF16 : target;
  if (ends_with(key, "mixer.impl.mixer.out_proj") || ends_with(key, "mixer.pass_lora_down") || ends_with(key, "mixer.pass_lora_up") ||
      ends_with(key, "depth_memory.metadata_write"))
    return LX_W_BF16;
  if (ends_with(key, "depth_memory.key") || ends_with(key, "depth_memory.value")) return target == LX_W_NVFP4 ? LX_W_FP8 : LX_W_BF16;
  switch (target) {
    case LX_W_INT8: return LX_W_INT8;
    case LX_W_BF16X: return LX_W_BF16X;
    case LX_W_FP8: {
      const bool quantised = is_expert(key) || ends_with(key, "mixer.impl.mixer.in_proj") || ends_with(key, "mixer.qkv") || ends_with(key, "mixer.out");
      return quantised ? LX_W_FP8 : LX_W_BF16;
    }
    case LX_W_NVFP4: return is_expert(key) ? LX_W_NVFP4 : ends_with(key, "moe.latent_up") ? LX_W_BF16 : LX_W_FP8;
    default: return LX_W_BF16;
  }
}

int stored_format(const Folder& f) {
  bool fp8 = false;
  for (const auto& [name, t] : f.tensors()) {
    if (t.stored == Stored::kU8 && ends_with(name, "weight")) return LX_W_NVFP4;
    if (t.stored == Stored::kFp8) fp8 = true;
  }
  return fp8 ? LX_W_FP8 : LX_W_BF16;
}

size_t data_row_bytes(int type, int64_t K) {
  switch (type) {
    case LX_W_BF16: return 2 * static_cast<size_t>(K);
    case LX_W_NVFP4: return static_cast<size_t>(K / 2);
    case LX_W_BF16X: return static_cast<size_t>(lx_bf16x_row_bytes(static_cast<int>(K)));
    default: return static_cast<size_t>(K);
  }
}
size_t scale_row_bytes(int type, int64_t K) { return type == LX_W_INT8 || type == LX_W_FP8 ? 4 : type == LX_W_NVFP4 ? static_cast<size_t>(K / 16) : 0; }

// ---- the loaded model --------------------------------------------------------------------------------------------------

struct Shape {
  int64_t E = 1, N = 0, K = 0;
  bool stack = false;
};
struct Plain {
  const void* data = nullptr;
  int dtype = LX_F32;
  std::vector<int64_t> shape;
};

struct Model {
  int format = LX_W_BF16;
  std::vector<void*> buffers;
  std::vector<size_t> sizes;
  std::map<std::string, lx_weight> projections;  // on the device
  std::map<std::string, Shape> shapes;           // every projection, loaded or skipped
  std::map<std::string, int> formats;            // and the format it is (or would be) held in
  std::map<std::string, Plain> plain;
  size_t peak = 0;
  ~Model() {
    for (void* b : buffers) (void)lx_rt_free(b);
  }
  size_t device_bytes() const {
    size_t n = 0;
    for (size_t s : sizes) n += s;
    return n;
  }
};

struct Projection {
  std::string key;
  const Tensor *data = nullptr, *scale = nullptr, *global = nullptr;
  int src = LX_W_BF16, dst = LX_W_BF16;
  Shape shape;
};

void must(int status, const std::string& what) {
  if (status != 0) refuse(what + " failed: " + lx_rt_error_string(status));
}

class Loader {
 public:
  Loader(const Folder& f, int target, int stored, bool skip_experts, Model& out)
      : folder_(f), target_(target), stored_(stored), skip_experts_(skip_experts), out_(out) {}
  Loader(const Loader&) = delete;
  Loader& operator=(const Loader&) = delete;
  // The conversion buffers go with the loader, also when run() leaves by an exception (a refused tensor, a failed
  // allocation half way through a folder).
  ~Loader() { release_scratch(); }

  void run() {
    std::vector<Projection> list = collect();  // the map's name order: the device layout does not depend on hash order
    const Projection* head = nullptr;
    for (const Projection& p : list)
      if (p.key == "embedding") head = &p;
    if (!head) refuse("the folder has no embedding.weight");
    plain_tensors();
    size_scratch(list);
    // The gather table is bf16 on the device whatever the folder holds; the tied head comes from it.
    const void* gather = nullptr;
    if (head->src == LX_W_BF16) {
      gather = out_.plain.at("embedding.weight").data;
    } else {
      void* table = keep(static_cast<size_t>(head->shape.N * head->shape.K) * 2);
      expert_as_bf16(*head, 0, table, globals(*head)[0]);
      gather = table;
      out_.plain["embedding.weight"] = Plain{table, LX_BF16, {head->shape.N, head->shape.K}};
    }
    for (const Projection& p : list) {
      if (p.key == "embedding") continue;
      out_.shapes[p.key] = p.shape;
      out_.formats[p.key] = p.dst;
      if (skip_experts_ && is_expert(p.key)) continue;  // its shape and format are kept, its bytes are not
      out_.projections[p.key] = p.dst == p.src ? as_stored(p) : convert(p, nullptr);
    }
    lx_weight h{};
    if (head->dst == LX_W_BF16) {
      h.type = LX_W_BF16, h.data = gather, h.global = 1.0f;
    } else if (head->dst == head->src) {
      h = as_stored(*head);
    } else {
      h = convert(*head, gather);  // from the gather table, which is already bf16 on the device
    }
    out_.projections["lm_head"] = h;
    out_.shapes["lm_head"] = Shape{1, head->shape.N, head->shape.K, false};
    out_.formats["lm_head"] = h.type;
    release_scratch();
    out_.peak = peak_;
  }

 private:
  const Folder& folder_;
  int target_, stored_;
  bool skip_experts_;
  Model& out_;
  size_t live_ = 0, peak_ = 0;
  void *bf16_ = nullptr, *qdata_ = nullptr, *qscale_ = nullptr;
  size_t scratch_bytes_ = 0;

  void* device(size_t bytes) {
    void* p = nullptr;
    must(lx_rt_alloc(&p, static_cast<int64_t>(bytes ? bytes : 1)), "allocating " + std::to_string(bytes) + " bytes");
    live_ += bytes;
    peak_ = std::max(peak_, live_);
    return p;
  }
  void* keep(size_t bytes) {
    void* p = device(bytes);
    out_.buffers.push_back(p);
    out_.sizes.push_back(bytes);
    return p;
  }
  static void upload(void* dst, const void* src, size_t bytes, const std::string& what) {
    if (!bytes) return;
    must(lx_rt_copy(dst, src, static_cast<int64_t>(bytes), LX_COPY_H2D, nullptr), "uploading " + what);
    must(lx_rt_stream_sync(nullptr), "uploading " + what);
  }

  static int format_of(const Tensor& t) {
    switch (t.stored) {
      case Stored::kBf16: return LX_W_BF16;
      case Stored::kFp8: return LX_W_FP8;
      case Stored::kU8: return LX_W_NVFP4;
      case Stored::kI8: return LX_W_INT8;
      default: refuse("a projection cannot be stored as " + t.dtype + " (" + t.name + ")");
    }
  }

  // The scale and global tensors of a quantised projection against the layouts the products take: one f32 scale per row
  // (FP8, INT8); one e4m3 block scale per 16 inputs of each row and one f32 global per expert (NVFP4). A folder that does
  // not match fails here, at load, not in a kernel.
  static void check_layout(const std::string& name, const Projection& p) {
    if (p.src == LX_W_BF16) return;
    const int64_t rows = p.shape.E * p.shape.N;
    if (p.src == LX_W_FP8 || p.src == LX_W_INT8) {
      if (p.scale->stored != Stored::kF32 || p.scale->numel() != rows)
        refuse("projection " + name + " needs one f32 scale per row (" + std::to_string(rows) + " values)");
      return;
    }
    if (p.shape.K % 16 != 0) refuse("NVFP4 projection " + name + " has K = " + std::to_string(p.shape.K) + ", not a multiple of 16");
    if (p.scale->stored != Stored::kFp8 || p.scale->numel() != rows * (p.shape.K / 16))
      refuse("NVFP4 projection " + name + " needs one e4m3 block scale per 16 inputs (" + std::to_string(rows * (p.shape.K / 16)) + " values)");
    if (!p.global) refuse("projection " + name + " has no weight_scale_2");
    const int64_t wanted = p.shape.stack ? p.shape.E : 1;
    if (p.global->stored != Stored::kF32 || p.global->numel() != wanted)
      refuse("NVFP4 projection " + name + " needs one f32 global per expert (" + std::to_string(wanted) + " values)");
  }

  std::vector<Projection> collect() const {
    std::vector<Projection> list;
    for (const auto& [name, t] : folder_.tensors()) {
      if (!ends_with(name, "weight") || name.size() <= 7) continue;
      const std::string key = key_of(name);
      if (has(name, "ngram") || name == "lm_head.weight" || !is_projection(key)) continue;
      Projection p;
      p.key = key;
      p.data = &t;
      p.scale = folder_.find(key + ".weight_scale");
      p.global = folder_.find(key + ".weight_scale_2");
      p.src = format_of(t);
      if (t.shape.size() == 3) p.shape.stack = true, p.shape.E = t.shape[0], p.shape.N = t.shape[1];
      else if (t.shape.size() == 2) p.shape.N = t.shape[0];
      else refuse("projection " + name + " has rank " + std::to_string(t.shape.size()));
      p.shape.K = p.src == LX_W_NVFP4 ? 2 * t.shape.back() : t.shape.back();
      if (p.src != LX_W_BF16 && !p.scale) refuse("projection " + name + " is quantized but has no weight_scale");
      check_layout(name, p);
      p.dst = target_ == stored_ ? p.src : recipe(target_, key);
      list.push_back(std::move(p));
    }
    return list;
  }

  std::vector<float> globals(const Projection& p) const {
    std::vector<float> g(static_cast<size_t>(p.shape.stack ? p.shape.E : 1), 1.0f);
    if (p.src == LX_W_NVFP4) std::memcpy(g.data(), p.global->data, g.size() * sizeof(float));
    return g;
  }

  // Every BF16 or F32 tensor that is neither a scale nor a projection's data (the gather table excepted), in one buffer.
  void plain_tensors() {
    std::vector<const Tensor*> list;
    size_t total = 0;
    for (const auto& [name, t] : folder_.tensors()) {
      if (is_scale(name) || has(name, "ngram") || name == "lm_head.weight") continue;
      if (t.stored != Stored::kBf16 && t.stored != Stored::kF32) continue;
      if (name != "embedding.weight" && ends_with(name, "weight") && name.size() > 7 && is_projection(key_of(name))) continue;
      list.push_back(&t);
      total += (t.bytes + 255) / 256 * 256;
    }
    uint8_t* base = static_cast<uint8_t*>(keep(total));
    size_t at = 0;
    for (const Tensor* t : list) {
      upload(base + at, t->data, t->bytes, t->name);
      out_.plain[t->name] = Plain{base + at, t->stored == Stored::kBf16 ? LX_BF16 : LX_F32, t->shape};
      at += (t->bytes + 255) / 256 * 256;
    }
  }

  // What a conversion needs beside the result: one expert's bf16 values (a whole stack's for the lossless target, which
  // encodes a stack in one piece) and, for a quantised folder, one expert's bytes and scales.
  void size_scratch(const std::vector<Projection>& list) {
    size_t bf16 = 0, data = 0, scale = 0;
    for (const Projection& p : list) {
      if (skip_experts_ && is_expert(p.key)) continue;
      // Held as the file has it: uploaded to its place, nothing converted (but a quantised embedding is always
      // dequantised once, into the gather table).
      if (p.dst == p.src && !(p.key == "embedding" && p.src != LX_W_BF16)) continue;
      if (p.key != "embedding") bf16 = std::max(bf16, static_cast<size_t>(p.dst == LX_W_BF16X ? p.shape.E : 1) * p.shape.N * p.shape.K * 2);
      if (p.src == LX_W_BF16) continue;
      data = std::max(data, static_cast<size_t>(p.shape.N) * data_row_bytes(p.src, p.shape.K));
      scale = std::max(scale, static_cast<size_t>(p.shape.N) * scale_row_bytes(p.src, p.shape.K));
    }
    bf16_ = device(bf16), scratch_bytes_ = bf16;
    qdata_ = device(data), scratch_bytes_ += data;
    qscale_ = device(scale), scratch_bytes_ += scale;
  }
  void release_scratch() {
    for (void** p : {&bf16_, &qdata_, &qscale_}) {
      if (*p) (void)lx_rt_free(*p);
      *p = nullptr;
    }
    live_ -= scratch_bytes_;
    scratch_bytes_ = 0;
  }

  // Expert e of a projection (the whole matrix of a plain one) as bf16 at `dst` on the device.
  void expert_as_bf16(const Projection& p, int64_t e, void* dst, float global) const {
    const int64_t N = p.shape.N, K = p.shape.K;
    if (p.src == LX_W_BF16) {
      upload(dst, p.data->data + e * N * K * 2, static_cast<size_t>(N * K * 2), p.key);
      return;
    }
    const size_t db = static_cast<size_t>(N) * data_row_bytes(p.src, K), sb = static_cast<size_t>(N) * scale_row_bytes(p.src, K);
    upload(qdata_, p.data->data + e * static_cast<int64_t>(db), db, p.key);
    upload(qscale_, p.scale->data + e * static_cast<int64_t>(sb), sb, p.key + ".weight_scale");
    lx_weight w{static_cast<lx_wtype>(p.src), qdata_, qscale_, global, nullptr};
    must(lx_dequantize_weight(&w, dst, N, static_cast<int>(K), nullptr), "dequantizing " + p.key);
    must(lx_rt_stream_sync(nullptr), "dequantizing " + p.key);
  }

  const float* expert_globals(const std::vector<float>& g) {
    void* d = keep(g.size() * sizeof(float));
    upload(d, g.data(), g.size() * sizeof(float), "expert globals");
    return static_cast<const float*>(d);
  }

  // The file's bytes, copied.
  lx_weight as_stored(const Projection& p) {
    const std::vector<float> g = globals(p);
    lx_weight w{};
    w.type = static_cast<lx_wtype>(p.src);
    void* data = keep(p.data->bytes);
    upload(data, p.data->data, p.data->bytes, p.key);
    w.data = data;
    if (p.scale) {
      void* s = keep(p.scale->bytes);
      upload(s, p.scale->data, p.scale->bytes, p.key + ".weight_scale");
      w.scale = s;
    }
    w.global = g[0];
    if (p.src == LX_W_NVFP4 && p.shape.stack) w.expert_global = expert_globals(g);
    return w;
  }

  // To the target's format, an expert at a time; `from` (a bf16 matrix on the device) stands in for the file's values
  // where they are on the device already, as the tied head's are.
  lx_weight convert(const Projection& p, const void* from) {
    const Shape& s = p.shape;
    const std::vector<float> src_globals = globals(p);
    lx_weight w{};
    w.type = static_cast<lx_wtype>(p.dst);
    w.global = 1.0f;
    if (p.dst == LX_W_BF16X) {
      // A stack is one encoding of E * N rows (its spill records follow all rows), so its bf16 values are gathered first.
      const void* bf16 = from;
      if (!bf16) {
        for (int64_t e = 0; e < s.E; ++e) expert_as_bf16(p, e, static_cast<uint8_t*>(bf16_) + static_cast<size_t>(e * s.N * s.K) * 2, src_globals[e]);
        bf16 = bf16_;
      }
      const int64_t need = lx_bf16x_bytes(bf16, s.E * s.N, static_cast<int>(s.K), nullptr);
      if (need < 0) refuse("lossless size of " + p.key + " failed");
      void* data = keep(static_cast<size_t>(need));
      must(lx_bf16x_encode(bf16, s.E * s.N, static_cast<int>(s.K), data, need, nullptr), "encoding " + p.key);
      must(lx_rt_stream_sync(nullptr), "encoding " + p.key);
      w.data = data;
      return w;
    }
    const size_t per_row = data_row_bytes(p.dst, s.K), per_scale = scale_row_bytes(p.dst, s.K);
    uint8_t* data = static_cast<uint8_t*>(keep(static_cast<size_t>(s.E * s.N) * per_row));
    uint8_t* scale = per_scale ? static_cast<uint8_t*>(keep(static_cast<size_t>(s.E * s.N) * per_scale)) : nullptr;
    std::vector<float> dst_globals(static_cast<size_t>(s.E), 1.0f);
    for (int64_t e = 0; e < s.E; ++e) {
      const void* bf16 = from;
      if (!bf16) {
        expert_as_bf16(p, e, bf16_, src_globals[e]);
        bf16 = bf16_;
      }
      if (p.dst == LX_W_BF16) {
        must(lx_rt_copy(data + e * s.N * per_row, bf16, s.N * s.K * 2, LX_COPY_D2D, nullptr), "copying " + p.key);
      } else {
        lx_weight q{static_cast<lx_wtype>(p.dst), data + e * s.N * static_cast<int64_t>(per_row),
                    scale ? scale + e * s.N * static_cast<int64_t>(per_scale) : nullptr, 1.0f, nullptr};
        must(lx_quantize_weight(bf16, &q, s.N, static_cast<int>(s.K), nullptr), "quantizing " + p.key);
        dst_globals[e] = q.global;
      }
      must(lx_rt_stream_sync(nullptr), "converting " + p.key);
    }
    w.data = data;
    w.scale = scale;
    w.global = dst_globals[0];
    if (p.dst == LX_W_NVFP4 && s.stack) w.expert_global = expert_globals(dst_globals);
    return w;
  }
};

thread_local std::string g_error;

int failed(const std::exception& e) {
  g_error = e.what();
  return fail(kInvalid);
}

// Why NVFP4 cannot load from a folder stored otherwise (engine/core/checkpoint.cpp:193-197).
std::string nvfp4_refusal(int stored) {
  return std::string("NVFP4 from ") + (stored == LX_W_FP8 ? "an FP8" : "a BF16") +
         " checkpoint is refused: round-to-nearest conversion fails its KL. No NVFP4 checkpoint of this model is published yet.";
}

}  // namespace ckpt
}  // namespace dro

using namespace dro;
using namespace dro::ckpt;

struct lx_ckpt {
  Model model;
  std::vector<std::string> names;
};

extern "C" {

const char* lx_ckpt_error(void) { return g_error.c_str(); }

int lx_ckpt_projection_format(lx_wtype target, const char* projection) {
  if (!projection) return -1;
  return recipe(target, key_of(projection));
}

int lx_ckpt_stored_format(const char* dir) {
  try {
    if (!dir) refuse("no folder");
    return stored_format(Folder(dir));
  } catch (const std::exception& e) {
    failed(e);
    return -1;
  }
}

int lx_ckpt_load(const char* dir, lx_wtype target, int skip_experts, lx_ckpt** out) {
  if (!dir || !out) return fail(kInvalid);
  *out = nullptr;
  try {
    if (target < LX_W_BF16 || target > LX_W_BF16X) refuse("no such target format");
    const Folder folder(dir);
    const int stored = stored_format(folder);
    if (target == LX_W_NVFP4 && stored != LX_W_NVFP4) refuse(nvfp4_refusal(stored));
    auto handle = std::make_unique<lx_ckpt>();
    handle->model.format = target;
    Loader(folder, target, stored, skip_experts != 0, handle->model).run();
    for (const auto& p : handle->model.projections) handle->names.push_back(p.first);
    *out = handle.release();
    return kOk;
  } catch (const std::exception& e) {
    return failed(e);
  }
}

void lx_ckpt_free(lx_ckpt* c) { delete c; }

const lx_weight* lx_ckpt_projection(const lx_ckpt* c, const char* name) {
  if (!c || !name) return nullptr;
  const auto it = c->model.projections.find(key_of(name));
  return it == c->model.projections.end() ? nullptr : &it->second;
}

int lx_ckpt_count(const lx_ckpt* c) { return c ? static_cast<int>(c->names.size()) : 0; }
const char* lx_ckpt_name(const lx_ckpt* c, int i) { return c && i >= 0 && i < static_cast<int>(c->names.size()) ? c->names[i].c_str() : nullptr; }

int lx_ckpt_shape(const lx_ckpt* c, const char* name, int64_t* E, int64_t* N, int64_t* K, int* stack) {
  if (!c || !name) return fail(kInvalid);
  const auto it = c->model.shapes.find(key_of(name));
  if (it == c->model.shapes.end()) return fail(kInvalid);
  if (E) *E = it->second.E;
  if (N) *N = it->second.N;
  if (K) *K = it->second.K;
  if (stack) *stack = it->second.stack ? 1 : 0;
  return kOk;
}

int lx_ckpt_format_of(const lx_ckpt* c, const char* name) {
  if (!c || !name) return -1;
  const auto it = c->model.formats.find(key_of(name));
  return it == c->model.formats.end() ? -1 : it->second;
}

int lx_ckpt_expert(const lx_ckpt* c, const char* name, int64_t e, lx_weight* out) {
  if (!c || !name || !out) return fail(kInvalid);
  const lx_weight* w = lx_ckpt_projection(c, name);
  try {
    if (!w) refuse(c->model.formats.count(key_of(name)) ? std::string(name) + " is not on the device: skip_experts left it off" : std::string("no projection ") + name);
    const Shape s = c->model.shapes.at(key_of(name));
    if (e < 0 || e >= s.E) refuse("expert " + std::to_string(e) + " is out of range for " + name);
    *out = *w;
    out->data = static_cast<const uint8_t*>(w->data) + static_cast<size_t>(e * s.N) * data_row_bytes(w->type, s.K);
    if (w->scale) out->scale = static_cast<const uint8_t*>(w->scale) + static_cast<size_t>(e * s.N) * scale_row_bytes(w->type, s.K);
    out->expert_global = nullptr;
    if (w->expert_global) {
      float g = 1.0f;
      must(lx_rt_copy(&g, w->expert_global + e, sizeof(float), LX_COPY_D2H, nullptr), "reading the expert global");
      must(lx_rt_stream_sync(nullptr), "reading the expert global");
      out->global = g;
    }
    return kOk;
  } catch (const std::exception& ex) {
    return failed(ex);
  }
}

int lx_ckpt_expert_bytes(const lx_ckpt* c, const char* name, int64_t* data, int64_t* scale) {
  if (!c || !name) return fail(kInvalid);
  const std::string key = key_of(name);
  const auto f = c->model.formats.find(key);
  if (f == c->model.formats.end()) return fail(kInvalid);
  const Shape s = c->model.shapes.at(key);
  if (data) *data = static_cast<int64_t>(static_cast<size_t>(s.N) * data_row_bytes(f->second, s.K));
  if (scale) *scale = static_cast<int64_t>(static_cast<size_t>(s.N) * scale_row_bytes(f->second, s.K));
  return kOk;
}

const void* lx_ckpt_tensor(const lx_ckpt* c, const char* name, lx_dtype* dtype, int* rank, int64_t* shape, int capacity) {
  if (!c || !name) return nullptr;
  const auto it = c->model.plain.find(name);
  if (it == c->model.plain.end()) return nullptr;
  if (dtype) *dtype = static_cast<lx_dtype>(it->second.dtype);
  if (rank) *rank = static_cast<int>(it->second.shape.size());
  for (int i = 0; shape && i < capacity && i < static_cast<int>(it->second.shape.size()); ++i) shape[i] = it->second.shape[i];
  return it->second.data;
}

int lx_ckpt_target(const lx_ckpt* c) { return c ? c->model.format : -1; }
int64_t lx_ckpt_device_bytes(const lx_ckpt* c) { return c ? static_cast<int64_t>(c->model.device_bytes()) : 0; }
int64_t lx_ckpt_peak_device_bytes(const lx_ckpt* c) { return c ? static_cast<int64_t>(c->model.peak) : 0; }

}  // extern "C"
