#include "gguf_model.hpp"

#include <fcntl.h>
#include <immintrin.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstring>
#include <stdexcept>
#include <utility>

namespace gufo_hip {
namespace {

[[noreturn]] void Malformed(const std::string& what) { throw std::runtime_error("GGUF: " + what); }

// The fixed-size metadata scalars of the container, by value type number:
// u8 i8 u16 i16 u32 i32 f32 bool | string array | u64 i64 f64.
enum MetaType : std::uint32_t {
  kMetaU8 = 0, kMetaI8, kMetaU16, kMetaI16, kMetaU32, kMetaI32, kMetaF32, kMetaBool,
  kMetaString, kMetaArray, kMetaU64, kMetaI64, kMetaF64,
};

// A bounds-checked walk over the header.
class Walker {
public:
  Walker(const std::uint8_t* data, std::size_t size) : data_(data), size_(size) {}

  template <typename T>
  T Take() {
    T value;
    std::memcpy(&value, Span(sizeof(T)), sizeof(T));
    return value;
  }
  std::string TakeString() {
    const auto length = Take<std::uint64_t>();
    const auto* chars = reinterpret_cast<const char*>(Span(length));
    return std::string(chars, length);
  }
  void Skip(std::uint64_t bytes) { Span(bytes); }
  std::size_t at() const { return at_; }

private:
  const std::uint8_t* Span(std::uint64_t bytes) {
    if (bytes > size_ - at_) Malformed("truncated header");
    const std::uint8_t* start = data_ + at_;
    at_ += static_cast<std::size_t>(bytes);
    return start;
  }
  const std::uint8_t* data_;
  std::size_t size_;
  std::size_t at_ = 0;
};

GgufFile::Value TakeScalar(Walker& in, std::uint32_t type) {
  switch (type) {
    case kMetaU8: return std::uint64_t{in.Take<std::uint8_t>()};
    case kMetaU16: return std::uint64_t{in.Take<std::uint16_t>()};
    case kMetaU32: return std::uint64_t{in.Take<std::uint32_t>()};
    case kMetaU64: return in.Take<std::uint64_t>();
    case kMetaI8: return std::int64_t{in.Take<std::int8_t>()};
    case kMetaI16: return std::int64_t{in.Take<std::int16_t>()};
    case kMetaI32: return std::int64_t{in.Take<std::int32_t>()};
    case kMetaI64: return in.Take<std::int64_t>();
    case kMetaF32: return static_cast<double>(in.Take<float>());
    case kMetaF64: return in.Take<double>();
    case kMetaBool: return in.Take<std::uint8_t>() != 0;
    case kMetaString: return in.TakeString();
    default: Malformed("unknown value type " + std::to_string(type));
  }
}

GgufFile::Value TakeValue(Walker& in, std::uint32_t type) {
  if (type != kMetaArray) return TakeScalar(in, type);
  GgufFile::ArrayOf list;
  list.item_type = in.Take<std::uint32_t>();
  list.count = in.Take<std::uint64_t>();
  if (list.item_type == kMetaArray) Malformed("nested arrays are not supported");
  for (std::uint64_t i = 0; i < list.count; ++i) TakeScalar(in, list.item_type);
  return list;
}

std::string ShapeText(const std::vector<std::uint64_t>& shape) {
  std::string out;
  for (const auto dim : shape) out += (out.empty() ? "" : ", ") + std::to_string(dim);
  return "[" + out + "]";
}

float HalfToFloat(std::uint16_t bits) { return _cvtsh_ss(bits); }

float BFloatToFloat(std::uint16_t bits) {
  const std::uint32_t wide = static_cast<std::uint32_t>(bits) << 16;
  float value;
  std::memcpy(&value, &wide, sizeof value);
  return value;
}

}  // namespace

std::size_t BlockElements(std::uint32_t type) {
  switch (type) {
    case kGgmlF32:
    case kGgmlF16:
    case kGgmlBF16: return 1;
    case kGgmlQ8_0: return 32;
    case kGgmlQ4_K:
    case kGgmlQ5_K:
    case kGgmlQ6_K: return 256;
    default: return 0;
  }
}

std::size_t BlockBytes(std::uint32_t type) {
  switch (type) {
    case kGgmlF32: return 4;
    case kGgmlF16:
    case kGgmlBF16: return 2;
    case kGgmlQ8_0: return 34;
    case kGgmlQ4_K: return 144;
    case kGgmlQ5_K: return 176;
    case kGgmlQ6_K: return 210;
    default: return 0;
  }
}

std::uint64_t GgufTensor::Rows() const {
  std::uint64_t rows = 1;
  for (std::size_t d = 1; d < shape.size(); ++d) rows *= shape[d];
  return rows;
}

// ---- the container ------------------------------------------------------------------

std::unique_ptr<GgufFile> GgufFile::Open(const std::string& path) {
  const int fd = ::open(path.c_str(), O_RDONLY | O_CLOEXEC);
  if (fd < 0) Malformed("cannot open " + path);
  struct stat info {};
  if (::fstat(fd, &info) != 0) {
    ::close(fd);
    Malformed("cannot stat " + path);
  }
  const auto size = static_cast<std::size_t>(info.st_size);
  void* map = size == 0 ? MAP_FAILED : ::mmap(nullptr, size, PROT_READ, MAP_PRIVATE, fd, 0);
  ::close(fd);
  if (map == MAP_FAILED) Malformed("cannot mmap " + path);
  std::unique_ptr<GgufFile> file(new GgufFile());
  file->base_ = static_cast<const std::uint8_t*>(map);
  file->size_ = size;
  file->mapped_ = true;
  file->Parse();
  return file;
}

std::unique_ptr<GgufFile> GgufFile::FromBytes(const std::uint8_t* bytes, std::size_t size) {
  std::unique_ptr<GgufFile> file(new GgufFile());
  file->base_ = bytes;
  file->size_ = size;
  file->Parse();
  return file;
}

GgufFile::~GgufFile() {
  if (mapped_) ::munmap(const_cast<std::uint8_t*>(base_), size_);
}

// Header, metadata, tensor records, padding, data (src/core/gguf.cpp:224-287 of the
// reference reads the same container).
void GgufFile::Parse() {
  Walker in(base_, size_);
  if (in.Take<std::uint32_t>() != 0x46554747u) Malformed("bad magic");  // "GGUF"
  const auto version = in.Take<std::uint32_t>();
  if (version != 3) Malformed("unsupported version " + std::to_string(version));
  const auto n_tensors = in.Take<std::uint64_t>();
  const auto n_values = in.Take<std::uint64_t>();
  for (std::uint64_t i = 0; i < n_values; ++i) {
    std::string key = in.TakeString();
    const auto type = in.Take<std::uint32_t>();
    metadata_.emplace(std::move(key), TakeValue(in, type));
  }
  std::vector<std::uint64_t> offsets;
  for (std::uint64_t i = 0; i < n_tensors; ++i) {
    GgufTensor t;
    t.name = in.TakeString();
    const auto rank = in.Take<std::uint32_t>();
    if (rank == 0 || rank > 4) Malformed("bad rank for " + t.name);
    for (std::uint32_t d = 0; d < rank; ++d) t.shape.push_back(in.Take<std::uint64_t>());
    t.type = in.Take<std::uint32_t>();
    const std::size_t block = BlockElements(t.type);
    if (block == 0) {
      Malformed("unsupported ggml type " + std::to_string(t.type) + " for " + t.name);
    }
    offsets.push_back(in.Take<std::uint64_t>());
    if (t.shape[0] % block != 0) {
      Malformed("row of " + t.name + " is not a whole number of blocks");
    }
    t.bytes = t.shape[0] / block * BlockBytes(t.type) * t.Rows();
    tensors_.push_back(std::move(t));
  }
  std::uint64_t alignment = 32;
  if (const Value* v = Find("general.alignment")) {
    if (const auto* u = std::get_if<std::uint64_t>(v)) alignment = *u;
  }
  if (alignment == 0) Malformed("general.alignment is zero");
  const std::uint64_t data_start = (in.at() + alignment - 1) / alignment * alignment;
  for (std::size_t i = 0; i < tensors_.size(); ++i) {
    GgufTensor& t = tensors_[i];
    const std::uint64_t begin = data_start + offsets[i];
    if (begin > size_ || t.bytes > size_ - begin) {
      Malformed("tensor " + t.name + " runs past the end of the file");
    }
    t.data = base_ + begin;
    by_name_.emplace(t.name, i);
  }
}

const GgufFile::Value* GgufFile::Find(std::string_view key) const {
  const auto it = metadata_.find(key);
  return it == metadata_.end() ? nullptr : &it->second;
}

std::uint64_t GgufFile::GetUInt(std::string_view key) const {
  const Value* v = Find(key);
  if (v == nullptr) Malformed("missing key " + std::string(key));
  if (const auto* u = std::get_if<std::uint64_t>(v)) return *u;
  if (const auto* i = std::get_if<std::int64_t>(v); i != nullptr && *i >= 0) {
    return static_cast<std::uint64_t>(*i);
  }
  Malformed("key " + std::string(key) + " is not an unsigned integer");
}

double GgufFile::GetFloat(std::string_view key) const {
  const Value* v = Find(key);
  const double* f = v == nullptr ? nullptr : std::get_if<double>(v);
  if (f == nullptr) Malformed("missing float key " + std::string(key));
  return *f;
}

std::string GgufFile::GetString(std::string_view key) const {
  const Value* v = Find(key);
  const std::string* s = v == nullptr ? nullptr : std::get_if<std::string>(v);
  if (s == nullptr) Malformed("missing string key " + std::string(key));
  return *s;
}

const GgufTensor* GgufFile::FindTensor(std::string_view name) const {
  const auto it = by_name_.find(name);
  return it == by_name_.end() ? nullptr : &tensors_[it->second];
}

const GgufTensor& GgufFile::Tensor(std::string_view name) const {
  const GgufTensor* t = FindTensor(name);
  if (t == nullptr) Malformed("missing tensor " + std::string(name));
  return *t;
}

// ---- the model's shape ----------------------------------------------------------------

ModelShape ReadShape(const GgufFile& file) {
  ModelShape s;
  s.architecture = file.GetString("general.architecture");
  if (s.architecture != "qwen35" && s.architecture != "qwen35moe") {
    throw std::runtime_error("not a Qwen3.5 GGUF: " + s.architecture);
  }
  const std::string prefix = s.architecture + ".";
  auto number = [&](const char* key) { return static_cast<int>(file.GetUInt(prefix + key)); };
  auto optional = [&](const char* key) {
    return file.Find(prefix + key) == nullptr ? 0 : number(key);
  };
  s.mtp_layers = optional("nextn_predict_layers");
  s.layers = number("block_count") - s.mtp_layers;
  s.hidden = number("embedding_length");
  s.ffn = optional("feed_forward_length");
  s.rms_eps = static_cast<float>(file.GetFloat(prefix + "attention.layer_norm_rms_epsilon"));
  s.full_attention_interval = number("full_attention_interval");
  s.heads = number("attention.head_count");
  s.kv_heads = number("attention.head_count_kv");
  s.head_dim = number("attention.key_length");
  s.rope_dim = number("rope.dimension_count");
  s.rope_theta = static_cast<float>(file.GetFloat(prefix + "rope.freq_base"));
  s.conv_kernel = number("ssm.conv_kernel");
  s.linear_head_dim = number("ssm.state_size");
  s.linear_key_heads = number("ssm.group_count");
  s.linear_value_heads = number("ssm.time_step_rank");
  s.experts = optional("expert_count");
  s.experts_used = optional("expert_used_count");
  s.expert_ffn = optional("expert_feed_forward_length");
  s.shared_expert_ffn = optional("expert_shared_feed_forward_length");

  const GgufTensor& embed = file.Tensor("token_embd.weight");
  if (embed.shape.size() < 2) {
    throw std::runtime_error("qwen35: token_embd.weight has shape " + ShapeText(embed.shape));
  }
  s.vocab = static_cast<int>(embed.shape[1]);
  s.tied_embeddings = file.FindTensor("output.weight") == nullptr;

  if (number("attention.value_length") != s.head_dim) {
    throw std::runtime_error("qwen35: key and value head dims differ");
  }
  if (number("ssm.inner_size") != s.LinearValueDim()) {
    throw std::runtime_error("qwen35: ssm.inner_size != value heads x dim");
  }
  if (s.layers <= 0 || s.full_attention_interval <= 0 || s.kv_heads <= 0 ||
      s.linear_key_heads <= 0 || s.heads % s.kv_heads != 0 ||
      s.linear_value_heads % s.linear_key_heads != 0) {
    throw std::runtime_error("qwen35: inconsistent shape metadata");
  }
  const bool mixture = s.architecture == "qwen35moe";
  const bool experts_ok = s.experts_used > 0 && s.experts_used <= s.experts &&
                          s.expert_ffn > 0 && s.shared_expert_ffn > 0;
  if (mixture != s.IsMoe() || (mixture && !experts_ok) || (!mixture && s.ffn <= 0)) {
    throw std::runtime_error("qwen35: inconsistent FFN or expert metadata");
  }
  return s;
}

bool HasMtpLayer(const GgufFile& file, const ModelShape& shape) {
  return shape.mtp_layers > 0 &&
         file.FindTensor("blk." + std::to_string(shape.layers) + ".nextn.eh_proj.weight") !=
             nullptr;
}

// ---- tensors by stage -----------------------------------------------------------------

std::vector<float> TensorFloats(const GgufTensor& tensor) {
  std::uint64_t count = 1;
  for (const auto dim : tensor.shape) count *= dim;
  std::vector<float> out(static_cast<std::size_t>(count));
  switch (tensor.type) {
    case kGgmlF32:
      std::memcpy(out.data(), tensor.data, out.size() * sizeof(float));
      break;
    case kGgmlF16:
    case kGgmlBF16:
      for (std::size_t i = 0; i < out.size(); ++i) {
        std::uint16_t bits;
        std::memcpy(&bits, tensor.data + 2 * i, 2);
        out[i] = tensor.type == kGgmlF16 ? HalfToFloat(bits) : BFloatToFloat(bits);
      }
      break;
    default:
      throw std::invalid_argument("qwen35: tensor " + tensor.name +
                                  " is block-quantized, not a vector of floats");
  }
  return out;
}

namespace {

// Looks tensors up, checks them and turns them into the records HipProjections takes.
class TableBuilder {
public:
  TableBuilder(const GgufFile& file, StageTable* table) : file_(file), table_(table) {}

  // `name` must be [cols, rows], [cols] when rows is 1, or with `experts`
  // [cols, rows, experts] (CheckShape, gguf_projections.cpp:25-46 of the reference).
  Tensor Checked(const std::string& name, std::uint64_t cols, std::uint64_t rows,
                 std::uint64_t experts = 0) {
    const GgufTensor& t = file_.Tensor(name);
    std::vector<std::uint64_t> want = {cols, rows};
    if (experts != 0) {
      want.push_back(experts);
    } else if (rows == 1 && t.shape.size() == 1) {
      want.pop_back();
    }
    if (t.shape != want) {
      throw std::runtime_error("qwen35: tensor " + t.name + " has shape " + ShapeText(t.shape) +
                               ", expected " + ShapeText(want));
    }
    Tensor out;
    out.name = t.name;
    out.shape = t.shape;
    if (t.type == kGgmlF16 || t.type == kGgmlBF16) {
      table_->widened.push_back(std::make_unique<std::vector<float>>(TensorFloats(t)));
      out.ggml_type = kGgmlF32;
      out.data = reinterpret_cast<const std::uint8_t*>(table_->widened.back()->data());
    } else {
      out.ggml_type = static_cast<int>(t.type);
      out.data = t.data;
    }
    return out;
  }

private:
  const GgufFile& file_;
  StageTable* table_;
};

}  // namespace

StageTable BuildStageTable(const GgufFile& file, const ModelShape& s) {
  StageTable table;
  TableBuilder find(file, &table);
  ModelTensors& model = table.tensors;
  const auto u = [](int v) { return static_cast<std::uint64_t>(v); };
  model.hidden = s.hidden;
  model.experts = s.experts;
  model.expert_ffn = s.expert_ffn;
  // Without output.weight the embedding is the head (tied), gguf_projections.cpp:105-107.
  model.lm_head = find.Checked(s.tied_embeddings ? "token_embd.weight" : "output.weight",
                               u(s.hidden), u(s.vocab));

  const std::uint64_t hidden = u(s.hidden);
  const std::uint64_t attn_dim = u(s.heads * s.head_dim);
  const std::uint64_t kv_dim = u(s.kv_heads * s.head_dim);
  const std::uint64_t key_dim = u(s.LinearKeyDim());
  const std::uint64_t value_dim = u(s.LinearValueDim());
  const std::uint64_t ffn = u(s.FfnWidth());
  const int loaded = s.layers + (HasMtpLayer(file, s) ? 1 : 0);
  for (int il = 0; il < loaded; ++il) {
    const std::string p = "blk." + std::to_string(il) + ".";
    LayerTensors layer;
    if (il >= s.layers) {
      layer.mtp_in = {find.Checked(p + "nextn.eh_proj.weight", 2 * hidden, hidden)};
    }
    if (s.IsMoe()) {
      // [expert logits | shared-expert gate logit]
      layer.router = {find.Checked(p + "ffn_gate_inp.weight", hidden, u(s.experts)),
                      find.Checked(p + "ffn_gate_inp_shexp.weight", hidden, 1)};
      layer.gate_exps =
          find.Checked(p + "ffn_gate_exps.weight", hidden, u(s.expert_ffn), u(s.experts));
      layer.up_exps =
          find.Checked(p + "ffn_up_exps.weight", hidden, u(s.expert_ffn), u(s.experts));
      layer.down_exps =
          find.Checked(p + "ffn_down_exps.weight", u(s.expert_ffn), hidden, u(s.experts));
    }
    // The dense feed-forward block, or the shared expert of a mixture layer.
    const std::string tail = s.IsMoe() ? "_shexp.weight" : ".weight";
    layer.ffn_in = {find.Checked(p + "ffn_gate" + tail, hidden, ffn),
                    find.Checked(p + "ffn_up" + tail, hidden, ffn)};
    layer.ffn_down = {find.Checked(p + "ffn_down" + tail, ffn, hidden)};
    if (s.IsFullAttention(il)) {
      // [q and its gate | k | v]
      layer.attention_in = {find.Checked(p + "attn_q.weight", hidden, 2 * attn_dim),
                            find.Checked(p + "attn_k.weight", hidden, kv_dim),
                            find.Checked(p + "attn_v.weight", hidden, kv_dim)};
      layer.mixer_out = {find.Checked(p + "attn_output.weight", attn_dim, hidden)};
    } else {
      // [qkv | z | alpha | beta]
      layer.linear_in = {find.Checked(p + "attn_qkv.weight", hidden, 2 * key_dim + value_dim),
                         find.Checked(p + "attn_gate.weight", hidden, value_dim),
                         find.Checked(p + "ssm_alpha.weight", hidden, u(s.linear_value_heads)),
                         find.Checked(p + "ssm_beta.weight", hidden, u(s.linear_value_heads))};
      layer.mixer_out = {find.Checked(p + "ssm_out.weight", value_dim, hidden)};
    }
    model.layers.push_back(std::move(layer));
  }
  return table;
}

// ---- a model in HBM -------------------------------------------------------------------

GgufModel::GgufModel(const std::string& path, int device) : file_(GgufFile::Open(path)) {
  shape_ = ReadShape(*file_);
  has_mtp_layer_ = HasMtpLayer(*file_, shape_);
  const StageTable table = BuildStageTable(*file_, shape_);
  auto add_bytes = [&](const Tensor& t) {
    if (t.data == nullptr) return;
    std::uint64_t values = 1;
    for (const auto dim : t.shape) values *= dim;
    const auto type = static_cast<std::uint32_t>(t.ggml_type);
    weight_bytes_ += values / BlockElements(type) * BlockBytes(type);
  };
  add_bytes(table.tensors.lm_head);
  for (const LayerTensors& l : table.tensors.layers) {
    for (const auto* stage : {&l.linear_in, &l.attention_in, &l.mixer_out, &l.ffn_in,
                              &l.ffn_down, &l.router, &l.mtp_in}) {
      for (const Tensor& t : *stage) add_bytes(t);
    }
    add_bytes(l.gate_exps);
    add_bytes(l.up_exps);
    add_bytes(l.down_exps);
  }
  projections_ = std::make_unique<HipProjections>(table.tensors, device);
  output_norm_ = TensorFloats(file_->Tensor("output_norm.weight"));
  for (std::size_t il = 0; il < table.tensors.layers.size(); ++il) {
    const std::string p = "blk." + std::to_string(il) + ".";
    attn_norm_.push_back(TensorFloats(file_->Tensor(p + "attn_norm.weight")));
    post_norm_.push_back(TensorFloats(file_->Tensor(p + "post_attention_norm.weight")));
  }
}

}  // namespace gufo_hip
