// Real model files for the MI355X backend: a GGUF v3 reader, the shape of a Qwen3.5 /
// Qwen3.6 text model read from its metadata, and the table that says which tensors of
// the file make up which stage of the forward pass.
//
// This is the part of the reference that sits between a .gguf file and its
// `Projections`: gguf::File (src/core/gguf.hpp:13-86, src/core/gguf.cpp:224-287),
// qwen35::ReadConfig (src/models/qwen35/config.cpp:18-72) and the constructor of
// GgufProjections (src/models/qwen35/gguf_projections.cpp:100-175).  Same keys, same
// tensor names, same shape checks, same exceptions (std::runtime_error with the
// offending name in the message); the result is a ModelTensors record that
// HipProjections uploads.  The reader maps the file and copies nothing: tensor bytes go
// from the page cache straight into the upload.
#pragma once

#include <cstddef>
#include <cstdint>
#include <map>
#include <memory>
#include <string>
#include <string_view>
#include <variant>
#include <vector>

#include "hip_projections.hpp"

namespace gufo_hip {

// ggml tensor types a model file may hold (gguf::GgmlType, src/core/gguf.hpp:16-24).
// The two 16-bit types occur in small tensors only; they are widened to fp32 when the
// stage table is built, which is also what the reference does before it multiplies
// them (gguf_projections.cpp:56-60).
enum GgmlType : std::uint32_t {
  kGgmlF32 = 0,
  kGgmlF16 = 1,
  kGgmlQ8_0 = 8,
  kGgmlQ4_K = 12,
  kGgmlQ5_K = 13,
  kGgmlQ6_K = 14,
  kGgmlBF16 = 30,
};

// Values per block and bytes per block of a type (quant::BlockElements / BlockBytes,
// src/core/quant.cpp:186-219); 0 for a type outside the list above.
std::size_t BlockElements(std::uint32_t type);
std::size_t BlockBytes(std::uint32_t type);

struct GgufTensor {
  std::string name;
  std::vector<std::uint64_t> shape;  // ggml order: shape[0] is the contiguous dimension
  std::uint32_t type = kGgmlF32;
  std::uint64_t bytes = 0;
  const std::uint8_t* data = nullptr;

  std::uint64_t RowElements() const { return shape.empty() ? 1 : shape[0]; }
  std::uint64_t Rows() const;  // product of the other dimensions
};

class GgufFile {
public:
  // A metadata value.  Arrays are stepped over: nothing on this path reads one (the
  // tokenizer's lists are the only arrays in these files); only their length is kept.
  struct ArrayOf {
    std::uint32_t item_type = 0;
    std::uint64_t count = 0;
  };
  using Value = std::variant<std::uint64_t, std::int64_t, double, bool, std::string, ArrayOf>;

  // Both throw std::runtime_error for I/O errors and malformed files, with the
  // reference's wording ("GGUF: bad magic", "GGUF: truncated header", ...).
  static std::unique_ptr<GgufFile> Open(const std::string& path);
  // `bytes` must outlive the object.
  static std::unique_ptr<GgufFile> FromBytes(const std::uint8_t* bytes, std::size_t size);
  ~GgufFile();
  GgufFile(const GgufFile&) = delete;
  GgufFile& operator=(const GgufFile&) = delete;

  const Value* Find(std::string_view key) const;
  // Typed getters; throw std::runtime_error when the key is missing or of another kind.
  // GetUInt also takes a signed value that is not negative.
  std::uint64_t GetUInt(std::string_view key) const;
  double GetFloat(std::string_view key) const;
  std::string GetString(std::string_view key) const;

  const GgufTensor* FindTensor(std::string_view name) const;
  const GgufTensor& Tensor(std::string_view name) const;  // throws if absent
  const std::vector<GgufTensor>& Tensors() const { return tensors_; }
  std::size_t MetadataCount() const { return metadata_.size(); }

private:
  GgufFile() = default;
  void Parse();

  const std::uint8_t* base_ = nullptr;
  std::size_t size_ = 0;
  bool mapped_ = false;
  std::map<std::string, Value, std::less<>> metadata_;
  std::vector<GgufTensor> tensors_;
  std::map<std::string, std::size_t, std::less<>> by_name_;
};

// qwen35::Config (src/models/qwen35/config.hpp:13-60), field for field.
struct ModelShape {
  std::string architecture;
  int layers = 0;      // decoder layers, without the MTP layers stored after them
  int mtp_layers = 0;
  int hidden = 0;
  int ffn = 0;  // dense FFN width, 0 for a mixture model
  int vocab = 0;
  float rms_eps = 0;
  int full_attention_interval = 0;
  int heads = 0;
  int kv_heads = 0;
  int head_dim = 0;
  int rope_dim = 0;
  float rope_theta = 0;
  int conv_kernel = 0;
  int linear_key_heads = 0;
  int linear_value_heads = 0;
  int linear_head_dim = 0;
  int experts = 0;
  int experts_used = 0;
  int expert_ffn = 0;
  int shared_expert_ffn = 0;
  bool tied_embeddings = false;

  bool IsMoe() const { return experts > 0; }
  int FfnWidth() const { return IsMoe() ? shared_expert_ffn : ffn; }
  bool IsFullAttention(int layer) const {
    return layer >= layers || (layer + 1) % full_attention_interval == 0;
  }
  int LinearKeyDim() const { return linear_key_heads * linear_head_dim; }
  int LinearValueDim() const { return linear_value_heads * linear_head_dim; }
};

// ReadConfig: throws std::runtime_error when the file is not a Qwen3.5 model, a key is
// missing or the shape metadata contradicts itself.
ModelShape ReadShape(const GgufFile& file);
// HasMtpLayer (config.cpp:74-78): the file declares MTP layers and holds the first one.
bool HasMtpLayer(const GgufFile& file, const ModelShape& shape);

// The tensors of every layer by stage, ready for HipProjections, plus the storage of
// the 16-bit tensors that had to be widened.  `file` must outlive the record.
struct StageTable {
  ModelTensors tensors;
  std::vector<std::unique_ptr<std::vector<float>>> widened;
};
// The constructor of GgufProjections: looks every tensor up by name, checks its shape
// against `shape` (std::runtime_error "qwen35: tensor <name> has shape [..], expected
// [..]") and files it under its stage.  Layers [0, shape.layers) and, if present, the
// MTP layer at index shape.layers.
StageTable BuildStageTable(const GgufFile& file, const ModelShape& shape);

// The fp32 vector a decoder keeps beside the products: any tensor of the file as
// floats (Decoder's ToFloats, src/models/qwen35/decoder.cpp:19-23,449-454): F32 as is,
// F16 and BF16 widened.  The norm weights of these files are F32; a block-quantized
// tensor throws std::invalid_argument.
std::vector<float> TensorFloats(const GgufTensor& tensor);

// A model file opened for this backend: the mapped file, its shape, the weights in HBM
// behind the Projections interface, and the norm weights of every layer.
class GgufModel {
public:
  // Throws what GgufFile::Open, ReadShape, BuildStageTable and HipProjections throw.
  explicit GgufModel(const std::string& path, int device = 0);

  const ModelShape& shape() const { return shape_; }
  const HipProjections& projections() const { return *projections_; }
  bool has_mtp_layer() const { return has_mtp_layer_; }
  // attn_norm / post_attention_norm of layer il (MTP layer included), output_norm.
  const std::vector<float>& attn_norm(int layer) const { return attn_norm_.at(layer); }
  const std::vector<float>& post_attention_norm(int layer) const {
    return post_norm_.at(layer);
  }
  const std::vector<float>& output_norm() const { return output_norm_; }
  // Bytes of weights uploaded, and tensor records in the file.
  std::uint64_t weight_bytes() const { return weight_bytes_; }
  std::size_t tensor_count() const { return file_->Tensors().size(); }

private:
  std::unique_ptr<GgufFile> file_;
  ModelShape shape_;
  bool has_mtp_layer_ = false;
  std::unique_ptr<HipProjections> projections_;
  std::vector<std::vector<float>> attn_norm_;
  std::vector<std::vector<float>> post_norm_;
  std::vector<float> output_norm_;
  std::uint64_t weight_bytes_ = 0;
};

}  // namespace gufo_hip
