// C++ host side of the MI355X backend: the reference's operator interface for the
// matrix products of a Qwen3.5 / Qwen3.6 forward pass, served by the C-ABI library
// (include/gufo_hip.h).
//
// `Stage` and `Projections` repeat qwen35::Stage and qwen35::Projections
// (src/models/qwen35/projections.hpp:14-59 of the reference) name for name, so a
// consumer that holds a `const Projections&` (Decoder, Reference, the test
// decorators) can be handed a HipProjections.  HipProjections takes the place of
// GgufProjections (src/models/qwen35/gguf_projections.hpp:19-58): same methods, same
// output layout (each row one token, the stage's matrices concatenated), same
// exceptions.  Where GgufProjections reads its tensors out of a mapped GGUF file,
// this class is handed them as `Tensor` records - the GGUF reader itself is not part
// of this backend - and copies them to HBM once.
#pragma once

#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>
#include <vector>

struct gufo_hip_matrix;

namespace gufo_hip {

// qwen35::Stage (projections.hpp:14-39): the products grouped by shared input.
enum class Stage {
  kLinearIn,     // [qkv | z | alpha | beta]
  kAttentionIn,  // [q and gate | k | v]
  kMixerOut,     // ssm_out or attn_output: hidden
  kFfnIn,        // [gate | up]: the dense FFN or the MoE shared expert
  kFfnDown,      // ffn_down: hidden
  kLmHead,       // vocab
  kRouter,       // [expert logits | shared-expert gate logit]
  kExpertIn,     // a routed expert's [gate | up]; ApplyExpert only
  kExpertDown,   // a routed expert's down projection; ApplyExpert only
  kMtpIn,        // nextn.eh_proj
};

// qwen35::Projections (projections.hpp:45-59).
class Projections {
public:
  virtual ~Projections() = default;
  // y[t] = W x[t] for `tokens` rows of the stage's input width; writes `tokens` rows of
  // the stage's output width.
  virtual void Apply(Stage stage, int layer, const float* x, int tokens, float* y) const = 0;
  // The same for routed expert `expert` of an MoE layer (kExpertIn or kExpertDown).
  virtual void ApplyExpert(Stage /*stage*/, int /*layer*/, int /*expert*/, const float* /*x*/,
                           int /*tokens*/, float* /*y*/) const {
    throw std::logic_error("qwen35: these projections have no MoE experts");
  }
};

// A weight tensor as a GGUF file describes it (gguf::TensorInfo,
// src/core/gguf.hpp:40-54): ggml order, shape[0] is the contiguous (row) dimension, so
// a matrix is [cols, rows] and an expert tensor [cols, rows, experts].  `data` points
// at the blocks as stored; it is read during construction only.
struct Tensor {
  std::string name;
  int ggml_type = 0;  // 0 = F32, 8 = Q8_0, 12 = Q4_K, 13 = Q5_K, 14 = Q6_K
  std::vector<std::uint64_t> shape;
  const std::uint8_t* data = nullptr;
};

// The tensors of one layer by stage, as GgufProjections::Layer groups them
// (gguf_projections.cpp:80-91).  A stage a layer does not have stays empty.
struct LayerTensors {
  std::vector<Tensor> linear_in;
  std::vector<Tensor> attention_in;
  std::vector<Tensor> mixer_out;
  std::vector<Tensor> ffn_in;
  std::vector<Tensor> ffn_down;
  std::vector<Tensor> router;
  std::vector<Tensor> mtp_in;
  // MoE layers: ffn_gate_exps, ffn_up_exps [hidden, expert_ffn, experts] and
  // ffn_down_exps [expert_ffn, hidden, experts].  Leave `data` null for a dense layer.
  Tensor gate_exps;
  Tensor up_exps;
  Tensor down_exps;
};

struct ModelTensors {
  int hidden = 0;
  int experts = 0;     // 0 for a dense model
  int expert_ffn = 0;
  Tensor lm_head;      // [hidden, vocab]
  std::vector<LayerTensors> layers;
};

class HipProjections : public Projections {
public:
  // Initialises the library on `device`, checks every tensor's shape and uploads the
  // weights.  Throws std::runtime_error when no MI355X is available (as the
  // reference's NPU stub does, src/npu/gemv_stub.cpp:8-10) or a shape is wrong
  // (gguf_projections.cpp:27-46), std::invalid_argument for a row that is not a whole
  // number of blocks or a type this backend does not take (src/core/quant.cpp:199,224).
  explicit HipProjections(const ModelTensors& model, int device = 0);
  ~HipProjections() override;
  HipProjections(const HipProjections&) = delete;
  HipProjections& operator=(const HipProjections&) = delete;

  void Apply(Stage stage, int layer, const float* x, int tokens, float* y) const override;
  void ApplyExpert(Stage stage, int layer, int expert, const float* x, int tokens,
                   float* y) const override;

  // Input and output widths of a stage (StageInputs / StageOutputs,
  // src/models/qwen35/reference.cpp:609-648), from the uploaded tensors.
  std::size_t StageInputs(Stage stage, int layer) const;
  std::size_t StageOutputs(Stage stage, int layer) const;

  // A stage on rows that stay in device memory, with the elementwise step the decoder
  // runs before it taken into the product - the reference's NPU products work the same
  // way (npu::Prologue and Q4nxGemv::Run(x, y, residual, tokens),
  // src/npu/gemv.hpp:58-63,146-150).  All pointers are device memory
  // (gufo_hip_malloc); the call is enqueued, not waited for.
  enum class Prologue {
    kPlain,    // x: tokens x StageInputs
    kSwiGlu,   // x: tokens x 2*StageInputs rows [gate | up] -> silu(gate) * up
               // (decoder.cpp:511-514); the kFfnIn output feeds kFfnDown directly
    kResNorm,  // RmsNorm(x + delta) * norm_weight (decoder.cpp:493,504-509); x + delta
               // goes to `residual`, the normalized rows to `normed` (either may be null)
  };
  struct DeviceInput {
    Prologue prologue = Prologue::kPlain;
    const float* x = nullptr;
    const float* delta = nullptr;        // kResNorm, may be null
    const float* norm_weight = nullptr;  // kResNorm
    float eps = 0.0f;                    // kResNorm: Config::rms_eps
    float* residual = nullptr;
    float* normed = nullptr;
  };
  void ApplyDevice(Stage stage, int layer, const DeviceInput& in, int tokens, float* y) const;
  // The stage's product with the greedy pick inside: index[t] (device memory) receives
  // the position of the first maximum of the stage's output row for token t, which is
  // never stored.  For Stage::kLmHead that is the greedy token (std::max_element over
  // the logits, src/core/sampling.cpp:327-329).  kPlain and kResNorm inputs.
  void PickDevice(Stage stage, int layer, const DeviceInput& in, int tokens,
                  std::int64_t* index) const;

  // A stage for many tokens at once on the matrix cores, the prefill shape: a_bf16
  // (device, tokens x stage input, bf16 as the reference's NPU prefill GEMM takes its
  // activations, src/npu/gemm.hpp:99-105), c (device) tokens x stage output fp32 in
  // Apply's layout.  Quantized row types only; held to 1e-3 relative, not Apply's 1e-4
  // (fp16 operands).  Enqueued, not waited for.
  void PrefillDevice(Stage stage, int layer, const std::uint16_t* a_bf16, std::size_t tokens,
                     float* c) const;
  // Keeps the stage's weights in PrefillDevice's own form as well (3.5 x their packed
  // size) so that later calls convert only their activations.
  void PreparePrefill(Stage stage, int layer);

  // The resident matrices of a stage, in the order of its parts, and the three expert
  // tensors of a mixture layer (gate, up, down; null for a dense layer): for callers that
  // drive the C entry points of gufo_hip.h themselves.  They belong to this object.
  std::vector<const gufo_hip_matrix*> StageHandles(Stage stage, int layer) const;
  void ExpertHandles(int layer, const gufo_hip_matrix** gate, const gufo_hip_matrix** up,
                     const gufo_hip_matrix** down) const;

  // qwen35::Route (src/models/qwen35/moe.cpp:16-42) on the device.
  void Route(const float* logits, int tokens, int k, int* chosen, float* weights) const;
  // The routed experts of one MoE layer in one call: what Decoder::MoeFfn /
  // Reference::Ffn compute with a Route and 2 k ApplyExpert calls
  // (src/models/qwen35/decoder.cpp:530-558, reference.cpp:562-606), without the
  // shared expert.  Tokens are grouped by expert on the device.
  void RoutedFfn(int layer, const float* x, int tokens, const int* chosen, const float* weights,
                 int k, float* y) const;
  // Decoder::MoeFfn whole on rows in device memory (decoder.cpp:530-558): the kRouter
  // product of x, Route, the k chosen experts and, with `shared` (the shared expert's
  // output, tokens x hidden; y may be the same rows), shared * SharedExpertScale of the
  // router's last logit as the start of the sum.  Enqueued, not waited for.
  void MoeLayerDevice(int layer, const float* x, int tokens, int k, const float* shared,
                      float* y) const;

private:
  struct Matrix {
    gufo_hip_matrix* handle = nullptr;
    std::size_t rows = 0;
    std::size_t cols = 0;
  };
  struct Layer;
  const std::vector<Matrix>* StageMatrices(Stage stage, int layer) const;
  Matrix Upload(const Tensor& tensor, std::uint64_t experts);
  void Release() noexcept;

  int hidden_ = 0;
  int experts_ = 0;
  int expert_ffn_ = 0;
  std::vector<Matrix> lm_head_;
  std::vector<Layer> layers_;
};

}  // namespace gufo_hip
