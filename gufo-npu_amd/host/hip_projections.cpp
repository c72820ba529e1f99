#include "hip_projections.hpp"

#include <utility>

#include "gufo_hip.h"

namespace gufo_hip {
namespace {

// The exception the reference throws where the C layer reports `code`
// (include/gufo_hip.h, "Status codes").
[[noreturn]] void Throw(int code) {
  const std::string message = gufo_hip_last_error();
  switch (code) {
    case GUFO_HIP_ERR_INVALID_ARGUMENT:
      throw std::invalid_argument(message);
    case GUFO_HIP_ERR_LOGIC:
      throw std::logic_error(message);
    case GUFO_HIP_ERR_OUT_OF_RANGE:
      throw std::out_of_range(message);
    default:
      throw std::runtime_error(message);
  }
}

void Check(int code) {
  if (code != GUFO_HIP_OK) Throw(code);
}

std::string ShapeText(const std::vector<std::uint64_t>& shape) {
  std::string out;
  for (const auto dim : shape) out += (out.empty() ? "" : ", ") + std::to_string(dim);
  return "[" + out + "]";
}

}  // namespace

struct HipProjections::Layer {
  std::vector<Matrix> linear_in;
  std::vector<Matrix> attention_in;
  std::vector<Matrix> mixer_out;
  std::vector<Matrix> ffn_in;
  std::vector<Matrix> ffn_down;
  std::vector<Matrix> router;
  std::vector<Matrix> mtp_in;
  Matrix gate_exps;
  Matrix up_exps;
  Matrix down_exps;
};

// `tensor` must be [cols, rows], [cols] when it has one row, or, with `experts`,
// [cols, rows, experts] (CheckShape, gguf_projections.cpp:25-46 of the reference).
HipProjections::Matrix HipProjections::Upload(const Tensor& tensor, std::uint64_t experts) {
  const auto& shape = tensor.shape;
  const bool ok = experts != 0 ? shape.size() == 3 && shape[2] == experts
                               : shape.size() == 2 || shape.size() == 1;
  if (!ok || tensor.data == nullptr) {
    throw std::runtime_error("qwen35: tensor " + tensor.name + " has shape " + ShapeText(shape) +
                             (experts != 0 ? ", expected [cols, rows, " + std::to_string(experts) + "]"
                                           : ", expected [cols, rows]"));
  }
  Matrix m;
  m.cols = static_cast<std::size_t>(shape[0]);
  m.rows = shape.size() == 1 ? 1 : static_cast<std::size_t>(shape[1]) *
                                       static_cast<std::size_t>(experts != 0 ? experts : 1);
  Check(gufo_hip_matrix_create(tensor.ggml_type, tensor.data, m.rows, m.cols, &m.handle));
  return m;
}

HipProjections::HipProjections(const ModelTensors& model, int device)
    : hidden_(model.hidden), experts_(model.experts), expert_ffn_(model.expert_ffn) {
  Check(gufo_hip_init(device));
  try {
    auto expect_cols = [](const Tensor& t, const Matrix& m, std::size_t cols) {
      if (m.cols != cols) {
        throw std::runtime_error("qwen35: tensor " + t.name + " has shape " + ShapeText(t.shape) +
                                 ", expected " + std::to_string(cols) + " columns");
      }
    };
    auto upload_stage = [&](const std::vector<Tensor>& tensors, std::vector<Matrix>* out) {
      for (const Tensor& t : tensors) {
        out->push_back(Upload(t, 0));
        // The matrices of a stage share their input (projections.hpp:8-11).
        expect_cols(t, out->back(), out->front().cols);
      }
    };
    if (model.lm_head.data != nullptr) {
      lm_head_.push_back(Upload(model.lm_head, 0));
      expect_cols(model.lm_head, lm_head_.back(), static_cast<std::size_t>(hidden_));
    }
    layers_.reserve(model.layers.size());
    for (const LayerTensors& src : model.layers) {
      layers_.emplace_back();
      Layer& layer = layers_.back();
      upload_stage(src.linear_in, &layer.linear_in);
      upload_stage(src.attention_in, &layer.attention_in);
      upload_stage(src.mixer_out, &layer.mixer_out);
      upload_stage(src.ffn_in, &layer.ffn_in);
      upload_stage(src.ffn_down, &layer.ffn_down);
      upload_stage(src.router, &layer.router);
      upload_stage(src.mtp_in, &layer.mtp_in);
      if (src.gate_exps.data != nullptr) {
        const auto e = static_cast<std::uint64_t>(experts_);
        const auto hidden = static_cast<std::size_t>(hidden_);
        const auto ffn = static_cast<std::size_t>(expert_ffn_);
        if (e == 0) throw std::runtime_error("qwen35: expert tensors in a model without experts");
        layer.gate_exps = Upload(src.gate_exps, e);
        layer.up_exps = Upload(src.up_exps, e);
        layer.down_exps = Upload(src.down_exps, e);
        // [hidden, expert_ffn, experts] twice and [expert_ffn, hidden, experts]
        // (gguf_projections.cpp:135-137).
        const struct {
          const Tensor* t;
          const Matrix* m;
          std::size_t cols, rows;
        } want[] = {{&src.gate_exps, &layer.gate_exps, hidden, ffn},
                    {&src.up_exps, &layer.up_exps, hidden, ffn},
                    {&src.down_exps, &layer.down_exps, ffn, hidden}};
        for (const auto& w : want) {
          if (w.m->cols != w.cols || w.m->rows != w.rows * e) {
            throw std::runtime_error(
                "qwen35: tensor " + w.t->name + " has shape " + ShapeText(w.t->shape) +
                ", expected " +
                ShapeText({w.cols, w.rows, static_cast<std::uint64_t>(experts_)}));
          }
        }
      }
    }
  } catch (...) {
    Release();
    throw;
  }
}

void HipProjections::Release() noexcept {
  auto drop = [](std::vector<Matrix>& v) {
    for (Matrix& m : v) {
      if (m.handle != nullptr) gufo_hip_matrix_destroy(m.handle);
    }
    v.clear();
  };
  drop(lm_head_);
  for (Layer& l : layers_) {
    drop(l.linear_in);
    drop(l.attention_in);
    drop(l.mixer_out);
    drop(l.ffn_in);
    drop(l.ffn_down);
    drop(l.router);
    drop(l.mtp_in);
    for (Matrix* m : {&l.gate_exps, &l.up_exps, &l.down_exps}) {
      if (m->handle != nullptr) gufo_hip_matrix_destroy(m->handle);
      m->handle = nullptr;
    }
  }
  layers_.clear();
}

HipProjections::~HipProjections() { Release(); }

const std::vector<HipProjections::Matrix>* HipProjections::StageMatrices(Stage stage,
                                                                         int layer) const {
  if (stage == Stage::kLmHead) return &lm_head_;
  const Layer& l = layers_.at(static_cast<std::size_t>(layer));  // std::out_of_range
  switch (stage) {
    case Stage::kLinearIn: return &l.linear_in;
    case Stage::kAttentionIn: return &l.attention_in;
    case Stage::kMixerOut: return &l.mixer_out;
    case Stage::kFfnIn: return &l.ffn_in;
    case Stage::kFfnDown: return &l.ffn_down;
    case Stage::kRouter: return &l.router;
    case Stage::kMtpIn: return &l.mtp_in;
    default: return nullptr;  // the expert stages go through ApplyExpert
  }
}

void HipProjections::Apply(Stage stage, int layer, const float* x, int tokens, float* y) const {
  const std::vector<Matrix>* parts = StageMatrices(stage, layer);
  if (parts == nullptr || parts->empty()) {
    throw std::logic_error("qwen35: no weights for this stage and layer");
  }
  std::vector<const gufo_hip_matrix*> handles;
  std::vector<std::size_t> first;
  std::vector<std::size_t> rows;
  for (const Matrix& m : *parts) {
    handles.push_back(m.handle);
    first.push_back(0);
    rows.push_back(m.rows);
  }
  Check(gufo_hip_gemv(handles.data(), first.data(), rows.data(), static_cast<int>(handles.size()),
                      x, tokens, y));
}

namespace {

gufo_hip_prologue ToC(const HipProjections::DeviceInput& in) {
  gufo_hip_prologue prologue = {};
  switch (in.prologue) {
    case HipProjections::Prologue::kPlain: prologue.kind = GUFO_HIP_PROLOGUE_PLAIN; break;
    case HipProjections::Prologue::kSwiGlu: prologue.kind = GUFO_HIP_PROLOGUE_SWIGLU; break;
    case HipProjections::Prologue::kResNorm:
      prologue.kind = GUFO_HIP_PROLOGUE_RESNORM;
      prologue.delta_dev = in.delta;
      prologue.norm_weight_dev = in.norm_weight;
      prologue.eps = in.eps;
      prologue.residual_out_dev = in.residual;
      prologue.normed_out_dev = in.normed;
      break;
  }
  return prologue;
}

// The handles of a stage's matrices with their whole row ranges.
struct WholeParts {
  std::vector<const gufo_hip_matrix*> handles;
  std::vector<std::size_t> first;
  std::vector<std::size_t> rows;
  int count() const { return static_cast<int>(handles.size()); }
};

}  // namespace

void HipProjections::ApplyDevice(Stage stage, int layer, const DeviceInput& in, int tokens,
                                 float* y) const {
  const std::vector<Matrix>* parts = StageMatrices(stage, layer);
  if (parts == nullptr || parts->empty()) {
    throw std::logic_error("qwen35: no weights for this stage and layer");
  }
  WholeParts whole;
  for (const Matrix& m : *parts) {
    whole.handles.push_back(m.handle);
    whole.first.push_back(0);
    whole.rows.push_back(m.rows);
  }
  const gufo_hip_prologue prologue = ToC(in);
  Check(gufo_hip_gemv_fused_dev(whole.handles.data(), whole.first.data(), whole.rows.data(),
                                whole.count(), &prologue, in.x, tokens, y));
}

std::vector<const gufo_hip_matrix*> HipProjections::StageHandles(Stage stage, int layer) const {
  const std::vector<Matrix>* parts = StageMatrices(stage, layer);
  std::vector<const gufo_hip_matrix*> handles;
  if (parts != nullptr) {
    for (const Matrix& m : *parts) handles.push_back(m.handle);
  }
  return handles;
}

void HipProjections::ExpertHandles(int layer, const gufo_hip_matrix** gate,
                                   const gufo_hip_matrix** up,
                                   const gufo_hip_matrix** down) const {
  const Layer& l = layers_.at(static_cast<std::size_t>(layer));
  if (gate != nullptr) *gate = l.gate_exps.handle;
  if (up != nullptr) *up = l.up_exps.handle;
  if (down != nullptr) *down = l.down_exps.handle;
}

void HipProjections::PrefillDevice(Stage stage, int layer, const std::uint16_t* a_bf16,
                                   std::size_t tokens, float* c) const {
  const std::vector<Matrix>* parts = StageMatrices(stage, layer);
  if (parts == nullptr || parts->empty()) {
    throw std::logic_error("qwen35: no weights for this stage and layer");
  }
  std::vector<const gufo_hip_matrix*> handles;
  for (const Matrix& m : *parts) handles.push_back(m.handle);
  Check(gufo_hip_gemm_bf16_parts_dev(handles.data(), static_cast<int>(handles.size()), a_bf16,
                                     tokens, c));
}

void HipProjections::PreparePrefill(Stage stage, int layer) {
  const std::vector<Matrix>* parts = StageMatrices(stage, layer);
  if (parts == nullptr || parts->empty()) {
    throw std::logic_error("qwen35: no weights for this stage and layer");
  }
  for (const Matrix& m : *parts) Check(gufo_hip_matrix_prepare_prefill(m.handle));
}

void HipProjections::PickDevice(Stage stage, int layer, const DeviceInput& in, int tokens,
                                std::int64_t* index) const {
  const std::vector<Matrix>* parts = StageMatrices(stage, layer);
  if (parts == nullptr || parts->empty()) {
    throw std::logic_error("qwen35: no weights for this stage and layer");
  }
  WholeParts whole;
  for (const Matrix& m : *parts) {
    whole.handles.push_back(m.handle);
    whole.first.push_back(0);
    whole.rows.push_back(m.rows);
  }
  const gufo_hip_prologue prologue = ToC(in);
  Check(gufo_hip_gemv_argmax_dev(whole.handles.data(), whole.first.data(), whole.rows.data(),
                                 whole.count(), &prologue, in.x, tokens, index));
}

void HipProjections::ApplyExpert(Stage stage, int layer, int expert, const float* x, int tokens,
                                 float* y) const {
  const Layer& l = layers_.at(static_cast<std::size_t>(layer));
  if (l.gate_exps.handle == nullptr || expert < 0 || expert >= experts_) {
    throw std::logic_error("qwen35: no such expert");
  }
  const auto e = static_cast<std::size_t>(expert);
  const auto ffn = static_cast<std::size_t>(expert_ffn_);
  const auto hidden = static_cast<std::size_t>(hidden_);
  switch (stage) {
    case Stage::kExpertIn: {
      // Rows [e*ffn, (e+1)*ffn) of gate and of up (gguf_projections.cpp:230-231).
      const gufo_hip_matrix* parts[2] = {l.gate_exps.handle, l.up_exps.handle};
      const std::size_t first[2] = {e * ffn, e * ffn};
      const std::size_t rows[2] = {ffn, ffn};
      Check(gufo_hip_gemv(parts, first, rows, 2, x, tokens, y));
      return;
    }
    case Stage::kExpertDown: {
      const gufo_hip_matrix* parts[1] = {l.down_exps.handle};
      const std::size_t first[1] = {e * hidden};
      const std::size_t rows[1] = {hidden};
      Check(gufo_hip_gemv(parts, first, rows, 1, x, tokens, y));
      return;
    }
    default:
      throw std::logic_error("qwen35: ApplyExpert takes expert stages only");
  }
}

std::size_t HipProjections::StageInputs(Stage stage, int layer) const {
  if (stage == Stage::kExpertIn) return static_cast<std::size_t>(hidden_);
  if (stage == Stage::kExpertDown) return static_cast<std::size_t>(expert_ffn_);
  const std::vector<Matrix>* parts = StageMatrices(stage, layer);
  return parts == nullptr || parts->empty() ? 0 : parts->front().cols;
}

std::size_t HipProjections::StageOutputs(Stage stage, int layer) const {
  if (stage == Stage::kExpertIn) return 2 * static_cast<std::size_t>(expert_ffn_);
  if (stage == Stage::kExpertDown) return static_cast<std::size_t>(hidden_);
  const std::vector<Matrix>* parts = StageMatrices(stage, layer);
  std::size_t total = 0;
  if (parts != nullptr) {
    for (const Matrix& m : *parts) total += m.rows;
  }
  return total;
}

void HipProjections::Route(const float* logits, int tokens, int k, int* chosen,
                           float* weights) const {
  Check(gufo_hip_route_topk(logits, tokens, experts_, k, chosen, weights));
}

void HipProjections::RoutedFfn(int layer, const float* x, int tokens, const int* chosen,
                               const float* weights, int k, float* y) const {
  const Layer& l = layers_.at(static_cast<std::size_t>(layer));
  if (l.gate_exps.handle == nullptr) {
    throw std::logic_error("qwen35: these projections have no MoE experts");
  }
  Check(gufo_hip_moe_ffn(l.gate_exps.handle, l.up_exps.handle, l.down_exps.handle, experts_, x,
                         tokens, chosen, weights, k, y));
}

void HipProjections::MoeLayerDevice(int layer, const float* x, int tokens, int k,
                                    const float* shared, float* y) const {
  const Layer& l = layers_.at(static_cast<std::size_t>(layer));
  if (l.gate_exps.handle == nullptr || l.router.empty()) {
    throw std::logic_error("qwen35: these projections have no MoE experts");
  }
  std::vector<const gufo_hip_matrix*> router;
  for (const Matrix& m : l.router) router.push_back(m.handle);
  Check(gufo_hip_moe_layer_dev(router.data(), static_cast<int>(router.size()),
                               l.gate_exps.handle, l.up_exps.handle, l.down_exps.handle,
                               experts_, k, x, tokens, shared, y));
}

}  // namespace gufo_hip
