// extern "C" layer over GgufModel (include/gufo_hip_model.h): exceptions become status
// codes, the message is kept per thread.
#include <algorithm>
#include <exception>
#include <new>
#include <stdexcept>
#include <string>
#include <vector>

#include "gguf_model.hpp"
#include "gufo_hip.h"
#include "gufo_hip_model.h"

struct gufo_model {
  gufo_hip::GgufModel impl;
  gufo_model(const std::string& path, int device) : impl(path, device) {}
};

namespace {

thread_local std::string g_error;

// Runs `body` and maps what it throws to the status code the exception stands for.
template <typename Body>
int Guarded(Body&& body) {
  try {
    body();
    return GUFO_HIP_OK;
  } catch (const std::invalid_argument& e) {
    g_error = e.what();
    return GUFO_HIP_ERR_INVALID_ARGUMENT;
  } catch (const std::out_of_range& e) {
    g_error = e.what();
    return GUFO_HIP_ERR_OUT_OF_RANGE;
  } catch (const std::logic_error& e) {
    g_error = e.what();
    return GUFO_HIP_ERR_LOGIC;
  } catch (const std::bad_alloc&) {
    g_error = "out of host memory";
    return GUFO_HIP_ERR_OUT_OF_MEMORY;
  } catch (const std::exception& e) {
    g_error = e.what();
    return GUFO_HIP_ERR_RUNTIME;
  }
}

void Fill(const gufo_hip::ModelShape& s, bool has_mtp_layer, std::size_t tensors,
          gufo_model_shape* out) {
  out->is_moe = s.architecture == "qwen35moe" ? 1 : 0;
  out->layers = s.layers;
  out->mtp_layers = s.mtp_layers;
  out->hidden = s.hidden;
  out->ffn = s.ffn;
  out->vocab = s.vocab;
  out->rms_eps = s.rms_eps;
  out->full_attention_interval = s.full_attention_interval;
  out->heads = s.heads;
  out->kv_heads = s.kv_heads;
  out->head_dim = s.head_dim;
  out->rope_dim = s.rope_dim;
  out->rope_theta = s.rope_theta;
  out->conv_kernel = s.conv_kernel;
  out->linear_key_heads = s.linear_key_heads;
  out->linear_value_heads = s.linear_value_heads;
  out->linear_head_dim = s.linear_head_dim;
  out->experts = s.experts;
  out->experts_used = s.experts_used;
  out->expert_ffn = s.expert_ffn;
  out->shared_expert_ffn = s.shared_expert_ffn;
  out->tied_embeddings = s.tied_embeddings ? 1 : 0;
  out->has_mtp_layer = has_mtp_layer ? 1 : 0;
  out->tensors = static_cast<int>(tensors);
}

gufo_hip::Stage StageOf(int stage) {
  if (stage < GUFO_STAGE_LINEAR_IN || stage > GUFO_STAGE_MTP_IN) {
    throw std::invalid_argument("unknown stage " + std::to_string(stage));
  }
  return static_cast<gufo_hip::Stage>(stage);
}

void RequireModel(const gufo_model* model) {
  if (model == nullptr) throw std::invalid_argument("model is null");
}

}  // namespace

extern "C" {

const char* gufo_model_last_error(void) { return g_error.c_str(); }

int gufo_model_inspect(const char* path, gufo_model_shape* shape) {
  return Guarded([&] {
    if (path == nullptr || shape == nullptr) throw std::invalid_argument("path or shape is null");
    const auto file = gufo_hip::GgufFile::Open(path);
    const gufo_hip::ModelShape s = gufo_hip::ReadShape(*file);
    gufo_hip::BuildStageTable(*file, s);  // the shape checks; nothing is uploaded
    Fill(s, gufo_hip::HasMtpLayer(*file, s), file->Tensors().size(), shape);
  });
}

int gufo_model_open(const char* path, int device, gufo_model** out) {
  return Guarded([&] {
    if (path == nullptr || out == nullptr) throw std::invalid_argument("path or out is null");
    *out = nullptr;
    *out = new gufo_model(path, device);
  });
}

int gufo_model_close(gufo_model* model) {
  return Guarded([&] { delete model; });
}

int gufo_model_get_shape(const gufo_model* model, gufo_model_shape* shape) {
  return Guarded([&] {
    RequireModel(model);
    if (shape == nullptr) throw std::invalid_argument("shape is null");
    Fill(model->impl.shape(), model->impl.has_mtp_layer(), model->impl.tensor_count(), shape);
  });
}

uint64_t gufo_model_weight_bytes(const gufo_model* model) {
  return model == nullptr ? 0 : model->impl.weight_bytes();
}

size_t gufo_model_stage_inputs(const gufo_model* model, int stage, int layer) {
  size_t n = 0;
  Guarded([&] {
    RequireModel(model);
    n = model->impl.projections().StageInputs(StageOf(stage), layer);
  });
  return n;
}

size_t gufo_model_stage_outputs(const gufo_model* model, int stage, int layer) {
  size_t n = 0;
  Guarded([&] {
    RequireModel(model);
    n = model->impl.projections().StageOutputs(StageOf(stage), layer);
  });
  return n;
}

int gufo_model_apply(const gufo_model* model, int stage, int layer, const float* x, int tokens,
                     float* y) {
  return Guarded([&] {
    RequireModel(model);
    model->impl.projections().Apply(StageOf(stage), layer, x, tokens, y);
  });
}

int gufo_model_apply_expert(const gufo_model* model, int stage, int layer, int expert,
                            const float* x, int tokens, float* y) {
  return Guarded([&] {
    RequireModel(model);
    model->impl.projections().ApplyExpert(StageOf(stage), layer, expert, x, tokens, y);
  });
}

int gufo_model_stage_matrices(const gufo_model* model, int stage, int layer,
                              const gufo_hip_matrix** out, int capacity, int* count) {
  return Guarded([&] {
    RequireModel(model);
    if (count == nullptr) throw std::invalid_argument("count is null");
    const auto handles = model->impl.projections().StageHandles(StageOf(stage), layer);
    *count = static_cast<int>(handles.size());
    if (out == nullptr) return;
    if (capacity < *count) {
      throw std::invalid_argument("room for " + std::to_string(capacity) + " of " +
                                  std::to_string(*count) + " matrices");
    }
    std::copy(handles.begin(), handles.end(), out);
  });
}

int gufo_model_expert_matrices(const gufo_model* model, int layer, const gufo_hip_matrix** gate,
                               const gufo_hip_matrix** up, const gufo_hip_matrix** down) {
  return Guarded([&] {
    RequireModel(model);
    model->impl.projections().ExpertHandles(layer, gate, up, down);
  });
}

int gufo_model_norm_weight(const gufo_model* model, int which, int layer, float* out) {
  return Guarded([&] {
    RequireModel(model);
    if (out == nullptr) throw std::invalid_argument("out is null");
    const std::vector<float>* w = nullptr;
    switch (which) {
      case 0: w = &model->impl.attn_norm(layer); break;
      case 1: w = &model->impl.post_attention_norm(layer); break;
      case 2: w = &model->impl.output_norm(); break;
      default: throw std::invalid_argument("unknown norm weight " + std::to_string(which));
    }
    std::copy(w->begin(), w->end(), out);
  });
}

}  // extern "C"
