// TEST INFRASTRUCTURE, NOT PRODUCT CODE.
//
// C entry points over the reference's own implementation of the quantized
// matrix-vector path, compiled from the reference's sources where they lie
// (see Makefile: -I$(REFERENCE)/src plus its core/quant.cpp and
// models/qwen35/moe.cpp).  Nothing of the reference is copied here: this file
// only calls it.  The result, oracle/_ref/libgufo_ref.so, validates the C
// restatement in kquant_oracle.c and is the "reference" CPU baseline the bench
// times beside the GPU.
//
// What is the reference's and what is this driver's:
//   * ref_half_to_float, ref_dequantize, ref_dot, ref_route, ref_silu and
//     ref_shared_expert_scale call quant::HalfToFloat, quant::Dequantize,
//     gguf_dot::DotQ4_K/DotQ5_K/DotQ6_K (the AVX2+FMA+F16C bodies, built with
//     -march=x86-64-v3 as the reference builds them), qwen35::Route, simd::Silu
//     and qwen35::SharedExpertScale.
//   * ref_matmul runs those dots over row ranges on the reference's SpinPool
//     (core/thread_pool.hpp) in jobs of 16 rows and writes
//     y[t*stride + offset + r], the loop of GgufProjections::MatMul
//     (models/qwen35/gguf_projections.cpp:239-286); the loop itself is restated
//     here because MatMul is a private member that needs a whole model file.
//   * ref_gguf_* open a GGUF file with the reference's reader (core/gguf.cpp), read its
//     Config (models/qwen35/config.cpp) and run the reference's GgufProjections itself
//     (models/qwen35/gguf_projections.cpp: stage table, shape checks, MatMul) - with a
//     model file, synthetic or real, nothing of that class needs restating.
//   * ref_decoder_* run the reference's Decoder (models/qwen35/decoder.cpp: embedding,
//     norms, mixers, residuals, the MoE loop) over a Projections of the caller's choice:
//     the reference's GgufProjections in either precision, or ForeignProjections, a
//     Projections whose two methods forward to a pair of C function pointers.  Handed
//     gufo_model_apply / gufo_model_apply_expert, that is the reference's own decoder
//     running on the MI355X backend: the binding a maintainer of the reference adds.
#include <algorithm>
#include <cstddef>
#include <cstdint>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "core/cpus.hpp"
#include "core/quant.hpp"
#include "core/simd.hpp"
#include "core/gguf.hpp"
#include "core/thread_pool.hpp"
#include "core/vec.hpp"
#include "models/qwen35/config.hpp"
#include "models/qwen35/decoder.hpp"
#include "models/qwen35/gguf_projections.hpp"
#include "models/qwen35/gguf_dot.hpp"
#include "models/qwen35/moe.hpp"

namespace {

using gufo_npu::gguf::GgmlType;
namespace dot = gufo_npu::qwen35::gguf_dot;

using RowDot = float (*)(const std::uint8_t*, const float*, std::size_t);

RowDot DotFor(int type) {
  switch (static_cast<GgmlType>(type)) {
    case GgmlType::kQ4_K: return &dot::DotQ4_K;
    case GgmlType::kQ5_K: return &dot::DotQ5_K;
    case GgmlType::kQ6_K: return &dot::DotQ6_K;
    case GgmlType::kQ8_0: return &dot::DotQ8_0;
    case GgmlType::kF32: return &dot::DotF32;
    default: return nullptr;
  }
}

struct Pool {
  explicit Pool(std::size_t workers) : pool(workers) {}
  gufo_npu::SpinPool pool;
  std::mutex run;
};

std::mutex g_pools_mutex;
std::vector<std::unique_ptr<Pool>> g_pools;  // index = threads

// A pool of `threads` threads in all (the caller included), kept for reuse.
Pool& PoolFor(std::size_t threads) {
  const std::lock_guard<std::mutex> lock(g_pools_mutex);
  if (g_pools.size() <= threads) g_pools.resize(threads + 1);
  if (!g_pools[threads]) g_pools[threads] = std::make_unique<Pool>(threads - 1);
  return *g_pools[threads];
}

}  // namespace

extern "C" {

float ref_half_to_float(std::uint16_t h) { return gufo_npu::quant::HalfToFloat(h); }

int ref_dequantize(int type, const std::uint8_t* src, float* dst, std::size_t n) {
  try {
    gufo_npu::quant::Dequantize(static_cast<GgmlType>(type), src, dst, n);
    return 0;
  } catch (...) {
    return -1;
  }
}

float ref_dot(int type, const std::uint8_t* row, const float* x, std::size_t n) {
  const RowDot fn = DotFor(type);
  return fn != nullptr ? fn(row, x, n) : 0.0f;
}

void ref_route(const float* logits, int experts, int k, int* chosen,
               float* weights) {
  gufo_npu::qwen35::Route(logits, experts, k, chosen, weights);
}

// core/simd.hpp:82-84: x / (1 + e^-x) in fp32.
float ref_silu(float x) { return gufo_npu::simd::Silu(x); }

// core/vec.hpp:56-63, in the AVX2 order of vec::Dot this build selects.
void ref_rms_norm(const float* x, const float* w, int n, float eps, float* out) {
  gufo_npu::vec::RmsNorm(x, w, n, eps, out);
}

float ref_shared_expert_scale(float logit) {
  return gufo_npu::qwen35::SharedExpertScale(logit);
}

// The reference's thread policy for these products: the caller plus
// HalfCpuWorkers() (core/cpus.hpp:53-55, gguf_projections.cpp:93-98).
int ref_default_threads() {
  return static_cast<int>(gufo_npu::HalfCpuWorkers() + 1);
}

int ref_usable_cpus() { return static_cast<int>(gufo_npu::UsableCpus()); }

// threads <= 0 selects ref_default_threads().
int ref_matmul(int n_parts, const std::uint8_t* const* data, const int* types,
               const std::size_t* first, const std::size_t* rows, std::size_t in,
               const float* x, int tokens, float* y, int threads) {
  constexpr std::size_t kChunk = 16;
  if (n_parts <= 0 || tokens < 0) return -1;
  std::vector<std::size_t> first_job = {0};
  std::size_t stride = 0;
  for (int p = 0; p < n_parts; ++p) {
    if (DotFor(types[p]) == nullptr) return -1;
    stride += rows[p];
    first_job.push_back(first_job.back() + (rows[p] + kChunk - 1) / kChunk);
  }
  std::size_t row_bytes_of[64];
  if (n_parts > 64) return -1;
  try {
    for (int p = 0; p < n_parts; ++p) {
      row_bytes_of[p] =
          gufo_npu::quant::RowBytes(static_cast<GgmlType>(types[p]), in);
    }
  } catch (...) {
    return -1;
  }
  Pool& pool = PoolFor(threads > 0 ? static_cast<std::size_t>(threads)
                                   : static_cast<std::size_t>(ref_default_threads()));
  const std::lock_guard<std::mutex> lock(pool.run);
  pool.pool.Run(first_job.back(), [&](std::size_t job) {
    std::size_t p = 0;
    std::size_t offset = 0;
    while (job >= first_job[p + 1]) {
      offset += rows[p];
      ++p;
    }
    const RowDot fused = DotFor(types[p]);
    const std::size_t begin = (job - first_job[p]) * kChunk;
    const std::size_t end = std::min(rows[p], begin + kChunk);
    for (std::size_t r = begin; r < end; ++r) {
      const std::uint8_t* row = data[p] + (first[p] + r) * row_bytes_of[p];
      for (int t = 0; t < tokens; ++t) {
        y[static_cast<std::size_t>(t) * stride + offset + r] =
            fused(row, x + static_cast<std::size_t>(t) * in, in);
      }
    }
  });
  return 0;
}

// ---- a whole model file through the reference's own classes ---------------------------

namespace {

struct RefModel {
  std::unique_ptr<gufo_npu::gguf::File> file;
  gufo_npu::qwen35::Config config;
  std::unique_ptr<gufo_npu::qwen35::GgufProjections> fused;  // Precision::kFloat
  std::unique_ptr<gufo_npu::qwen35::GgufProjections> exact;  // Precision::kDouble
};

thread_local std::string g_ref_error;

}  // namespace

const char* ref_last_error() { return g_ref_error.c_str(); }

// nullptr (and ref_last_error) when the reference rejects the file.
void* ref_gguf_open(const char* path) {
  try {
    auto model = std::make_unique<RefModel>();
    model->file = gufo_npu::gguf::File::Open(path);
    model->config = gufo_npu::qwen35::ReadConfig(*model->file);
    using gufo_npu::qwen35::GgufProjections;
    model->fused = std::make_unique<GgufProjections>(*model->file,
                                                     GgufProjections::Precision::kFloat);
    model->exact = std::make_unique<GgufProjections>(*model->file,
                                                     GgufProjections::Precision::kDouble);
    return model.release();
  } catch (const std::exception& e) {
    g_ref_error = e.what();
    return nullptr;
  }
}

void ref_gguf_close(void* handle) { delete static_cast<RefModel*>(handle); }

// The Config fields, in the order of models/qwen35/config.hpp:13-52:
// layers, mtp_layers, hidden, ffn, vocab, full_attention_interval, heads, kv_heads,
// head_dim, rope_dim, conv_kernel, linear_key_heads, linear_value_heads,
// linear_head_dim, experts, experts_used, expert_ffn, shared_expert_ffn,
// tied_embeddings, has_mtp_layer (HasMtpLayer).
void ref_gguf_config(void* handle, int* out, float* rms_eps) {
  const RefModel& m = *static_cast<RefModel*>(handle);
  const auto& c = m.config;
  const int fields[20] = {c.layers, c.mtp_layers, c.hidden, c.ffn, c.vocab,
                          c.full_attention_interval, c.heads, c.kv_heads, c.head_dim,
                          c.rope_dim, c.conv_kernel, c.linear_key_heads,
                          c.linear_value_heads, c.linear_head_dim, c.experts,
                          c.experts_used, c.expert_ffn, c.shared_expert_ffn,
                          c.tied_embeddings ? 1 : 0,
                          gufo_npu::qwen35::HasMtpLayer(*m.file, c) ? 1 : 0};
  std::copy(fields, fields + 20, out);
  *rms_eps = c.rms_eps;
}

// Stage numbers follow qwen35::Stage (models/qwen35/projections.hpp:14-39).  expert < 0:
// Apply; otherwise ApplyExpert.  Returns 0, or -1 with ref_last_error set when the
// reference throws.
int ref_gguf_apply(void* handle, int stage, int layer, int expert, const float* x, int tokens,
                   float* y, int exact) {
  const RefModel& m = *static_cast<RefModel*>(handle);
  const auto& proj = exact != 0 ? *m.exact : *m.fused;
  const auto s = static_cast<gufo_npu::qwen35::Stage>(stage);
  try {
    if (expert < 0) {
      proj.Apply(s, layer, x, tokens, y);
    } else {
      proj.ApplyExpert(s, layer, expert, x, tokens, y);
    }
    return 0;
  } catch (const std::exception& e) {
    g_ref_error = e.what();
    return -1;
  }
}

// ---- the reference's decoder over any Projections --------------------------------------

namespace {

// qwen35::Projections over C entry points with the signatures of gufo_model_apply and
// gufo_model_apply_expert (include/gufo_hip_model.h); a non-zero status becomes the
// exception a consumer of Projections expects.
class ForeignProjections : public gufo_npu::qwen35::Projections {
public:
  using ApplyFn = int (*)(const void*, int, int, const float*, int, float*);
  using ApplyExpertFn = int (*)(const void*, int, int, int, const float*, int, float*);
  ForeignProjections(const void* model, ApplyFn apply, ApplyExpertFn apply_expert)
      : model_(model), apply_(apply), apply_expert_(apply_expert) {}
  void Apply(gufo_npu::qwen35::Stage stage, int layer, const float* x, int tokens,
             float* y) const override {
    ++calls;
    if (apply_(model_, static_cast<int>(stage), layer, x, tokens, y) != 0) {
      throw std::runtime_error("foreign Projections::Apply failed");
    }
  }
  void ApplyExpert(gufo_npu::qwen35::Stage stage, int layer, int expert, const float* x,
                   int tokens, float* y) const override {
    ++calls;
    if (apply_expert_(model_, static_cast<int>(stage), layer, expert, x, tokens, y) != 0) {
      throw std::runtime_error("foreign Projections::ApplyExpert failed");
    }
  }
  mutable long calls = 0;

private:
  const void* model_;
  ApplyFn apply_;
  ApplyExpertFn apply_expert_;
};

struct RefDecoder {
  std::unique_ptr<ForeignProjections> foreign;
  std::unique_ptr<gufo_npu::qwen35::Decoder> decoder;
  gufo_npu::qwen35::Decoder::State state;
};

}  // namespace

// which: 0 = GgufProjections fp32, 1 = GgufProjections double, 2 = the foreign entry
// points.  `model` is a ref_gguf_open handle and must outlive the decoder.
void* ref_decoder_open(void* model, int which, const void* foreign_model, void* apply,
                       void* apply_expert) {
  try {
    RefModel& m = *static_cast<RefModel*>(model);
    auto d = std::make_unique<RefDecoder>();
    const gufo_npu::qwen35::Projections* projections = nullptr;
    if (which == 2) {
      d->foreign = std::make_unique<ForeignProjections>(
          foreign_model, reinterpret_cast<ForeignProjections::ApplyFn>(apply),
          reinterpret_cast<ForeignProjections::ApplyExpertFn>(apply_expert));
      projections = d->foreign.get();
    } else {
      projections = which == 1 ? m.exact.get() : m.fused.get();
    }
    d->decoder = std::make_unique<gufo_npu::qwen35::Decoder>(*m.file, *projections);
    d->state = d->decoder->NewState();
    return d.release();
  } catch (const std::exception& e) {
    g_ref_error = e.what();
    return nullptr;
  }
}

void ref_decoder_close(void* handle) { delete static_cast<RefDecoder*>(handle); }

// Decoder::Step at the decoder's own position; copies the vocab logits out.
int ref_decoder_step(void* handle, int token, float* logits) {
  RefDecoder& d = *static_cast<RefDecoder*>(handle);
  try {
    const std::vector<float>& out = d.decoder->Step(token, d.state);
    std::copy(out.begin(), out.end(), logits);
    return 0;
  } catch (const std::exception& e) {
    g_ref_error = e.what();
    return -1;
  }
}

void ref_decoder_reset(void* handle) {
  RefDecoder& d = *static_cast<RefDecoder*>(handle);
  d.state = d.decoder->NewState();
}

long ref_decoder_foreign_calls(void* handle) {
  const RefDecoder& d = *static_cast<RefDecoder*>(handle);
  return d.foreign ? d.foreign->calls : 0;
}

}  // extern "C"
