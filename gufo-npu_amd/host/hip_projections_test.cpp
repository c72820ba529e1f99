// HipProjections against the CPU checker, in the style of the reference's own tests
// (plain main(), one line per case, exit 1 on failure): every stage of a dense and of
// an MoE layer through Apply / ApplyExpert, the layout of concatenated outputs, the
// routed-expert call, a decorator over the interface, and the exceptions.
//
//   hip_projections_test                  needs an MI355X
//   hip_projections_test --no-device      on a machine without one: the constructor
//                                         must throw std::runtime_error
//
// The checker is oracle/kquant_oracle.c (dequantize + double sum), linked in; the
// bar is rel-L2 <= 1e-4 as for the kernels.
#include <immintrin.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <new>
#include <random>
#include <stdexcept>
#include <string>
#include <vector>

#include "gufo_hip.h"
#include "hip_projections.hpp"
#include "kquant_oracle.h"

namespace {

using gufo_hip::HipProjections;
using gufo_hip::LayerTensors;
using gufo_hip::ModelTensors;
using gufo_hip::Stage;
using gufo_hip::Tensor;

constexpr double kTolerance = 1e-4;
int g_failures = 0;

void Report(const std::string& name, bool ok, double value = -1) {
  if (value >= 0) {
    std::printf("%s: %.2e %s\n", name.c_str(), value, ok ? "ok" : "FAIL");
  } else {
    std::printf("%s %s\n", name.c_str(), ok ? "ok" : "FAIL");
  }
  std::fflush(stdout);
  g_failures += ok ? 0 : 1;
}

// Random blocks with finite fp16 scales (|N(0, 0.02)|), as the bench generates them.
struct Weights {
  int type;
  std::size_t rows, cols;
  std::vector<std::uint8_t> bytes;
};

std::uint16_t ToHalf(float f) {
  return static_cast<std::uint16_t>(_cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT));
}

Weights RandomWeights(int type, std::size_t rows, std::size_t cols, std::mt19937& rng) {
  Weights w{type, rows, cols, {}};
  const std::size_t block = gufo_oracle_block_bytes(type);
  w.bytes.resize(rows * cols / 256 * block);
  for (auto& b : w.bytes) b = static_cast<std::uint8_t>(rng());
  std::normal_distribution<float> normal(0.0f, 0.02f);
  for (std::size_t at = 0; at < w.bytes.size(); at += block) {
    if (type == GUFO_ORACLE_Q6_K) {
      const std::uint16_t d = ToHalf(std::fabs(normal(rng)));
      std::memcpy(&w.bytes[at + 208], &d, 2);
    } else {
      const std::uint16_t d = ToHalf(std::fabs(normal(rng)));
      const std::uint16_t dmin = ToHalf(std::fabs(normal(rng)));
      std::memcpy(&w.bytes[at], &d, 2);
      std::memcpy(&w.bytes[at + 2], &dmin, 2);
    }
  }
  return w;
}

Tensor AsTensor(const std::string& name, const Weights& w, std::uint64_t experts = 0) {
  Tensor t;
  t.name = name;
  t.ggml_type = w.type;
  t.data = w.bytes.data();
  if (experts != 0) {
    t.shape = {w.cols, w.rows / experts, experts};
  } else {
    t.shape = {w.cols, w.rows};
  }
  return t;
}

std::vector<float> RandomActivations(std::size_t n, std::mt19937& rng, float scale = 1.0f) {
  std::normal_distribution<float> normal(0.0f, 1.0f);
  std::vector<float> x(n);
  for (auto& v : x) v = scale * normal(rng);
  return x;
}

double RelL2(const std::vector<float>& got, const std::vector<float>& want) {
  double num = 0, den = 0;
  for (std::size_t i = 0; i < want.size(); ++i) {
    const double d = static_cast<double>(got[i]) - want[i];
    num += d * d;
    den += static_cast<double>(want[i]) * want[i];
  }
  return std::sqrt(num / (den > 0 ? den : 1));
}

// y = [W_0 x | W_1 x | ...] by the checker, double accumulation.
std::vector<float> Expected(const std::vector<const Weights*>& parts,
                            const std::vector<std::size_t>& first,
                            const std::vector<std::size_t>& rows, const std::vector<float>& x,
                            int tokens) {
  std::vector<const std::uint8_t*> data;
  std::vector<int> types;
  std::size_t stride = 0;
  for (std::size_t p = 0; p < parts.size(); ++p) {
    data.push_back(parts[p]->bytes.data());
    types.push_back(parts[p]->type);
    stride += rows[p];
  }
  std::vector<float> y(static_cast<std::size_t>(tokens) * stride);
  gufo_oracle_matmul(static_cast<int>(parts.size()), data.data(), types.data(), first.data(),
                     rows.data(), parts[0]->cols, x.data(), tokens, y.data(), 1, 4);
  return y;
}

std::vector<float> ExpectedWhole(const std::vector<const Weights*>& parts,
                                 const std::vector<float>& x, int tokens) {
  std::vector<std::size_t> first(parts.size(), 0), rows;
  for (const Weights* w : parts) rows.push_back(w->rows);
  return Expected(parts, first, rows, x, tokens);
}

template <typename Exception, typename Fn>
bool Throws(Fn&& fn) {
  try {
    fn();
  } catch (const Exception&) {
    return true;
  } catch (...) {
    return false;
  }
  return false;
}

// A decorator over the interface, as the reference's tests wrap their projections
// (RoutingLog, FollowRouting): counts the calls and forwards them.
class Counting : public gufo_hip::Projections {
public:
  explicit Counting(const gufo_hip::Projections& inner) : inner_(inner) {}
  void Apply(Stage stage, int layer, const float* x, int tokens, float* y) const override {
    ++calls;
    inner_.Apply(stage, layer, x, tokens, y);
  }
  void ApplyExpert(Stage stage, int layer, int expert, const float* x, int tokens,
                   float* y) const override {
    ++calls;
    inner_.ApplyExpert(stage, layer, expert, x, tokens, y);
  }
  mutable int calls = 0;

private:
  const gufo_hip::Projections& inner_;
};

int RunNoDevice() {
  std::mt19937 rng(1);
  const Weights head = RandomWeights(GUFO_ORACLE_Q4_K, 64, 256, rng);
  ModelTensors model;
  model.hidden = 256;
  model.lm_head = AsTensor("token_embd.weight", head);
  Report("constructor without a device throws std::runtime_error",
         Throws<std::runtime_error>([&] { HipProjections p(model); }));
  return g_failures == 0 ? 0 : 1;
}

void RunDense(std::mt19937& rng) {
  const std::size_t hidden = 512, ffn = 768, vocab = 1000, attn = 256, kv = 128;
  const Weights q = RandomWeights(GUFO_ORACLE_Q5_K, 2 * attn, hidden, rng);
  const Weights k = RandomWeights(GUFO_ORACLE_Q5_K, kv, hidden, rng);
  const Weights v = RandomWeights(GUFO_ORACLE_Q6_K, kv, hidden, rng);
  const Weights o = RandomWeights(GUFO_ORACLE_Q4_K, hidden, attn, rng);
  const Weights gate = RandomWeights(GUFO_ORACLE_Q4_K, ffn, hidden, rng);
  const Weights up = RandomWeights(GUFO_ORACLE_Q4_K, ffn, hidden, rng);
  const Weights down = RandomWeights(GUFO_ORACLE_Q6_K, hidden, ffn, rng);
  const Weights head = RandomWeights(GUFO_ORACLE_Q6_K, vocab, hidden, rng);

  ModelTensors model;
  model.hidden = static_cast<int>(hidden);
  model.lm_head = AsTensor("token_embd.weight", head);
  LayerTensors layer;
  layer.attention_in = {AsTensor("blk.0.attn_q.weight", q), AsTensor("blk.0.attn_k.weight", k),
                        AsTensor("blk.0.attn_v.weight", v)};
  layer.mixer_out = {AsTensor("blk.0.attn_output.weight", o)};
  layer.ffn_in = {AsTensor("blk.0.ffn_gate.weight", gate), AsTensor("blk.0.ffn_up.weight", up)};
  layer.ffn_down = {AsTensor("blk.0.ffn_down.weight", down)};
  model.layers.push_back(layer);
  const HipProjections proj(model);
  const Counting counted(proj);

  struct Case {
    const char* name;
    Stage stage;
    int layer;
    std::vector<const Weights*> parts;
  };
  const Case cases[] = {
      {"kAttentionIn [q|k|v] Q5_K,Q5_K,Q6_K", Stage::kAttentionIn, 0, {&q, &k, &v}},
      {"kMixerOut Q4_K", Stage::kMixerOut, 0, {&o}},
      {"kFfnIn [gate|up] Q4_K", Stage::kFfnIn, 0, {&gate, &up}},
      {"kFfnDown Q6_K", Stage::kFfnDown, 0, {&down}},
      {"kLmHead Q6_K", Stage::kLmHead, -1, {&head}},
  };
  for (const Case& c : cases) {
    for (const int tokens : {1, 3, 5}) {
      const std::size_t in = c.parts[0]->cols;
      const auto x = RandomActivations(static_cast<std::size_t>(tokens) * in, rng);
      const auto want = ExpectedWhole(c.parts, x, tokens);
      std::vector<float> got(want.size(), -7.0f);
      counted.Apply(c.stage, c.layer, x.data(), tokens, got.data());
      const double err = RelL2(got, want);
      Report(std::string(c.name) + " tokens=" + std::to_string(tokens), err <= kTolerance, err);
      if (proj.StageInputs(c.stage, c.layer) != in ||
          proj.StageOutputs(c.stage, c.layer) * tokens != want.size()) {
        Report(std::string(c.name) + " stage widths", false);
      }
    }
  }
  Report("decorator forwarded every call", counted.calls == 15);

  // tokens = 0 writes nothing; a stage this layer does not have throws.
  float untouched = 3.0f;
  proj.Apply(Stage::kFfnIn, 0, nullptr, 0, &untouched);
  Report("tokens = 0 is a no-op", untouched == 3.0f);
  const auto x = RandomActivations(hidden, rng);
  std::vector<float> y(4096);
  Report("missing stage throws std::logic_error", Throws<std::logic_error>([&] {
           proj.Apply(Stage::kRouter, 0, x.data(), 1, y.data());
         }));
  Report("expert stage through Apply throws std::logic_error", Throws<std::logic_error>([&] {
           proj.Apply(Stage::kExpertIn, 0, x.data(), 1, y.data());
         }));
  Report("ApplyExpert on a dense model throws std::logic_error", Throws<std::logic_error>([&] {
           proj.ApplyExpert(Stage::kExpertIn, 0, 0, x.data(), 1, y.data());
         }));
  Report("layer out of range throws std::out_of_range", Throws<std::out_of_range>([&] {
           proj.Apply(Stage::kFfnIn, 3, x.data(), 1, y.data());
         }));
  Report("negative token count throws std::invalid_argument", Throws<std::invalid_argument>([&] {
           proj.Apply(Stage::kFfnIn, 0, x.data(), -1, y.data());
         }));

  // Construction checks.
  ModelTensors bad = model;
  bad.layers[0].ffn_in[1].shape = {256, ffn};  // up does not share gate's input
  const Weights narrow = RandomWeights(GUFO_ORACLE_Q4_K, ffn, 256, rng);
  bad.layers[0].ffn_in[1].data = narrow.bytes.data();
  Report("mismatched stage input throws std::runtime_error",
         Throws<std::runtime_error>([&] { HipProjections p(bad); }));
  bad = model;
  bad.layers[0].ffn_down[0].shape = {ffn, hidden, 2};
  Report("wrong rank throws std::runtime_error",
         Throws<std::runtime_error>([&] { HipProjections p(bad); }));
  bad = model;
  bad.layers[0].ffn_down[0].shape = {700, hidden};
  Report("partial block throws std::invalid_argument",
         Throws<std::invalid_argument>([&] { HipProjections p(bad); }));
  bad = model;
  bad.layers[0].ffn_down[0].ggml_type = 1;  // F16: not a row type GgufProjections takes
  Report("unsupported type throws std::invalid_argument",
         Throws<std::invalid_argument>([&] { HipProjections p(bad); }));
}

void RunMoe(std::mt19937& rng) {
  const int experts = 8, top = 3;
  const std::size_t hidden = 512, ffn = 256;
  const Weights gate = RandomWeights(GUFO_ORACLE_Q4_K, experts * ffn, hidden, rng);
  const Weights up = RandomWeights(GUFO_ORACLE_Q4_K, experts * ffn, hidden, rng);
  const Weights down = RandomWeights(GUFO_ORACLE_Q5_K, experts * hidden, ffn, rng);
  ModelTensors model;
  model.hidden = static_cast<int>(hidden);
  model.experts = experts;
  model.expert_ffn = static_cast<int>(ffn);
  LayerTensors layer;
  layer.gate_exps = AsTensor("blk.0.ffn_gate_exps.weight", gate, experts);
  layer.up_exps = AsTensor("blk.0.ffn_up_exps.weight", up, experts);
  layer.down_exps = AsTensor("blk.0.ffn_down_exps.weight", down, experts);
  model.layers.push_back(layer);
  const HipProjections proj(model);

  for (const int expert : {0, 5, 7}) {
    for (const int tokens : {1, 4}) {
      const auto e = static_cast<std::size_t>(expert);
      const auto x = RandomActivations(static_cast<std::size_t>(tokens) * hidden, rng);
      const auto want = Expected({&gate, &up}, {e * ffn, e * ffn}, {ffn, ffn}, x, tokens);
      std::vector<float> got(want.size());
      proj.ApplyExpert(Stage::kExpertIn, 0, expert, x.data(), tokens, got.data());
      double err = RelL2(got, want);
      Report("kExpertIn expert " + std::to_string(expert) + " tokens=" + std::to_string(tokens),
             err <= kTolerance, err);
      const auto a = RandomActivations(static_cast<std::size_t>(tokens) * ffn, rng);
      const auto want_down = Expected({&down}, {e * hidden}, {hidden}, a, tokens);
      std::vector<float> got_down(want_down.size());
      proj.ApplyExpert(Stage::kExpertDown, 0, expert, a.data(), tokens, got_down.data());
      err = RelL2(got_down, want_down);
      Report("kExpertDown expert " + std::to_string(expert) + " tokens=" + std::to_string(tokens),
             err <= kTolerance, err);
    }
  }

  // Route + the routed FFN against the checker's Reference::Ffn restatement.
  const int tokens = 6;
  const auto logits = RandomActivations(static_cast<std::size_t>(tokens) * experts, rng);
  const auto x = RandomActivations(static_cast<std::size_t>(tokens) * hidden, rng, 0.05f);
  std::vector<int> chosen(tokens * top), want_chosen(tokens * top);
  std::vector<float> weights(tokens * top), want_weights(tokens * top);
  std::vector<float> y(tokens * hidden), want_y(tokens * hidden);
  proj.Route(logits.data(), tokens, top, chosen.data(), weights.data());
  gufo_oracle_moe_ffn(gate.bytes.data(), gate.type, up.bytes.data(), up.type, down.bytes.data(),
                      down.type, experts, static_cast<int>(hidden), static_cast<int>(ffn),
                      logits.data(), x.data(), tokens, top, want_chosen.data(),
                      want_weights.data(), want_y.data(), 1, 4);
  Report("Route indices identical", chosen == want_chosen);
  Report("Route weights", RelL2(weights, want_weights) <= 1e-6, RelL2(weights, want_weights));
  proj.RoutedFfn(0, x.data(), tokens, chosen.data(), weights.data(), top, y.data());
  Report("RoutedFfn", RelL2(y, want_y) <= kTolerance, RelL2(y, want_y));

  std::vector<float> scratch(4096);
  Report("expert out of range throws std::logic_error", Throws<std::logic_error>([&] {
           proj.ApplyExpert(Stage::kExpertIn, 0, experts, x.data(), 1, scratch.data());
         }));
  Report("ApplyExpert with a dense stage throws std::logic_error", Throws<std::logic_error>([&] {
           proj.ApplyExpert(Stage::kFfnIn, 0, 0, x.data(), 1, scratch.data());
         }));
  ModelTensors bad = model;
  bad.layers[0].down_exps.shape = {ffn, hidden, 4};
  Report("expert tensor with the wrong expert count throws std::runtime_error",
         Throws<std::runtime_error>([&] { HipProjections p(bad); }));
}

// Rows of floats in device memory.
class DeviceRows {
public:
  explicit DeviceRows(std::size_t n) : n_(n) {
    void* p = nullptr;
    if (gufo_hip_malloc(&p, n * sizeof(float)) != GUFO_HIP_OK) throw std::bad_alloc();
    data_ = static_cast<float*>(p);
  }
  explicit DeviceRows(const std::vector<float>& host) : DeviceRows(host.size()) {
    gufo_hip_memcpy_h2d(data_, host.data(), n_ * sizeof(float));
  }
  ~DeviceRows() { gufo_hip_free(data_); }
  DeviceRows(const DeviceRows&) = delete;
  DeviceRows& operator=(const DeviceRows&) = delete;
  float* get() const { return data_; }
  std::vector<float> Download() const {
    std::vector<float> host(n_);
    gufo_hip_memcpy_d2h(host.data(), data_, n_ * sizeof(float));
    return host;
  }

private:
  std::size_t n_;
  float* data_ = nullptr;
};

// The second half of a dense decoder layer on rows that stay on the device
// (src/models/qwen35/decoder.cpp:504-515,519-521 of the reference): the residual add
// and RmsNorm inside the kFfnIn product, SwiGLU inside the kFfnDown product - two
// launches - against the same steps taken one at a time by the checker.
void RunDeviceChain(std::mt19937& rng) {
  const std::size_t hidden = 512, ffn = 768;
  const float eps = 1e-6f;
  const Weights gate = RandomWeights(GUFO_ORACLE_Q4_K, ffn, hidden, rng);
  const Weights up = RandomWeights(GUFO_ORACLE_Q4_K, ffn, hidden, rng);
  const Weights down = RandomWeights(GUFO_ORACLE_Q6_K, hidden, ffn, rng);
  ModelTensors model;
  model.hidden = static_cast<int>(hidden);
  LayerTensors layer;
  layer.ffn_in = {AsTensor("blk.0.ffn_gate.weight", gate), AsTensor("blk.0.ffn_up.weight", up)};
  layer.ffn_down = {AsTensor("blk.0.ffn_down.weight", down)};
  model.layers.push_back(layer);
  const HipProjections proj(model);

  for (const int tokens : {1, 2, 4}) {
    const auto n = static_cast<std::size_t>(tokens);
    const auto h = RandomActivations(n * hidden, rng);
    const auto mixer_out = RandomActivations(n * hidden, rng, 0.5f);
    auto norm_weight = RandomActivations(hidden, rng, 0.1f);
    for (auto& w : norm_weight) w += 1.0f;

    std::vector<float> want_h(n * hidden), normed(n * hidden), act(n * ffn);
    for (std::size_t t = 0; t < n; ++t) {
      gufo_oracle_res_norm(&h[t * hidden], &mixer_out[t * hidden], norm_weight.data(), hidden,
                           eps, &want_h[t * hidden], &normed[t * hidden]);
    }
    auto gate_up = ExpectedWhole({&gate, &up}, normed, tokens);
    // Synthetic weights are not zero-mean: keep the activation of order one.
    for (auto& v : gate_up) v *= 1.0f / 64;
    for (std::size_t t = 0; t < n; ++t) {
      gufo_oracle_swiglu(&gate_up[t * 2 * ffn], ffn, &act[t * ffn]);
    }
    const auto want_y = ExpectedWhole({&down}, act, tokens);

    const DeviceRows d_h(h), d_mixer(mixer_out), d_weight(norm_weight);
    const DeviceRows d_residual(n * hidden), d_gate_up(n * 2 * ffn), d_y(n * hidden);
    HipProjections::DeviceInput in;
    in.prologue = HipProjections::Prologue::kResNorm;
    in.x = d_h.get();
    in.delta = d_mixer.get();
    in.norm_weight = d_weight.get();
    in.eps = eps;
    in.residual = d_residual.get();
    proj.ApplyDevice(Stage::kFfnIn, 0, in, tokens, d_gate_up.get());
    auto scaled = d_gate_up.Download();
    for (auto& v : scaled) v *= 1.0f / 64;
    const DeviceRows d_scaled(scaled);
    HipProjections::DeviceInput act_in;
    act_in.prologue = HipProjections::Prologue::kSwiGlu;
    act_in.x = d_scaled.get();
    proj.ApplyDevice(Stage::kFfnDown, 0, act_in, tokens, d_y.get());

    const std::string tag = " tokens=" + std::to_string(tokens);
    Report("ApplyDevice kResNorm residual row is x + delta exactly" + tag,
           d_residual.Download() == want_h);
    double err = RelL2(scaled, gate_up);
    Report("ApplyDevice kFfnIn with kResNorm" + tag, err <= kTolerance, err);
    err = RelL2(d_y.Download(), want_y);
    Report("ApplyDevice kFfnDown with kSwiGlu" + tag, err <= 2 * kTolerance, err);
  }
  const DeviceRows d_x(std::vector<float>(hidden, 1.0f)), d_y(2 * ffn);
  HipProjections::DeviceInput no_weight;
  no_weight.prologue = HipProjections::Prologue::kResNorm;
  no_weight.x = d_x.get();
  Report("kResNorm without a norm weight throws std::invalid_argument",
         Throws<std::invalid_argument>(
             [&] { proj.ApplyDevice(Stage::kFfnIn, 0, no_weight, 1, d_y.get()); }));
  Report("ApplyDevice on a missing stage throws std::logic_error", Throws<std::logic_error>([&] {
           proj.ApplyDevice(Stage::kRouter, 0, no_weight, 1, d_y.get());
         }));
}

// The greedy token straight from the head product: PickDevice against Apply followed by
// std::max_element, with and without the output norm in front.
void RunPick(std::mt19937& rng) {
  const std::size_t hidden = 512, vocab = 3000;
  const Weights head = RandomWeights(GUFO_ORACLE_Q6_K, vocab, hidden, rng);
  ModelTensors model;
  model.hidden = static_cast<int>(hidden);
  model.lm_head = AsTensor("token_embd.weight", head);
  const HipProjections proj(model);
  for (const int tokens : {1, 4}) {
    const auto n = static_cast<std::size_t>(tokens);
    const auto x = RandomActivations(n * hidden, rng);
    std::vector<float> logits(n * vocab);
    proj.Apply(Stage::kLmHead, -1, x.data(), tokens, logits.data());
    const DeviceRows d_x(x), d_index(2 * n);  // 2 floats = one int64 per token
    HipProjections::DeviceInput in;
    in.x = d_x.get();
    proj.PickDevice(Stage::kLmHead, -1, in, tokens, reinterpret_cast<std::int64_t*>(d_index.get()));
    const auto raw = d_index.Download();
    bool same = true;
    for (std::size_t t = 0; t < n; ++t) {
      std::int64_t got;
      std::memcpy(&got, &raw[2 * t], sizeof got);
      const float* row = &logits[t * vocab];
      same = same && got == std::max_element(row, row + vocab) - row;
    }
    Report("PickDevice kLmHead equals max_element of Apply tokens=" + std::to_string(tokens),
           same);
  }
}

// A stage for many tokens on the matrix cores: PrefillDevice against Apply on the same
// (bf16-representable) activations, before and after PreparePrefill.
void RunPrefill(std::mt19937& rng) {
  const std::size_t hidden = 512, ffn = 320, tokens = 70;
  const Weights gate = RandomWeights(GUFO_ORACLE_Q4_K, ffn, hidden, rng);
  const Weights up = RandomWeights(GUFO_ORACLE_Q5_K, ffn, hidden, rng);
  ModelTensors model;
  model.hidden = static_cast<int>(hidden);
  LayerTensors layer;
  layer.ffn_in = {AsTensor("blk.0.ffn_gate.weight", gate), AsTensor("blk.0.ffn_up.weight", up)};
  model.layers.push_back(layer);
  HipProjections proj(model);

  auto x = RandomActivations(tokens * hidden, rng);
  std::vector<std::uint16_t> bits(x.size());
  for (std::size_t i = 0; i < x.size(); ++i) {  // round to bf16, nearest even
    std::uint32_t u;
    std::memcpy(&u, &x[i], 4);
    u = (u + 0x7FFFu + ((u >> 16) & 1u)) & 0xFFFF0000u;
    std::memcpy(&x[i], &u, 4);
    bits[i] = static_cast<std::uint16_t>(u >> 16);
  }
  std::vector<float> want(tokens * 2 * ffn);
  proj.Apply(Stage::kFfnIn, 0, x.data(), static_cast<int>(tokens), want.data());

  void* d_bits = nullptr;
  if (gufo_hip_malloc(&d_bits, bits.size() * 2) != GUFO_HIP_OK) throw std::bad_alloc();
  gufo_hip_memcpy_h2d(d_bits, bits.data(), bits.size() * 2);
  const DeviceRows d_c(want.size());
  proj.PrefillDevice(Stage::kFfnIn, 0, static_cast<const std::uint16_t*>(d_bits), tokens,
                     d_c.get());
  const auto first = d_c.Download();
  double err = RelL2(first, want);
  Report("PrefillDevice kFfnIn equals Apply within 1e-3", err <= 1e-3, err);
  proj.PreparePrefill(Stage::kFfnIn, 0);
  proj.PrefillDevice(Stage::kFfnIn, 0, static_cast<const std::uint16_t*>(d_bits), tokens,
                     d_c.get());
  Report("PrefillDevice after PreparePrefill: the same bits", d_c.Download() == first);
  Report("PrefillDevice on a missing stage throws std::logic_error", Throws<std::logic_error>([&] {
           proj.PrefillDevice(Stage::kFfnDown, 0, static_cast<const std::uint16_t*>(d_bits),
                              tokens, d_c.get());
         }));
  gufo_hip_free(d_bits);
}

// Decoder::MoeFfn in one call on device rows (src/models/qwen35/decoder.cpp:530-558)
// against the same steps through the host-pointer methods: the kRouter product (two
// tensors: the experts' rows and the shared expert's gate row), Route, RoutedFfn, and the
// shared expert's rows scaled by the sigmoid of the last logit.
void RunMoeLayer(std::mt19937& rng) {
  const int experts = 8, top = 3;
  const std::size_t hidden = 512, ffn = 256;
  const Weights gate = RandomWeights(GUFO_ORACLE_Q4_K, experts * ffn, hidden, rng);
  const Weights up = RandomWeights(GUFO_ORACLE_Q4_K, experts * ffn, hidden, rng);
  const Weights down = RandomWeights(GUFO_ORACLE_Q6_K, experts * hidden, ffn, rng);
  const Weights router = RandomWeights(GUFO_ORACLE_Q5_K, experts, hidden, rng);
  const Weights shared_gate = RandomWeights(GUFO_ORACLE_Q5_K, 1, hidden, rng);
  ModelTensors model;
  model.hidden = static_cast<int>(hidden);
  model.experts = experts;
  model.expert_ffn = static_cast<int>(ffn);
  LayerTensors layer;
  layer.gate_exps = AsTensor("blk.0.ffn_gate_exps.weight", gate, experts);
  layer.up_exps = AsTensor("blk.0.ffn_up_exps.weight", up, experts);
  layer.down_exps = AsTensor("blk.0.ffn_down_exps.weight", down, experts);
  layer.router = {AsTensor("blk.0.ffn_gate_inp.weight", router),
                  AsTensor("blk.0.ffn_gate_inp_shexp.weight", shared_gate)};
  model.layers.push_back(layer);
  const HipProjections proj(model);

  for (const int tokens : {1, 5}) {
    const auto n = static_cast<std::size_t>(tokens);
    const auto x = RandomActivations(n * hidden, rng, 0.02f);
    const auto shared = RandomActivations(n * hidden, rng, 100.0f);
    std::vector<float> logits(n * (experts + 1)), routing(n * experts);
    proj.Apply(Stage::kRouter, 0, x.data(), tokens, logits.data());
    for (std::size_t t = 0; t < n; ++t) {
      std::copy_n(&logits[t * (experts + 1)], experts, &routing[t * experts]);
    }
    std::vector<int> chosen(n * top);
    std::vector<float> weights(n * top), routed(n * hidden), want(n * hidden);
    proj.Route(routing.data(), tokens, top, chosen.data(), weights.data());
    proj.RoutedFfn(0, x.data(), tokens, chosen.data(), weights.data(), top, routed.data());
    for (std::size_t t = 0; t < n; ++t) {
      const double logit = logits[t * (experts + 1) + experts];
      const auto scale = static_cast<float>(1.0 / (1.0 + std::exp(-logit)));
      for (std::size_t i = 0; i < hidden; ++i) {
        want[t * hidden + i] = static_cast<float>(
            static_cast<double>(shared[t * hidden + i] * scale) + routed[t * hidden + i]);
      }
    }
    const DeviceRows d_x(x), d_shared(shared), d_y(n * hidden);
    proj.MoeLayerDevice(0, d_x.get(), tokens, top, d_shared.get(), d_y.get());
    const std::string tag = " tokens=" + std::to_string(tokens);
    double err = RelL2(d_y.Download(), want);
    Report("MoeLayerDevice with a shared expert" + tag, err <= 1e-6, err);
    proj.MoeLayerDevice(0, d_x.get(), tokens, top, nullptr, d_y.get());
    err = RelL2(d_y.Download(), routed);
    Report("MoeLayerDevice without one equals RoutedFfn" + tag, err == 0.0, err);
  }
}

}  // namespace

int main(int argc, char** argv) {
  if (argc > 1 && std::string(argv[1]) == "--no-device") return RunNoDevice();
  std::mt19937 rng(20261105);
  try {
    RunDense(rng);
    RunMoe(rng);
    RunMoeLayer(rng);
    RunPrefill(rng);
    RunDeviceChain(rng);
    RunPick(rng);
  } catch (const std::exception& e) {
    std::fprintf(stderr, "FAIL: unexpected exception: %s\n", e.what());
    return 1;
  }
  if (g_failures != 0) {
    std::fprintf(stderr, "FAIL: %d cases\n", g_failures);
    return 1;
  }
  std::puts("PASS");
  return 0;
}
