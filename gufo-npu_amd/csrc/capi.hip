// The C-ABI of include/gufo_hip.h: argument checks, device residency of the
// matrices, launch planning and the one stream every call is ordered on.
#include "../../include/gufo_hip.h"

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <new>
#include <string>

#include "kernels.hpp"
#include "kquant_common.hpp"

struct gufo_hip_matrix {
  int type;
  size_t rows;
  size_t cols;
  size_t row_bytes;
  size_t bytes;
  uint8_t* data;  // device
  // The weights as fp16 fragments for the prefill product, once
  // gufo_hip_matrix_prepare_prefill has been called (device; null before).
  void* prefill_fragments = nullptr;
};

struct gufo_hip_graph {
  hipGraph_t graph;
  hipGraphExec_t exec;
};

namespace {

using gufo::GemvLaunch;
using gufo::kMaxGemvParts;
using gufo::kMaxGemvTokens;

thread_local std::string t_error;

int Fail(int code, const char* format, ...) {
  char text[512];
  va_list args;
  va_start(args, format);
  std::vsnprintf(text, sizeof text, format, args);
  va_end(args);
  t_error = text;
  return code;
}

// A device allocation that only grows.  Growing waits for the stream first: work
// in flight may still use the old block.
struct Scratch {
  void* ptr = nullptr;
  size_t capacity = 0;
};

struct State {
  std::mutex mutex;
  bool ready = false;
  int device = -1;
  hipStream_t stream = nullptr;
  hipEvent_t timer_begin = nullptr;
  hipEvent_t timer_end = nullptr;
  char name[256] = {0};
  int compute_units = 0;
  long live_matrices = 0;
  bool moe_pending = false;  // an expert call since the last synchronize
  bool capturing = false;    // between capture_begin and capture_end
  Scratch small;             // argmax partials + result, MoE tables header
  Scratch stage_x;           // host-pointer variants: device copies of x, y, ...
  Scratch stage_y;
  Scratch stage_ids;
  Scratch stage_weights;
  Scratch moe_tables;   // counts, offsets, pairs, valid flags, segments
  Scratch moe_gate_up;  // pairs x 2*ffn
  Scratch moe_out;      // pairs x hidden
  Scratch moe_route;    // whole-layer call: router logits, then ids, then weights
  Scratch gemm_work;    // prefill: both operands as fp16
  Scratch stage_c;      // prefill, host-pointer variant: device copy of C
};

State g_state;

#define GUFO_HIP_TRY(expr)                                                        \
  do {                                                                            \
    const hipError_t gufo_status_ = (expr);                                       \
    if (gufo_status_ != hipSuccess) {                                             \
      return Fail(gufo_status_ == hipErrorOutOfMemory ? GUFO_HIP_ERR_OUT_OF_MEMORY \
                                                      : GUFO_HIP_ERR_RUNTIME,     \
                  "%s: %s", #expr, hipGetErrorString(gufo_status_));              \
    }                                                                             \
  } while (0)

#define GUFO_TRY(expr)                      \
  do {                                      \
    const int gufo_code_ = (expr);          \
    if (gufo_code_ != GUFO_HIP_OK) return gufo_code_; \
  } while (0)

int RequireReady() {
  if (!g_state.ready) {
    return Fail(GUFO_HIP_ERR_NOT_INITIALIZED, "gufo_hip_init has not been called");
  }
  return GUFO_HIP_OK;
}

int Reserve(Scratch* s, size_t bytes) {
  if (bytes <= s->capacity) return GUFO_HIP_OK;
  if (g_state.capturing) {
    return Fail(GUFO_HIP_ERR_LOGIC,
                "a recorded call needs %zu bytes of scratch; make the same call once "
                "before recording",
                bytes);
  }
  GUFO_HIP_TRY(hipStreamSynchronize(g_state.stream));
  if (s->ptr != nullptr) {
    GUFO_HIP_TRY(hipFree(s->ptr));
    s->ptr = nullptr;
    s->capacity = 0;
  }
  const size_t rounded = (bytes + 0xFFFFu) & ~static_cast<size_t>(0xFFFFu);
  GUFO_HIP_TRY(hipMalloc(&s->ptr, rounded));
  s->capacity = rounded;
  return GUFO_HIP_OK;
}

void Release(Scratch* s) {
  if (s->ptr != nullptr) (void)hipFree(s->ptr);
  s->ptr = nullptr;
  s->capacity = 0;
}

// Layout of State::small.
constexpr size_t kArgmaxPartialBytes = static_cast<size_t>(gufo::kArgmaxBlocks) * 8;
constexpr size_t kArgmaxResultOffset = kArgmaxPartialBytes;
constexpr size_t kMoeHeaderOffset = kArgmaxResultOffset + 64;
// The product with the pick inside: per-workgroup candidates of up to four tokens (at
// most kPickGroups workgroups per launch).
constexpr size_t kPickGroups = 1024;
constexpr size_t kPickPartialOffset = kMoeHeaderOffset + 64;
constexpr size_t kSmallBytes = kPickPartialOffset + kMaxGemvTokens * kPickGroups * 8;

// Device addresses of the grouping tables inside State::moe_tables.
struct MoeTablePointers {
  int* counts;
  int* offsets;
  int* pairs;
  uint8_t* valid;
  gufo::MoeSegment* segments;
  gufo::MoeTables* header;
};

size_t Align16(size_t v) { return (v + 15) & ~static_cast<size_t>(15); }

int ReserveMoeTables(int n_pairs, int experts, MoeTablePointers* out) {
  const size_t counts_bytes = Align16(sizeof(int) * static_cast<size_t>(experts));
  const size_t offsets_bytes = Align16(sizeof(int) * (static_cast<size_t>(experts) + 1));
  const size_t pairs_bytes = Align16(sizeof(int) * static_cast<size_t>(n_pairs));
  const size_t valid_bytes = Align16(static_cast<size_t>(n_pairs));
  const size_t segment_bytes =
      Align16(sizeof(gufo::MoeSegment) * static_cast<size_t>(n_pairs));
  GUFO_TRY(Reserve(&g_state.moe_tables, counts_bytes + offsets_bytes + pairs_bytes +
                                            valid_bytes + segment_bytes + 16));
  uint8_t* base = static_cast<uint8_t*>(g_state.moe_tables.ptr);
  out->counts = reinterpret_cast<int*>(base);
  base += counts_bytes;
  out->offsets = reinterpret_cast<int*>(base);
  base += offsets_bytes;
  out->pairs = reinterpret_cast<int*>(base);
  base += pairs_bytes;
  out->valid = base;
  base += valid_bytes;
  out->segments = reinterpret_cast<gufo::MoeSegment*>(base);
  out->header = reinterpret_cast<gufo::MoeTables*>(
      static_cast<uint8_t*>(g_state.small.ptr) + kMoeHeaderOffset);
  return GUFO_HIP_OK;
}

bool Aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// The checks GgufProjections makes when it is built and when a stage is applied
// (src/models/qwen35/gguf_projections.cpp:27-46,213-215 of the reference).
int CheckParts(const gufo_hip_matrix* const* parts, const size_t* first_row,
               const size_t* n_rows, int n_parts, int tokens, size_t* stride) {
  if (n_parts <= 0 || parts == nullptr || first_row == nullptr || n_rows == nullptr) {
    return Fail(GUFO_HIP_ERR_LOGIC, "no weights for this product (n_parts = %d)", n_parts);
  }
  if (tokens < 0) return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "tokens = %d", tokens);
  size_t total = 0;
  for (int p = 0; p < n_parts; ++p) {
    if (parts[p] == nullptr) return Fail(GUFO_HIP_ERR_LOGIC, "part %d has no matrix", p);
    if (parts[p]->cols != parts[0]->cols) {
      return Fail(GUFO_HIP_ERR_SHAPE,
                  "part %d has %zu columns, expected %zu: parts of one product share "
                  "their input",
                  p, parts[p]->cols, parts[0]->cols);
    }
    if (first_row[p] > parts[p]->rows || n_rows[p] > parts[p]->rows - first_row[p]) {
      return Fail(GUFO_HIP_ERR_OUT_OF_RANGE,
                  "part %d: rows [%zu, %zu) of a matrix with %zu rows", p, first_row[p],
                  first_row[p] + n_rows[p], parts[p]->rows);
    }
    total += n_rows[p];
  }
  if (total > 0xFFFFFFF0ull) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "%zu output rows exceed the launch limit",
                total);
  }
  *stride = total;
  return GUFO_HIP_OK;
}

bool Overlap(const void* a, size_t a_bytes, const void* b, size_t b_bytes) {
  if (a == nullptr || b == nullptr) return false;
  const uintptr_t a0 = reinterpret_cast<uintptr_t>(a);
  const uintptr_t b0 = reinterpret_cast<uintptr_t>(b);
  return a0 < b0 + b_bytes && b0 < a0 + a_bytes;
}

// The operands of a prologue, checked for a call of `tokens` rows of `cols` values.
int CheckPrologue(const gufo::GemvPrologue& in, const float* x, const float* y, int tokens,
                  size_t cols, size_t stride) {
  if (in.kind == gufo::kProloguePlain || in.kind == gufo::kPrologueSwiGlu) return GUFO_HIP_OK;
  if (in.kind != gufo::kPrologueResNorm) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "unknown prologue kind %d", in.kind);
  }
  if (in.norm_weight == nullptr) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "the resnorm prologue needs a norm weight");
  }
  if (!(in.eps >= 0.0f)) return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "eps = %g", in.eps);
  if (!Aligned16(in.delta) || !Aligned16(in.norm_weight) || !Aligned16(in.residual_out) ||
      !Aligned16(in.normed_out)) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT,
                "the rows of a resnorm prologue must be 16-byte aligned");
  }
  // Workgroup 0 stores these rows while the others still read x, delta and the weight.
  const size_t bytes = static_cast<size_t>(tokens) * cols * sizeof(float);
  const size_t y_bytes = static_cast<size_t>(tokens) * stride * sizeof(float);
  float* const outs[2] = {in.residual_out, in.normed_out};
  for (float* out : outs) {
    if (Overlap(out, bytes, x, bytes) || Overlap(out, bytes, in.delta, bytes) ||
        Overlap(out, bytes, in.norm_weight, cols * sizeof(float)) ||
        Overlap(out, bytes, y, y_bytes)) {
      return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT,
                  "residual_out and normed_out must not overlap x, delta, the norm weight "
                  "or y");
    }
  }
  if (Overlap(in.residual_out, bytes, in.normed_out, bytes)) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "residual_out and normed_out overlap");
  }
  return GUFO_HIP_OK;
}

int GemvDevLocked(const gufo_hip_matrix* const* parts, const size_t* first_row,
                  const size_t* n_rows, int n_parts, const gufo::GemvPrologue& in,
                  const float* x, int tokens, float* y) {
  size_t stride = 0;
  GUFO_TRY(CheckParts(parts, first_row, n_rows, n_parts, tokens, &stride));
  if (tokens == 0 || stride == 0) return GUFO_HIP_OK;
  if (x == nullptr || y == nullptr) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "x or y is null");
  }
  if (!Aligned16(x)) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "x must be 16-byte aligned");
  }
  const size_t cols = parts[0]->cols;
  GUFO_TRY(CheckPrologue(in, x, y, tokens, cols, stride));
  if (in.kind != gufo::kProloguePlain) {
    for (int p = 0; p < n_parts; ++p) {
      if (parts[p]->type == gufo::kTypeF32) {
        return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT,
                    "part %d holds fp32 rows, which take no prologue", p);
      }
    }
  }
  const size_t x_row_floats = in.kind == gufo::kPrologueSwiGlu ? 2 * cols : cols;
  // Token columns per pass over the weights: what the narrowest type's LDS need
  // allows for rows this wide.
  int per_pass = kMaxGemvTokens;
  for (int p = 0; p < n_parts; ++p) {
    const int fit = gufo::GemvMaxTokens(parts[p]->type,
                                        static_cast<uint32_t>(cols / gufo::kSuperBlock));
    if (fit < per_pass) per_pass = fit;
  }
  if (per_pass < 1) {
    return Fail(GUFO_HIP_ERR_SHAPE, "rows of %zu values exceed what one workgroup can stage",
                cols);
  }
  for (int t0 = 0; t0 < tokens; t0 += per_pass) {
    const int nt = tokens - t0 < per_pass ? tokens - t0 : per_pass;
    size_t offset = 0;
    int p = 0;
    while (p < n_parts) {
      // One launch per run of parts of one type.
      GemvLaunch launch;
      std::memset(&launch, 0, sizeof launch);
      const int type = parts[p]->type;
      uint32_t total = 0;
      uint32_t count = 0;
      while (p < n_parts && parts[p]->type == type &&
             count < static_cast<uint32_t>(kMaxGemvParts)) {
        launch.part[count].rows = parts[p]->data + first_row[p] * parts[p]->row_bytes;
        launch.part[count].n_rows = static_cast<uint32_t>(n_rows[p]);
        launch.part[count].y_offset = static_cast<uint32_t>(offset);
        offset += n_rows[p];
        total += static_cast<uint32_t>(n_rows[p]);
        ++count;
        ++p;
      }
      launch.n_parts = count;
      launch.total_rows = total;
      launch.blocks_per_row = static_cast<uint32_t>(cols / gufo::kSuperBlock);
      launch.y_stride = static_cast<uint32_t>(stride);
      // The operands of this pass's first token.
      gufo::GemvPrologue pass_in = in;
      const size_t row0 = static_cast<size_t>(t0) * cols;
      if (in.delta != nullptr) pass_in.delta = in.delta + row0;
      if (in.residual_out != nullptr) pass_in.residual_out = in.residual_out + row0;
      if (in.normed_out != nullptr) pass_in.normed_out = in.normed_out + row0;
      GUFO_HIP_TRY(gufo::LaunchGemvFused(type, launch, pass_in,
                                         x + static_cast<size_t>(t0) * x_row_floats, nt,
                                         y + static_cast<size_t>(t0) * stride,
                                         g_state.stream));
    }
  }
  return GUFO_HIP_OK;
}

int ToPrologue(const gufo_hip_prologue* prologue, gufo::GemvPrologue* in) {
  *in = gufo::GemvPrologue{};
  if (prologue == nullptr) return GUFO_HIP_OK;
  switch (prologue->kind) {
    case GUFO_HIP_PROLOGUE_PLAIN: in->kind = gufo::kProloguePlain; break;
    case GUFO_HIP_PROLOGUE_SWIGLU: in->kind = gufo::kPrologueSwiGlu; break;
    case GUFO_HIP_PROLOGUE_RESNORM:
      in->kind = gufo::kPrologueResNorm;
      in->delta = prologue->delta_dev;
      in->norm_weight = prologue->norm_weight_dev;
      in->eps = prologue->eps;
      in->residual_out = prologue->residual_out_dev;
      in->normed_out = prologue->normed_out_dev;
      break;
    default:
      return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "unknown prologue kind %d", prologue->kind);
  }
  return GUFO_HIP_OK;
}

// The product and the greedy pick over each of its rows: index[t] = position of the first
// maximum of y[t].  The pick rides inside the product's kernel when the call is a single
// launch of the quantized kernels; otherwise the product goes into library scratch and
// the pick kernels read it.
int PickDevLocked(const gufo_hip_matrix* const* parts, const size_t* first_row,
                  const size_t* n_rows, int n_parts, const gufo::GemvPrologue& in,
                  const float* x, int tokens, int64_t* index) {
  size_t stride = 0;
  GUFO_TRY(CheckParts(parts, first_row, n_rows, n_parts, tokens, &stride));
  if (tokens == 0) return GUFO_HIP_OK;
  if (stride == 0) return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "no output rows to pick from");
  if (x == nullptr || index == nullptr) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "x or index is null");
  }
  if (in.kind == gufo::kPrologueSwiGlu) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "the pick takes the plain and resnorm prologues");
  }
  const size_t cols = parts[0]->cols;
  const int type = parts[0]->type;
  bool one_launch = type != gufo::kTypeF32 && n_parts <= kMaxGemvParts &&
                    tokens <= gufo::GemvMaxTokens(type, static_cast<uint32_t>(cols / 256)) &&
                    gufo::GemvPickPartialBytes(tokens) <= kMaxGemvTokens * kPickGroups * 8;
  for (int p = 1; p < n_parts; ++p) one_launch = one_launch && parts[p]->type == type;
  if (!one_launch) {
    GUFO_TRY(Reserve(&g_state.stage_y, static_cast<size_t>(tokens) * stride * sizeof(float)));
    float* y = static_cast<float*>(g_state.stage_y.ptr);
    GUFO_TRY(GemvDevLocked(parts, first_row, n_rows, n_parts, in, x, tokens, y));
    for (int t = 0; t < tokens; ++t) {
      GUFO_HIP_TRY(gufo::LaunchArgmax(y + static_cast<size_t>(t) * stride, stride,
                                      g_state.small.ptr, index + t, g_state.stream));
    }
    return GUFO_HIP_OK;
  }
  if (!Aligned16(x)) return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "x must be 16-byte aligned");
  GUFO_TRY(CheckPrologue(in, x, nullptr, tokens, cols, stride));
  GemvLaunch launch;
  std::memset(&launch, 0, sizeof launch);
  size_t offset = 0;
  for (int p = 0; p < n_parts; ++p) {
    launch.part[p].rows = parts[p]->data + first_row[p] * parts[p]->row_bytes;
    launch.part[p].n_rows = static_cast<uint32_t>(n_rows[p]);
    launch.part[p].y_offset = static_cast<uint32_t>(offset);
    offset += n_rows[p];
  }
  launch.n_parts = static_cast<uint32_t>(n_parts);
  launch.total_rows = static_cast<uint32_t>(stride);
  launch.blocks_per_row = static_cast<uint32_t>(cols / gufo::kSuperBlock);
  launch.y_stride = static_cast<uint32_t>(stride);
  uint8_t* small = static_cast<uint8_t*>(g_state.small.ptr);
  gufo::GemvPick pick;
  pick.partial = small + kPickPartialOffset;
  pick.index = index;
  GUFO_HIP_TRY(gufo::LaunchGemvPick(type, launch, in, x, tokens, pick, g_state.stream));
  return GUFO_HIP_OK;
}

int CopyIn(Scratch* stage, const void* host, size_t bytes) {
  GUFO_TRY(Reserve(stage, bytes > 0 ? bytes : 16));
  if (bytes > 0) {
    GUFO_HIP_TRY(hipMemcpyAsync(stage->ptr, host, bytes, hipMemcpyHostToDevice,
                                g_state.stream));
  }
  return GUFO_HIP_OK;
}

int CopyOut(void* host, const void* device, size_t bytes) {
  if (bytes > 0) {
    GUFO_HIP_TRY(hipMemcpyAsync(host, device, bytes, hipMemcpyDeviceToHost,
                                g_state.stream));
  }
  GUFO_HIP_TRY(hipStreamSynchronize(g_state.stream));
  return GUFO_HIP_OK;
}

int RouteDevLocked(const float* logits, size_t logit_stride, int tokens, int experts, int k,
                   int* ids, float* weights) {
  if (tokens < 0 || k <= 0 || experts <= 0 || k > experts) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "route: tokens %d, experts %d, k %d",
                tokens, experts, k);
  }
  if (experts > gufo::kMaxRouteExperts || k > gufo::kMaxRouteK) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT,
                "route: at most %d experts and k <= %d are supported",
                gufo::kMaxRouteExperts, gufo::kMaxRouteK);
  }
  if (tokens == 0) return GUFO_HIP_OK;
  GUFO_HIP_TRY(gufo::LaunchRoute(logits, logit_stride, tokens, experts, k, ids, weights,
                                 g_state.stream));
  return GUFO_HIP_OK;
}

// segments_only: the caller reads the segment list, pair_valid and the header, not the
// per-expert counts, offsets and pair order.
int GroupDevLocked(const int* ids, int tokens, int k, int experts, bool segments_only,
                   MoeTablePointers* tables) {
  if (tokens < 0 || k <= 0 || experts <= 0) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "group: tokens %d, k %d, experts %d",
                tokens, k, experts);
  }
  const long n_pairs = static_cast<long>(tokens) * k;
  if (n_pairs > gufo::kMaxGroupPairs || experts > gufo::kMaxGroupExperts) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT,
                "group: at most %d (token, slot) pairs and %d experts per call",
                gufo::kMaxGroupPairs, gufo::kMaxGroupExperts);
  }
  GUFO_TRY(ReserveMoeTables(static_cast<int>(n_pairs > 0 ? n_pairs : 1), experts, tables));
  const int capacity = tokens < kMaxGemvTokens ? (tokens > 0 ? tokens : 1) : kMaxGemvTokens;
  if (segments_only && n_pairs <= gufo::kMaxSmallGroupPairs) {
    GUFO_HIP_TRY(gufo::LaunchMoeGroupSmall(ids, static_cast<int>(n_pairs), experts, capacity,
                                           tables->valid, tables->segments, tables->header,
                                           g_state.stream));
    return GUFO_HIP_OK;
  }
  GUFO_HIP_TRY(gufo::LaunchMoeGroup(ids, static_cast<int>(n_pairs), experts, capacity,
                                    tables->counts, tables->offsets, tables->pairs,
                                    tables->valid, tables->segments, tables->header,
                                    g_state.stream));
  return GUFO_HIP_OK;
}

int MoeFfnDevLocked(const gufo_hip_matrix* gate, const gufo_hip_matrix* up,
                    const gufo_hip_matrix* down, int experts, const float* x, int tokens,
                    const int* ids, const float* weights, int k,
                    const gufo::MoeShared& shared, float* y) {
  if (gate == nullptr || up == nullptr || down == nullptr) {
    return Fail(GUFO_HIP_ERR_LOGIC, "these projections have no MoE experts");
  }
  if (experts <= 0 || tokens < 0 || k <= 0) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "moe: experts %d, tokens %d, k %d",
                experts, tokens, k);
  }
  const size_t e = static_cast<size_t>(experts);
  const size_t hidden = gate->cols;
  if (gate->rows % e != 0 || up->rows != gate->rows || up->cols != hidden ||
      down->rows != e * hidden || down->cols * e != gate->rows) {
    return Fail(GUFO_HIP_ERR_SHAPE,
                "expert tensors gate [%zu x %zu], up [%zu x %zu], down [%zu x %zu] do "
                "not describe %d experts of one width",
                gate->rows, gate->cols, up->rows, up->cols, down->rows, down->cols,
                experts);
  }
  const size_t ffn = gate->rows / e;
  for (const gufo_hip_matrix* m : {gate, up, down}) {
    if (m->type != GUFO_HIP_Q4_K && m->type != GUFO_HIP_Q5_K && m->type != GUFO_HIP_Q6_K) {
      return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT,
                  "expert tensors must be Q4_K, Q5_K or Q6_K; this one has ggml type %d",
                  m->type);
    }
  }
  if (tokens == 0) return GUFO_HIP_OK;
  if (x == nullptr || y == nullptr || ids == nullptr || weights == nullptr) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "moe: null buffer");
  }
  if (!Aligned16(x)) return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "x must be 16-byte aligned");
  // One token: its slots are the segments, nothing to group (a kernel launch less per
  // decode step); the combine fills the header from the ids instead.
  const bool direct = tokens == 1;
  MoeTablePointers tables;
  if (direct) {
    GUFO_TRY(ReserveMoeTables(k, experts, &tables));
  } else {
    GUFO_TRY(GroupDevLocked(ids, tokens, k, experts, true, &tables));
  }
  const size_t n_pairs = static_cast<size_t>(tokens) * k;
  GUFO_TRY(Reserve(&g_state.moe_gate_up, n_pairs * 2 * ffn * sizeof(float)));
  GUFO_TRY(Reserve(&g_state.moe_out, n_pairs * hidden * sizeof(float)));
  float* gate_up = static_cast<float*>(g_state.moe_gate_up.ptr);
  float* routed = static_cast<float*>(g_state.moe_out.ptr);

  // The grouping kernel cuts segments at min(tokens, 4) pairs.
  const int max_pairs = tokens < kMaxGemvTokens ? tokens : kMaxGemvTokens;
  gufo::MoeGemvArgs args;
  std::memset(&args, 0, sizeof args);
  args.tables = tables.header;
  args.segments = tables.segments;
  args.k = static_cast<uint32_t>(k);
  args.direct_ids = direct ? ids : nullptr;
  args.experts = experts;

  // [gate | up] of every pair: kExpertIn's layout.
  args.x = x;
  args.x_row_floats = hidden;
  args.y = gate_up;
  const gufo_hip_matrix* in_parts[2] = {gate, up};
  for (int first = 0; first < 2;) {
    GemvLaunch launch;
    std::memset(&launch, 0, sizeof launch);
    int count = 0;
    const int type = in_parts[first]->type;
    for (int p = first; p < 2 && in_parts[p]->type == type; ++p) {
      launch.part[count].rows = in_parts[p]->data;
      launch.part[count].n_rows = static_cast<uint32_t>(ffn);
      launch.part[count].y_offset = static_cast<uint32_t>(p * ffn);
      ++count;
    }
    args.expert_bytes = ffn * in_parts[first]->row_bytes;
    launch.n_parts = static_cast<uint32_t>(count);
    launch.total_rows = static_cast<uint32_t>(count * ffn);
    launch.blocks_per_row = static_cast<uint32_t>(hidden / gufo::kSuperBlock);
    launch.y_stride = static_cast<uint32_t>(2 * ffn);
    GUFO_HIP_TRY(gufo::LaunchMoeGemv(type, launch, args, false,
                                     static_cast<uint32_t>(n_pairs), max_pairs,
                                     g_state.stream));
    first += count;
  }

  // down over silu(gate) * up of every pair.
  {
    GemvLaunch launch;
    std::memset(&launch, 0, sizeof launch);
    launch.part[0].rows = down->data;
    launch.part[0].n_rows = static_cast<uint32_t>(hidden);
    launch.part[0].y_offset = 0;
    launch.n_parts = 1;
    launch.total_rows = static_cast<uint32_t>(hidden);
    launch.blocks_per_row = static_cast<uint32_t>(ffn / gufo::kSuperBlock);
    launch.y_stride = static_cast<uint32_t>(hidden);
    args.x = gate_up;
    args.x_row_floats = 2 * ffn;
    args.y = routed;
    args.expert_bytes = hidden * down->row_bytes;
    GUFO_HIP_TRY(gufo::LaunchMoeGemv(down->type, launch, args, true,
                                     static_cast<uint32_t>(n_pairs), max_pairs,
                                     g_state.stream));
  }
  if (direct) {
    GUFO_HIP_TRY(gufo::LaunchMoeCombineDirect(routed, weights, ids, experts, k,
                                              static_cast<int>(hidden), shared, y,
                                              tables.header, g_state.stream));
  } else {
    GUFO_HIP_TRY(gufo::LaunchMoeCombine(routed, weights, tables.valid, tokens, k,
                                        static_cast<int>(hidden), shared, y, g_state.stream));
  }
  g_state.moe_pending = true;
  return GUFO_HIP_OK;
}

// After a synchronize: were any expert ids of the calls since the last one out of
// range?  GgufProjections::ApplyExpert throws std::logic_error for those
// (src/models/qwen35/gguf_projections.cpp:222-224 of the reference).
int CheckMoeIdsLocked() {
  if (!g_state.moe_pending) return GUFO_HIP_OK;
  g_state.moe_pending = false;
  gufo::MoeTables header;
  GUFO_HIP_TRY(hipMemcpy(&header,
                         static_cast<uint8_t*>(g_state.small.ptr) + kMoeHeaderOffset,
                         sizeof header, hipMemcpyDeviceToHost));
  if (header.n_invalid != 0) {
    return Fail(GUFO_HIP_ERR_LOGIC, "no such expert: %d routed ids were out of range",
                header.n_invalid);
  }
  return GUFO_HIP_OK;
}

}  // namespace

extern "C" {

int gufo_hip_init(int device) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  if (g_state.ready) {
    if (g_state.device == device) return GUFO_HIP_OK;
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT,
                "already initialised on device %d; shut down first", g_state.device);
  }
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) {
    (void)hipGetLastError();
    return Fail(GUFO_HIP_ERR_NO_DEVICE, "gufo_hip: no HIP device is available");
  }
  if (device < 0 || device >= count) {
    return Fail(GUFO_HIP_ERR_NO_DEVICE, "gufo_hip: device %d of %d does not exist", device,
                count);
  }
  hipDeviceProp_t prop;
  GUFO_HIP_TRY(hipGetDeviceProperties(&prop, device));
  if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
    return Fail(GUFO_HIP_ERR_NO_DEVICE,
                "gufo_hip: device %d is %s; this library is built for gfx950 only", device,
                prop.gcnArchName);
  }
  GUFO_HIP_TRY(hipSetDevice(device));
  GUFO_HIP_TRY(hipStreamCreateWithFlags(&g_state.stream, hipStreamNonBlocking));
  GUFO_HIP_TRY(hipEventCreate(&g_state.timer_begin));
  GUFO_HIP_TRY(hipEventCreate(&g_state.timer_end));
  std::snprintf(g_state.name, sizeof g_state.name, "%s (%s)", prop.gcnArchName, prop.name);
  g_state.compute_units = prop.multiProcessorCount;
  gufo::SetGemvComputeUnits(prop.multiProcessorCount);
  g_state.device = device;
  g_state.ready = true;
  const int code = Reserve(&g_state.small, kSmallBytes);
  if (code != GUFO_HIP_OK) {
    g_state.ready = false;
    return code;
  }
  GUFO_HIP_TRY(hipMemsetAsync(g_state.small.ptr, 0, kSmallBytes, g_state.stream));
  GUFO_HIP_TRY(hipStreamSynchronize(g_state.stream));
  return GUFO_HIP_OK;
}

int gufo_hip_shutdown(void) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  if (!g_state.ready) return GUFO_HIP_OK;
  if (g_state.live_matrices != 0) {
    return Fail(GUFO_HIP_ERR_LOGIC, "%ld matrices are still alive", g_state.live_matrices);
  }
  (void)hipStreamSynchronize(g_state.stream);
  Release(&g_state.small);
  Release(&g_state.stage_x);
  Release(&g_state.stage_y);
  Release(&g_state.stage_ids);
  Release(&g_state.stage_weights);
  Release(&g_state.moe_tables);
  Release(&g_state.moe_gate_up);
  Release(&g_state.moe_out);
  Release(&g_state.moe_route);
  Release(&g_state.gemm_work);
  Release(&g_state.stage_c);
  (void)hipEventDestroy(g_state.timer_begin);
  (void)hipEventDestroy(g_state.timer_end);
  (void)hipStreamDestroy(g_state.stream);
  g_state.stream = nullptr;
  g_state.ready = false;
  g_state.device = -1;
  return GUFO_HIP_OK;
}

const char* gufo_hip_last_error(void) { return t_error.c_str(); }

int gufo_hip_device_info(char* name, size_t name_bytes, int* compute_units) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  if (name != nullptr && name_bytes > 0) std::snprintf(name, name_bytes, "%s", g_state.name);
  if (compute_units != nullptr) *compute_units = g_state.compute_units;
  return GUFO_HIP_OK;
}

size_t gufo_hip_block_bytes(int ggml_type) {
  return static_cast<size_t>(gufo::FormatBlockBytes(ggml_type));
}

size_t gufo_hip_row_bytes(int ggml_type, size_t cols) {
  const size_t per_super_block = static_cast<size_t>(gufo::BlockBytes(ggml_type));
  if (per_super_block == 0 || cols % gufo::kSuperBlock != 0) return 0;
  return cols / gufo::kSuperBlock * per_super_block;
}

int gufo_hip_malloc(void** device_ptr, size_t bytes) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  if (device_ptr == nullptr) return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "null out pointer");
  *device_ptr = nullptr;
  GUFO_HIP_TRY(hipMalloc(device_ptr, bytes > 0 ? bytes : 16));
  return GUFO_HIP_OK;
}

int gufo_hip_free(void* device_ptr) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  if (device_ptr == nullptr) return GUFO_HIP_OK;
  GUFO_HIP_TRY(hipStreamSynchronize(g_state.stream));
  GUFO_HIP_TRY(hipFree(device_ptr));
  return GUFO_HIP_OK;
}

int gufo_hip_memcpy_h2d(void* device_dst, const void* host_src, size_t bytes) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  if (bytes == 0) return GUFO_HIP_OK;
  GUFO_HIP_TRY(hipMemcpyAsync(device_dst, host_src, bytes, hipMemcpyHostToDevice,
                              g_state.stream));
  GUFO_HIP_TRY(hipStreamSynchronize(g_state.stream));
  return GUFO_HIP_OK;
}

int gufo_hip_memcpy_d2h(void* host_dst, const void* device_src, size_t bytes) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  return CopyOut(host_dst, device_src, bytes);
}

int gufo_hip_synchronize(void) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  GUFO_HIP_TRY(hipStreamSynchronize(g_state.stream));
  return CheckMoeIdsLocked();
}

int gufo_hip_matrix_create(int ggml_type, const void* host_blocks, size_t rows,
                           size_t cols, gufo_hip_matrix** out) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  if (out == nullptr) return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "null out pointer");
  *out = nullptr;
  if (gufo_hip_block_bytes(ggml_type) == 0) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "unknown ggml type %d", ggml_type);
  }
  const size_t row_bytes = gufo_hip_row_bytes(ggml_type, cols);
  if (row_bytes == 0) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT,
                "row is not a whole number of blocks (%zu values; this backend takes rows "
                "of a multiple of 256 values for every type)",
                cols);
  }
  if (rows > 0xFFFFFFF0ull || cols > (1ull << 24)) {
    return Fail(GUFO_HIP_ERR_SHAPE, "matrix %zu x %zu exceeds the launch limits", rows, cols);
  }
  if (host_blocks == nullptr && rows != 0) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "null weight data");
  }
  gufo_hip_matrix* m = new (std::nothrow) gufo_hip_matrix;
  if (m == nullptr) return Fail(GUFO_HIP_ERR_OUT_OF_MEMORY, "host allocation failed");
  m->type = ggml_type;
  m->rows = rows;
  m->cols = cols;
  m->row_bytes = row_bytes;
  m->bytes = rows * row_bytes;
  m->data = nullptr;
  // 64 spare bytes: the last lanes of a wave may prefetch past the final block.
  const hipError_t status =
      hipMalloc(reinterpret_cast<void**>(&m->data), m->bytes + 64);
  if (status != hipSuccess) {
    delete m;
    return Fail(GUFO_HIP_ERR_OUT_OF_MEMORY, "hipMalloc of %zu bytes: %s", rows * row_bytes,
                hipGetErrorString(status));
  }
  hipError_t copy = hipSuccess;
  if (m->bytes > 0) {
    copy = hipMemcpyAsync(m->data, host_blocks, m->bytes, hipMemcpyHostToDevice,
                          g_state.stream);
  }
  if (copy == hipSuccess) {
    copy = hipMemsetAsync(m->data + m->bytes, 0, 64, g_state.stream);
  }
  if (copy == hipSuccess) copy = hipStreamSynchronize(g_state.stream);
  if (copy != hipSuccess) {
    (void)hipFree(m->data);
    delete m;
    return Fail(GUFO_HIP_ERR_RUNTIME, "upload of the matrix: %s", hipGetErrorString(copy));
  }
  ++g_state.live_matrices;
  *out = m;
  return GUFO_HIP_OK;
}

int gufo_hip_matrix_destroy(gufo_hip_matrix* m) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  if (m == nullptr) return GUFO_HIP_OK;
  GUFO_TRY(RequireReady());
  GUFO_HIP_TRY(hipStreamSynchronize(g_state.stream));
  if (m->prefill_fragments != nullptr) GUFO_HIP_TRY(hipFree(m->prefill_fragments));
  GUFO_HIP_TRY(hipFree(m->data));
  delete m;
  --g_state.live_matrices;
  return GUFO_HIP_OK;
}

int gufo_hip_matrix_prepare_prefill(gufo_hip_matrix* m) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  if (m == nullptr) return Fail(GUFO_HIP_ERR_LOGIC, "no weights for this product");
  if (!gufo::GemmTakesType(m->type)) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT,
                "the prefill GEMM takes Q4_K, Q5_K, Q6_K or Q8_0 weights; this matrix has "
                "ggml type %d",
                m->type);
  }
  if (m->prefill_fragments != nullptr || m->rows == 0) return GUFO_HIP_OK;
  if (g_state.capturing) {
    return Fail(GUFO_HIP_ERR_LOGIC, "a matrix cannot be prepared while recording");
  }
  const uint32_t nb = static_cast<uint32_t>(m->cols / gufo::kSuperBlock);
  const size_t bytes = gufo::GemmWeightBytes(static_cast<uint32_t>(m->rows), nb);
  void* fragments = nullptr;
  const hipError_t status = hipMalloc(&fragments, bytes);
  if (status != hipSuccess) {
    return Fail(GUFO_HIP_ERR_OUT_OF_MEMORY, "hipMalloc of %zu bytes: %s", bytes,
                hipGetErrorString(status));
  }
  const hipError_t launched = gufo::LaunchGemmPrepareWeights(
      m->type, m->data, static_cast<uint32_t>(m->rows), nb, fragments, g_state.stream);
  if (launched != hipSuccess) {
    (void)hipFree(fragments);
    return Fail(GUFO_HIP_ERR_RUNTIME, "pre-pass: %s", hipGetErrorString(launched));
  }
  m->prefill_fragments = fragments;
  return GUFO_HIP_OK;
}

int gufo_hip_matrix_info(const gufo_hip_matrix* m, int* ggml_type, size_t* rows,
                         size_t* cols, size_t* bytes) {
  if (m == nullptr) return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "null matrix");
  if (ggml_type != nullptr) *ggml_type = m->type;
  if (rows != nullptr) *rows = m->rows;
  if (cols != nullptr) *cols = m->cols;
  if (bytes != nullptr) *bytes = m->bytes;
  return GUFO_HIP_OK;
}

int gufo_hip_gemv_dev(const gufo_hip_matrix* const* parts, const size_t* first_row,
                      const size_t* n_rows, int n_parts, const float* x_dev, int tokens,
                      float* y_dev) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  return GemvDevLocked(parts, first_row, n_rows, n_parts, gufo::GemvPrologue{}, x_dev, tokens,
                       y_dev);
}

int gufo_hip_gemv_fused_dev(const gufo_hip_matrix* const* parts, const size_t* first_row,
                            const size_t* n_rows, int n_parts,
                            const gufo_hip_prologue* prologue, const float* x_dev, int tokens,
                            float* y_dev) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  gufo::GemvPrologue in;
  GUFO_TRY(ToPrologue(prologue, &in));
  return GemvDevLocked(parts, first_row, n_rows, n_parts, in, x_dev, tokens, y_dev);
}

int gufo_hip_gemv_argmax_dev(const gufo_hip_matrix* const* parts, const size_t* first_row,
                             const size_t* n_rows, int n_parts,
                             const gufo_hip_prologue* prologue, const float* x_dev, int tokens,
                             int64_t* index_dev) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  gufo::GemvPrologue in;
  GUFO_TRY(ToPrologue(prologue, &in));
  return PickDevLocked(parts, first_row, n_rows, n_parts, in, x_dev, tokens, index_dev);
}

int gufo_hip_matrix_gather_rows(const gufo_hip_matrix* src, const int64_t* rows_host,
                                size_t n, gufo_hip_matrix** out) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  if (out == nullptr) return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "null out pointer");
  *out = nullptr;
  if (src == nullptr || (rows_host == nullptr && n != 0)) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "null matrix or row list");
  }
  for (size_t i = 0; i < n; ++i) {
    if (rows_host[i] < 0 || static_cast<uint64_t>(rows_host[i]) >= src->rows) {
      return Fail(GUFO_HIP_ERR_OUT_OF_RANGE, "row %lld of a matrix with %zu rows",
                  static_cast<long long>(rows_host[i]), src->rows);
    }
  }
  gufo_hip_matrix* m = new (std::nothrow) gufo_hip_matrix(*src);
  if (m == nullptr) return Fail(GUFO_HIP_ERR_OUT_OF_MEMORY, "host allocation failed");
  m->rows = n;
  m->bytes = n * src->row_bytes;
  m->data = nullptr;
  m->prefill_fragments = nullptr;  // the source's are its own
  hipError_t status = hipMalloc(reinterpret_cast<void**>(&m->data), m->bytes + 64);
  if (status != hipSuccess) {
    delete m;
    return Fail(GUFO_HIP_ERR_OUT_OF_MEMORY, "hipMalloc of %zu bytes: %s", n * src->row_bytes,
                hipGetErrorString(status));
  }
  // One device copy per run of consecutive rows (a draft vocabulary is mostly runs).
  for (size_t i = 0; i < n && status == hipSuccess;) {
    size_t run = 1;
    while (i + run < n && rows_host[i + run] == rows_host[i] + static_cast<int64_t>(run)) ++run;
    status = hipMemcpyAsync(m->data + i * src->row_bytes,
                            src->data + static_cast<size_t>(rows_host[i]) * src->row_bytes,
                            run * src->row_bytes, hipMemcpyDeviceToDevice, g_state.stream);
    i += run;
  }
  if (status == hipSuccess) status = hipMemsetAsync(m->data + m->bytes, 0, 64, g_state.stream);
  if (status == hipSuccess) status = hipStreamSynchronize(g_state.stream);
  if (status != hipSuccess) {
    (void)hipFree(m->data);
    delete m;
    return Fail(GUFO_HIP_ERR_RUNTIME, "gathering rows: %s", hipGetErrorString(status));
  }
  ++g_state.live_matrices;
  *out = m;
  return GUFO_HIP_OK;
}

int gufo_hip_gemv(const gufo_hip_matrix* const* parts, const size_t* first_row,
                  const size_t* n_rows, int n_parts, const float* x_host, int tokens,
                  float* y_host) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  size_t stride = 0;
  GUFO_TRY(CheckParts(parts, first_row, n_rows, n_parts, tokens, &stride));
  if (tokens == 0 || stride == 0) return GUFO_HIP_OK;
  if (x_host == nullptr || y_host == nullptr) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "x or y is null");
  }
  const size_t x_bytes = static_cast<size_t>(tokens) * parts[0]->cols * sizeof(float);
  const size_t y_bytes = static_cast<size_t>(tokens) * stride * sizeof(float);
  GUFO_TRY(CopyIn(&g_state.stage_x, x_host, x_bytes));
  GUFO_TRY(Reserve(&g_state.stage_y, y_bytes));
  GUFO_TRY(GemvDevLocked(parts, first_row, n_rows, n_parts, gufo::GemvPrologue{},
                         static_cast<const float*>(g_state.stage_x.ptr), tokens,
                         static_cast<float*>(g_state.stage_y.ptr)));
  return CopyOut(y_host, g_state.stage_y.ptr, y_bytes);
}

int gufo_hip_argmax_dev(const float* logits_dev, size_t n, int64_t* index_host) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  if (logits_dev == nullptr || index_host == nullptr || n == 0) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "argmax: empty input");
  }
  uint8_t* small = static_cast<uint8_t*>(g_state.small.ptr);
  int64_t* result = reinterpret_cast<int64_t*>(small + kArgmaxResultOffset);
  GUFO_HIP_TRY(gufo::LaunchArgmax(logits_dev, n, small, result, g_state.stream));
  return CopyOut(index_host, result, sizeof(int64_t));
}

int gufo_hip_route_topk_dev(const float* logits_dev, int tokens, int experts, int k,
                            int* ids_dev, float* weights_dev) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  return RouteDevLocked(logits_dev, static_cast<size_t>(experts > 0 ? experts : 0), tokens,
                        experts, k, ids_dev, weights_dev);
}

int gufo_hip_route_topk(const float* logits_host, int tokens, int experts, int k,
                        int* ids_host, float* weights_host) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  if (tokens < 0 || k <= 0 || experts <= 0 || k > experts) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "route: tokens %d, experts %d, k %d",
                tokens, experts, k);
  }
  if (tokens == 0) return GUFO_HIP_OK;
  const size_t n = static_cast<size_t>(tokens) * k;
  GUFO_TRY(CopyIn(&g_state.stage_x, logits_host,
                  static_cast<size_t>(tokens) * experts * sizeof(float)));
  GUFO_TRY(Reserve(&g_state.stage_ids, n * sizeof(int)));
  GUFO_TRY(Reserve(&g_state.stage_weights, n * sizeof(float)));
  GUFO_TRY(RouteDevLocked(static_cast<const float*>(g_state.stage_x.ptr),
                          static_cast<size_t>(experts), tokens, experts, k,
                          static_cast<int*>(g_state.stage_ids.ptr),
                          static_cast<float*>(g_state.stage_weights.ptr)));
  GUFO_TRY(CopyOut(ids_host, g_state.stage_ids.ptr, n * sizeof(int)));
  return CopyOut(weights_host, g_state.stage_weights.ptr, n * sizeof(float));
}

int gufo_hip_moe_group(const int* ids_host, int tokens, int k, int experts,
                       int* counts_host, int* offsets_host, int* pairs_host,
                       int* distinct_host) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  if (tokens < 0 || k <= 0 || experts <= 0) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "group: tokens %d, k %d, experts %d",
                tokens, k, experts);
  }
  const size_t n = static_cast<size_t>(tokens) * k;
  GUFO_TRY(CopyIn(&g_state.stage_ids, ids_host, n * sizeof(int)));
  MoeTablePointers tables;
  GUFO_TRY(GroupDevLocked(static_cast<const int*>(g_state.stage_ids.ptr), tokens, k,
                          experts, false, &tables));
  gufo::MoeTables header;
  GUFO_TRY(CopyOut(&header, tables.header, sizeof header));
  if (header.n_invalid != 0) {
    return Fail(GUFO_HIP_ERR_LOGIC, "no such expert: %d routed ids were out of range",
                header.n_invalid);
  }
  if (counts_host != nullptr) {
    GUFO_TRY(CopyOut(counts_host, tables.counts, sizeof(int) * experts));
  }
  if (offsets_host != nullptr) {
    GUFO_TRY(CopyOut(offsets_host, tables.offsets, sizeof(int) * (experts + 1)));
  }
  if (pairs_host != nullptr) GUFO_TRY(CopyOut(pairs_host, tables.pairs, sizeof(int) * n));
  if (distinct_host != nullptr) *distinct_host = header.n_distinct;
  return GUFO_HIP_OK;
}

int gufo_hip_moe_ffn_dev(const gufo_hip_matrix* gate, const gufo_hip_matrix* up,
                         const gufo_hip_matrix* down, int experts, const float* x_dev,
                         int tokens, const int* ids_dev, const float* weights_dev, int k,
                         float* y_dev) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  return MoeFfnDevLocked(gate, up, down, experts, x_dev, tokens, ids_dev, weights_dev, k,
                         gufo::MoeShared{}, y_dev);
}

int gufo_hip_moe_layer_dev(const gufo_hip_matrix* const* router_parts, int n_router_parts,
                           const gufo_hip_matrix* gate, const gufo_hip_matrix* up,
                           const gufo_hip_matrix* down, int experts, int k,
                           const float* x_dev, int tokens, const float* shared_dev,
                           float* y_dev) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  if (router_parts == nullptr || n_router_parts < 1 || n_router_parts > kMaxGemvParts) {
    return Fail(GUFO_HIP_ERR_LOGIC, "these projections have no router");
  }
  if (experts <= 0 || tokens < 0 || k <= 0 || k > experts) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "moe: experts %d, tokens %d, k %d", experts,
                tokens, k);
  }
  // The router stage yields one logit per expert, and one more - the shared expert's
  // gate, a tensor of its own - when the model has a shared expert
  // (src/models/qwen35/gguf_projections.cpp:127-131, decoder.cpp:537-539).
  size_t first_rows[kMaxGemvParts] = {0};
  size_t part_rows[kMaxGemvParts] = {0};
  size_t logits = 0;
  for (int p = 0; p < n_router_parts; ++p) {
    if (router_parts[p] == nullptr) {
      return Fail(GUFO_HIP_ERR_LOGIC, "these projections have no router");
    }
    part_rows[p] = router_parts[p]->rows;
    logits += part_rows[p];
  }
  const size_t needed = static_cast<size_t>(experts) + (shared_dev != nullptr ? 1 : 0);
  if (logits < needed || logits > static_cast<size_t>(experts) + 1) {
    return Fail(GUFO_HIP_ERR_SHAPE,
                "a router of %zu rows does not serve %d experts %s a shared expert", logits,
                experts, shared_dev != nullptr ? "and" : "without");
  }
  if (gate != nullptr && router_parts[0]->cols != gate->cols) {
    return Fail(GUFO_HIP_ERR_SHAPE, "router rows of %zu values, expert rows of %zu",
                router_parts[0]->cols, gate->cols);
  }
  if (tokens == 0) return GUFO_HIP_OK;
  const size_t n = static_cast<size_t>(tokens);
  const size_t logit_bytes = Align16(n * logits * sizeof(float));
  const size_t id_bytes = Align16(n * k * sizeof(int));
  GUFO_TRY(Reserve(&g_state.moe_route, logit_bytes + id_bytes + n * k * sizeof(float)));
  uint8_t* base = static_cast<uint8_t*>(g_state.moe_route.ptr);
  float* logit = reinterpret_cast<float*>(base);
  int* ids = reinterpret_cast<int*>(base + logit_bytes);
  float* weights = reinterpret_cast<float*>(base + logit_bytes + id_bytes);
  GUFO_TRY(GemvDevLocked(router_parts, first_rows, part_rows, n_router_parts,
                         gufo::GemvPrologue{}, x_dev, tokens, logit));
  GUFO_TRY(RouteDevLocked(logit, logits, tokens, experts, k, ids, weights));
  gufo::MoeShared shared;
  if (shared_dev != nullptr) {
    shared.rows = shared_dev;
    shared.gate_logit = logit + experts;
    shared.gate_stride = logits;
  }
  return MoeFfnDevLocked(gate, up, down, experts, x_dev, tokens, ids, weights, k, shared,
                         y_dev);
}

int gufo_hip_moe_ffn(const gufo_hip_matrix* gate, const gufo_hip_matrix* up,
                     const gufo_hip_matrix* down, int experts, const float* x_host,
                     int tokens, const int* ids_host, const float* weights_host, int k,
                     float* y_host) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  if (gate == nullptr) return Fail(GUFO_HIP_ERR_LOGIC, "these projections have no MoE experts");
  if (tokens < 0 || k <= 0) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "moe: tokens %d, k %d", tokens, k);
  }
  if (tokens == 0) return GUFO_HIP_OK;
  const size_t n = static_cast<size_t>(tokens) * k;
  const size_t hidden = gate->cols;
  for (size_t i = 0; i < n; ++i) {
    if (ids_host[i] < 0 || ids_host[i] >= experts) {
      return Fail(GUFO_HIP_ERR_LOGIC, "no such expert: %d", ids_host[i]);
    }
  }
  GUFO_TRY(CopyIn(&g_state.stage_x, x_host, tokens * hidden * sizeof(float)));
  GUFO_TRY(CopyIn(&g_state.stage_ids, ids_host, n * sizeof(int)));
  GUFO_TRY(CopyIn(&g_state.stage_weights, weights_host, n * sizeof(float)));
  GUFO_TRY(Reserve(&g_state.stage_y, tokens * hidden * sizeof(float)));
  GUFO_TRY(MoeFfnDevLocked(gate, up, down, experts,
                           static_cast<const float*>(g_state.stage_x.ptr), tokens,
                           static_cast<const int*>(g_state.stage_ids.ptr),
                           static_cast<const float*>(g_state.stage_weights.ptr), k,
                           gufo::MoeShared{}, static_cast<float*>(g_state.stage_y.ptr)));
  GUFO_TRY(CopyOut(y_host, g_state.stage_y.ptr, tokens * hidden * sizeof(float)));
  return CheckMoeIdsLocked();
}

namespace {

// The matrices of one stage (whole, sharing their input) against m rows of activations:
// c[t*stride + offset_p + r], stride = the sum of their rows - MatMul's layout with
// tokens = m (src/models/qwen35/gguf_projections.cpp:239-286).
int GemmPartsDevLocked(const gufo_hip_matrix* const* parts, int n_parts, const uint16_t* a,
                       size_t m, float* c, bool q4k_only) {
  if (parts == nullptr || n_parts < 1) {
    return Fail(GUFO_HIP_ERR_LOGIC, "no weights for this product");
  }
  size_t stride = 0;
  size_t own_weights = 0;
  for (int p = 0; p < n_parts; ++p) {
    const gufo_hip_matrix* w = parts[p];
    if (w == nullptr) return Fail(GUFO_HIP_ERR_LOGIC, "no weights for this product");
    if (q4k_only && w->type != GUFO_HIP_Q4_K) {
      return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT,
                  "this entry point takes Q4_K weights; this matrix has ggml type %d", w->type);
    }
    if (!gufo::GemmTakesType(w->type)) {
      return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT,
                  "the prefill GEMM takes Q4_K, Q5_K, Q6_K or Q8_0 weights; this matrix has "
                  "ggml type %d",
                  w->type);
    }
    if (w->cols != parts[0]->cols) {
      return Fail(GUFO_HIP_ERR_SHAPE, "part %d has rows of %zu values, part 0 of %zu", p,
                  w->cols, parts[0]->cols);
    }
    stride += w->rows;
    // A prepared matrix brings its fragments; otherwise the workspace holds them for the
    // duration of its product (one matrix after the other, so the largest decides).
    if (w->prefill_fragments == nullptr) {
      const size_t bytes = gufo::GemmWeightBytes(
          static_cast<uint32_t>(w->rows), static_cast<uint32_t>(w->cols / gufo::kSuperBlock));
      if (bytes > own_weights) own_weights = bytes;
    }
  }
  if (m == 0 || stride == 0) return GUFO_HIP_OK;
  if (a == nullptr || c == nullptr) return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "a or c is null");
  if (!Aligned16(a)) return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "a must be 16-byte aligned");
  const uint32_t nb = static_cast<uint32_t>(parts[0]->cols / gufo::kSuperBlock);
  if (m > (1ull << 24) || stride > 0xFFFFFFFFull) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "%zu tokens x %zu outputs exceed the launch limit",
                m, stride);
  }
  GUFO_TRY(Reserve(&g_state.gemm_work, gufo::GemmActivationBytes(m, nb) + own_weights));
  size_t offset = 0;
  bool converted = false;  // the activations are converted by the first launch
  for (int p = 0; p < n_parts; ++p) {
    const gufo_hip_matrix* w = parts[p];
    if (w->rows == 0) continue;
    GUFO_HIP_TRY(gufo::LaunchGemm(w->type, w->data, static_cast<uint32_t>(w->rows), nb,
                                  w->prefill_fragments, converted ? nullptr : a, m,
                                  g_state.gemm_work.ptr, c + offset,
                                  static_cast<uint32_t>(stride), g_state.stream));
    converted = true;
    offset += w->rows;
  }
  return GUFO_HIP_OK;
}

int GemmDevLocked(const gufo_hip_matrix* w, const uint16_t* a, size_t m, float* c,
                  bool q4k_only) {
  return GemmPartsDevLocked(&w, 1, a, m, c, q4k_only);
}

int GemmHostLocked(const gufo_hip_matrix* w, const uint16_t* a_bf16_host, size_t m,
                   float* c_host, bool q4k_only) {
  if (w == nullptr) return Fail(GUFO_HIP_ERR_LOGIC, "no weights for this product");
  if (m == 0 || w->rows == 0) return GUFO_HIP_OK;
  if (a_bf16_host == nullptr || c_host == nullptr) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "a or c is null");
  }
  const size_t a_bytes = m * w->cols * sizeof(uint16_t);
  const size_t c_bytes = m * w->rows * sizeof(float);
  GUFO_TRY(CopyIn(&g_state.stage_x, a_bf16_host, a_bytes));
  GUFO_TRY(Reserve(&g_state.stage_c, c_bytes));
  GUFO_TRY(GemmDevLocked(w, static_cast<const uint16_t*>(g_state.stage_x.ptr), m,
                         static_cast<float*>(g_state.stage_c.ptr), q4k_only));
  return CopyOut(c_host, g_state.stage_c.ptr, c_bytes);
}

}  // namespace

int gufo_hip_gemm_bf16_dev(const gufo_hip_matrix* w, const uint16_t* a_bf16_dev, size_t m,
                           float* c_dev) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  return GemmDevLocked(w, a_bf16_dev, m, c_dev, false);
}

int gufo_hip_gemm_bf16_parts_dev(const gufo_hip_matrix* const* parts, int n_parts,
                                 const uint16_t* a_bf16_dev, size_t m, float* c_dev) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  return GemmPartsDevLocked(parts, n_parts, a_bf16_dev, m, c_dev, false);
}

int gufo_hip_gemm_bf16(const gufo_hip_matrix* w, const uint16_t* a_bf16_host, size_t m,
                       float* c_host) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  return GemmHostLocked(w, a_bf16_host, m, c_host, false);
}

int gufo_hip_gemm_q4k_bf16_dev(const gufo_hip_matrix* w, const uint16_t* a_bf16_dev,
                               size_t m, float* c_dev) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  return GemmDevLocked(w, a_bf16_dev, m, c_dev, true);
}

int gufo_hip_gemm_q4k_bf16(const gufo_hip_matrix* w, const uint16_t* a_bf16_host, size_t m,
                           float* c_host) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  return GemmHostLocked(w, a_bf16_host, m, c_host, true);
}

int gufo_hip_capture_begin(void) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  if (g_state.capturing) return Fail(GUFO_HIP_ERR_LOGIC, "already recording");
  GUFO_HIP_TRY(hipStreamBeginCapture(g_state.stream, hipStreamCaptureModeThreadLocal));
  g_state.capturing = true;
  return GUFO_HIP_OK;
}

int gufo_hip_capture_end(gufo_hip_graph** out) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  if (out == nullptr) return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "null out pointer");
  *out = nullptr;
  if (!g_state.capturing) return Fail(GUFO_HIP_ERR_LOGIC, "not recording");
  g_state.capturing = false;
  hipGraph_t graph = nullptr;
  GUFO_HIP_TRY(hipStreamEndCapture(g_state.stream, &graph));
  hipGraphExec_t exec = nullptr;
  const hipError_t status = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  if (status != hipSuccess) {
    (void)hipGraphDestroy(graph);
    return Fail(GUFO_HIP_ERR_RUNTIME, "hipGraphInstantiate: %s", hipGetErrorString(status));
  }
  gufo_hip_graph* g = new (std::nothrow) gufo_hip_graph;
  if (g == nullptr) {
    (void)hipGraphExecDestroy(exec);
    (void)hipGraphDestroy(graph);
    return Fail(GUFO_HIP_ERR_OUT_OF_MEMORY, "host allocation failed");
  }
  g->graph = graph;
  g->exec = exec;
  *out = g;
  return GUFO_HIP_OK;
}

int gufo_hip_graph_launch(gufo_hip_graph* graph) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  if (graph == nullptr) return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "null graph");
  if (g_state.capturing) return Fail(GUFO_HIP_ERR_LOGIC, "a graph cannot be launched while recording");
  GUFO_HIP_TRY(hipGraphLaunch(graph->exec, g_state.stream));
  return GUFO_HIP_OK;
}

int gufo_hip_graph_destroy(gufo_hip_graph* graph) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  if (graph == nullptr) return GUFO_HIP_OK;
  GUFO_TRY(RequireReady());
  GUFO_HIP_TRY(hipStreamSynchronize(g_state.stream));
  (void)hipGraphExecDestroy(graph->exec);
  (void)hipGraphDestroy(graph->graph);
  delete graph;
  return GUFO_HIP_OK;
}

int gufo_hip_timer_begin(void) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  GUFO_HIP_TRY(hipEventRecord(g_state.timer_begin, g_state.stream));
  return GUFO_HIP_OK;
}

int gufo_hip_timer_end(float* milliseconds) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  if (milliseconds == nullptr) return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "null out pointer");
  GUFO_HIP_TRY(hipEventRecord(g_state.timer_end, g_state.stream));
  GUFO_HIP_TRY(hipEventSynchronize(g_state.timer_end));
  GUFO_HIP_TRY(hipEventElapsedTime(milliseconds, g_state.timer_begin, g_state.timer_end));
  return GUFO_HIP_OK;
}

int gufo_hip_read_probe_dev(const void* src_dev, size_t bytes, uint32_t* sink_dev) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  if (src_dev == nullptr || sink_dev == nullptr || !Aligned16(src_dev)) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "read probe: null or unaligned buffer");
  }
  GUFO_HIP_TRY(gufo::LaunchReadProbe(src_dev, bytes, sink_dev, g_state.stream));
  return GUFO_HIP_OK;
}

int gufo_hip_write_probe_dev(void* dst_dev, size_t bytes) {
  const std::lock_guard<std::mutex> lock(g_state.mutex);
  GUFO_TRY(RequireReady());
  if (dst_dev == nullptr || !Aligned16(dst_dev)) {
    return Fail(GUFO_HIP_ERR_INVALID_ARGUMENT, "write probe: null or unaligned buffer");
  }
  GUFO_HIP_TRY(gufo::LaunchWriteProbe(dst_dev, bytes, g_state.stream));
  return GUFO_HIP_OK;
}

}  // extern "C"
