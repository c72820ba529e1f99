// Internal interface between the C-ABI layer (capi.hip) and the kernel files.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace gufo {

constexpr int kMaxGemvParts = 8;   // row ranges per launch
constexpr int kMaxGemvTokens = 4;  // token columns per pass over the weights

// One row range of a launch: `rows` points at the first byte of its first row.
struct GemvPart {
  const uint8_t* rows;
  uint32_t n_rows;
  uint32_t y_offset;  // column of the range's first output within a y row
};

struct GemvLaunch {
  GemvPart part[kMaxGemvParts];
  uint32_t n_parts;
  uint32_t total_rows;      // sum of n_rows
  uint32_t blocks_per_row;  // cols / 256
  uint32_t y_stride;        // floats between token rows of y
};

// LDS a product kernel may use: the whole LDS of a gfx950 compute unit.
constexpr size_t kGemvMaxLdsBytes = 160 * 1024;

// The compute-unit count of the device, which sizes the persistent launches.
void SetGemvComputeUnits(int compute_units);
int DeviceComputeUnits();

// Token columns one launch can carry for rows of blocks_per_row super-blocks: the
// quantized activation rows of all columns must fit in LDS together (at most
// kMaxGemvTokens).
int GemvMaxTokens(int type, uint32_t blocks_per_row);

// y[t*y_stride + part.y_offset + r] = row r of part . x[t*cols ...], t < tokens.
// All parts are of `type`.  tokens in 1..GemvMaxTokens(type, blocks_per_row).
hipError_t LaunchGemv(int type, const GemvLaunch& launch, const float* x, int tokens,
                      float* y, hipStream_t stream);

// What a dense product does to its activation rows before multiplying: the elementwise
// steps the reference's decoder runs between its products
// (src/models/qwen35/decoder.cpp:493-521), and its NPU GEMV fuses as input stages
// (src/npu/gemv.hpp:58-63).
constexpr int kProloguePlain = 0;    // x[t] as given
constexpr int kPrologueSwiGlu = 1;   // x[t] holds [gate | up] (2*cols): silu(gate) * up
constexpr int kPrologueResNorm = 2;  // RmsNorm(x[t] + delta[t]) * norm_weight
struct GemvPrologue {
  int kind = kProloguePlain;
  // kPrologueResNorm only; token rows are cols floats apart.
  const float* delta = nullptr;        // added to x before the norm, or null
  const float* norm_weight = nullptr;  // cols
  float eps = 0.0f;
  float* residual_out = nullptr;  // <- x + delta, or null
  float* normed_out = nullptr;    // <- the normalized rows, or null
};

// LaunchGemv with a prologue.  K-quant and Q8_0 rows; fp32 rows take kProloguePlain only.
// The outputs of kPrologueResNorm must not overlap x, delta or each other: other
// workgroups are still reading those rows when workgroup 0 stores.
hipError_t LaunchGemvFused(int type, const GemvLaunch& launch, const GemvPrologue& in,
                           const float* x, int tokens, float* y, hipStream_t stream);

// The greedy pick taken inside the product: instead of storing y, every workgroup keeps
// the best (value, position) of the outputs it forms per token, and a one-workgroup-per-
// token kernel behind it takes the best of those - the head's logits never reach memory
// (the draft head of the reference's NPU decoder feeds std::max_element the same way,
// src/models/qwen36_35b_a3b/npu_decoder.cpp:968-973).
struct GemvPick {
  void* partial = nullptr;   // GemvPickPartialBytes(tokens) bytes
  int64_t* index = nullptr;  // tokens results: position of the first maximum of y[t]
  float* value = nullptr;    // tokens maxima, or null
};
size_t GemvPickPartialBytes(int tokens);
// One product launch only: K-quant or Q8_0 rows, tokens within GemvMaxTokens.
hipError_t LaunchGemvPick(int type, const GemvLaunch& launch, const GemvPrologue& in,
                          const float* x, int tokens, const GemvPick& pick,
                          hipStream_t stream);

// The same for rows stored as fp32 (LaunchGemv forwards type 0 here).
hipError_t LaunchGemvF32(const GemvLaunch& launch, const float* x, int tokens, float* y,
                         hipStream_t stream);

// ---- mixture of experts ------------------------------------------------------

// One routed expert and up to four of the (token, slot) pairs that chose it.
// pair = token * k + slot.
struct MoeSegment {
  int32_t expert;
  int32_t n_pairs;
  int32_t pair[kMaxGemvTokens];
};

// Written by the grouping kernel, read by the expert kernels.
struct MoeTables {
  int32_t n_segments;
  int32_t n_distinct;  // experts chosen by at least one pair
  int32_t n_invalid;   // pairs whose expert id is out of range (dropped)
  int32_t pad;
};

struct MoeGemvArgs {
  const MoeTables* tables;
  const MoeSegment* segments;
  const float* x;       // activation rows
  size_t x_row_floats;  // floats between activation rows
  float* y;             // output rows, one per pair, y_stride floats apart
  uint32_t k;           // slots per token
  size_t expert_bytes;  // bytes between experts, the same for every part of a launch
  // One-token calls need no grouping: with direct_ids set, segment s is slot s alone,
  // its expert direct_ids[s] (skipped when not below `experts`), and tables / segments
  // are not read.
  const int32_t* direct_ids;
  int32_t experts;
};

// As LaunchGemv, once per segment: part p's rows start at
// part[p].rows + segment.expert * expert_bytes.  max_pairs bounds the pairs of a
// segment (the call's token count, at most kMaxGemvTokens).  swiglu = false: column t reads
// x row (pair / k); swiglu = true: column t reads the pair's own row of 2*cols
// values [gate | up] and the product is taken with silu(gate) * up.
hipError_t LaunchMoeGemv(int type, const GemvLaunch& launch, const MoeGemvArgs& moe,
                         bool swiglu, uint32_t max_segments, int max_pairs,
                         hipStream_t stream);

// Softmax (double) top-k routing of `tokens` rows of `experts` logits, the rows
// logit_stride floats apart (a router with a shared-expert gate yields experts + 1).
constexpr int kMaxRouteExperts = 1024;
constexpr int kMaxRouteK = 64;
hipError_t LaunchRoute(const float* logits, size_t logit_stride, int tokens, int experts, int k,
                       int* ids, float* weights, hipStream_t stream);

// The shared expert's contribution to a combine: its output rows (tokens x hidden; null:
// none) and each token's gate logit (gate_stride floats apart).
struct MoeShared {
  const float* rows = nullptr;
  const float* gate_logit = nullptr;
  size_t gate_stride = 0;
};

// Groups the n_pairs = tokens*k pairs by expert: counts[experts],
// offsets[experts+1], pairs[n_pairs] (ascending pair id within an expert),
// pair_valid[n_pairs], the segment list (at most n_pairs entries, `capacity` pairs
// each at most) and *tables.
constexpr int kMaxGroupExperts = 1024;
constexpr int kMaxGroupPairs = 8192;
hipError_t LaunchMoeGroup(const int* ids, int n_pairs, int experts, int capacity,
                          int* counts, int* offsets, int* pairs, uint8_t* pair_valid,
                          MoeSegment* segments, MoeTables* tables, hipStream_t stream);

// The same pair_valid, segment list and *tables for a call of at most
// kMaxSmallGroupPairs pairs, without the per-expert tables: what the expert kernels
// read, in one wave.
constexpr int kMaxSmallGroupPairs = 64;
hipError_t LaunchMoeGroupSmall(const int* ids, int n_pairs, int experts, int capacity,
                               uint8_t* pair_valid, MoeSegment* segments, MoeTables* tables,
                               hipStream_t stream);

// y[t][i] = sum over slots in order of weights[t*k+slot] * rows[(t*k+slot)][i],
// accumulated in double; invalid pairs are skipped.  With shared.rows the sum starts from
// shared.rows[t][i] * sigmoid(gate logit of t); y may then be shared.rows itself.
hipError_t LaunchMoeCombine(const float* rows, const float* weights,
                            const uint8_t* pair_valid, int tokens, int k, int hidden,
                            const MoeShared& shared, float* y, hipStream_t stream);

// The same for one token whose pairs were not grouped: a slot is valid when its id is
// below `experts`; also fills *tables from the ids (what the grouping kernel would have
// written), so that out-of-range ids are reported as after a grouped call.
hipError_t LaunchMoeCombineDirect(const float* rows, const float* weights, const int32_t* ids,
                                  int experts, int k, int hidden, const MoeShared& shared,
                                  float* y, MoeTables* tables, hipStream_t stream);

// ---- prefill ------------------------------------------------------------------

// Both operands of the prefill product as fp16: bytes of the activations of `tokens`
// rows, and of a matrix's weights as matrix-instruction fragments.
size_t GemmActivationBytes(size_t tokens, uint32_t blocks_per_row);
size_t GemmWeightBytes(uint32_t rows, uint32_t blocks_per_row);

// Row types LaunchGemm takes: Q4_K, Q5_K, Q6_K, Q8_0.
bool GemmTakesType(int type);

// The weights of w as fragments (GemmWeightBytes), once, for every product that follows.
hipError_t LaunchGemmPrepareWeights(int type, const uint8_t* w, uint32_t rows,
                                    uint32_t blocks_per_row, void* fragments,
                                    hipStream_t stream);

// c[t*c_stride + r] = row r of the matrix w (rows of `type`) . a[t], a given as bf16
// (tokens x blocks_per_row*256), on the matrix cores with fp32 accumulation.
// `fragments`: what LaunchGemmPrepareWeights wrote for w, or null; `workspace` holds
// GemmActivationBytes, plus GemmWeightBytes when fragments is null.  A null a_bf16 means
// the workspace still holds the converted activations of the call before (the next
// matrix of a stage, which shares its input).
hipError_t LaunchGemm(int type, const uint8_t* w, uint32_t rows, uint32_t blocks_per_row,
                      const void* fragments, const uint16_t* a_bf16, size_t tokens,
                      void* workspace, float* c, uint32_t c_stride, hipStream_t stream);

// index of the first maximum of v[0..n) -> *out (device); scratch holds
// 2*kArgmaxBlocks entries of 8 bytes.
constexpr int kArgmaxBlocks = 1024;
hipError_t LaunchArgmax(const float* v, size_t n, void* scratch, int64_t* out,
                        hipStream_t stream);

// Streaming read of `bytes` (multiple of 16); *sink is written only if a lane's
// xor of its dwords equals a magic constant, which keeps the loads alive.
hipError_t LaunchReadProbe(const void* src, size_t bytes, uint32_t* sink,
                           hipStream_t stream);

// Streaming write of `bytes` (multiple of 16) of a constant.
hipError_t LaunchWriteProbe(void* dst, size_t bytes, hipStream_t stream);

}  // namespace gufo
