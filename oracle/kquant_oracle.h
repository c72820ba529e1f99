/*
 * TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * CPU restatement of the reference's GGUF K-quant matrix-vector path, used as the
 * checker for the HIP kernels and as the timed CPU baseline. Only tests, the smoke
 * check and the bench's cpu_baseline leg may link or load it; the shipped library
 * never does.
 *
 * Every function names the reference source it restates (paths under the
 * reference's src/).  Pinning status of each function (what, other than a retyped
 * formula, fixes its output):
 *   half_to_float      fp16 known-answer table of tests/core/quant_test.cpp:51-70,
 *                      exhaustive comparison of all 65,536 inputs with numpy float16
 *   dequantize         bit-exact against the gguf-py fixtures Q4_K/Q5_K/Q6_K/Q8_0
 *                      .{bin,f32} (tests/fixtures/quant) and against the compiled
 *                      reference; F32 is a copy
 *   scale_min_k4       round trip through the packer's inverse over all 64x64 values
 *   dot_q4_k/q5_k/q6_k, dot_q8_0, dot_f32
 *                      closed form: dequantize + double sum, limit 2e-5 of sum|w x|
 *                      (tests/models/qwen35/gguf_dot_test.cpp:116); compiled reference
 *   matmul             "each output is one dot product": equality with single dots at
 *                      the documented index t*stride+offset+r; compiled reference
 *   route              brute-force stable sort on small inputs, engineered ties,
 *                      floor case; compiled reference Route
 *   moe_group/moe_ffn  grouped result equals the per-token ungrouped result
 *   argmax             first maximum wins (std::max_element semantics)
 *   rms_norm/res_norm  closed form in double (x / sqrt(mean x^2 + eps) * w); constant
 *                      rows, whose norm is sign(c) / sqrt(1 + eps / c^2); invariance to
 *                      scaling the row by a power of two when eps = 0; compiled
 *                      reference vec::RmsNorm
 *   swiglu             closed form in double; silu(0) = 0, silu(x) -> x for large x,
 *                      silu(-x) = silu(x) - x
 */
#ifndef GUFO_KQUANT_ORACLE_H_
#define GUFO_KQUANT_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ggml type ids (core/gguf.hpp:16-24). */
enum {
  GUFO_ORACLE_F32 = 0,
  GUFO_ORACLE_Q8_0 = 8,
  GUFO_ORACLE_Q4_K = 12,
  GUFO_ORACLE_Q5_K = 13,
  GUFO_ORACLE_Q6_K = 14
};

/* core/quant.cpp:129-155 */
float gufo_oracle_half_to_float(uint16_t h);
/* core/quant.cpp:202-219; 0 for a type this path does not cover */
size_t gufo_oracle_block_bytes(int type);
/* core/quant.cpp:186-200; 0 for a type this path does not cover */
size_t gufo_oracle_block_elements(int type);
/* core/quant.cpp:221-227; 0 when n is not a whole number of blocks */
size_t gufo_oracle_row_bytes(int type, size_t n);
/* core/quant.cpp:158-167 */
void gufo_oracle_scale_min_k4(size_t j, const uint8_t* packed, uint8_t* scale,
                              uint8_t* min);
/* core/quant.cpp:33-125,229-263; returns 0, or -1 on unknown type / partial block */
int gufo_oracle_dequantize(int type, const uint8_t* src, float* dst, size_t n);

/* models/qwen35/gguf_dot.hpp:156-182 (portable body of DotK4<false>) */
float gufo_oracle_dot_q4_k(const uint8_t* row, const float* x, size_t n);
/* models/qwen35/gguf_dot.hpp:156-182 (portable body of DotK4<true>) */
float gufo_oracle_dot_q5_k(const uint8_t* row, const float* x, size_t n);
/* models/qwen35/gguf_dot.hpp:260-289 (portable body of DotQ6_K) */
float gufo_oracle_dot_q6_k(const uint8_t* row, const float* x, size_t n);
/* models/qwen35/gguf_dot.hpp:62-74 (portable body of DotQ8_0) */
float gufo_oracle_dot_q8_0(const uint8_t* row, const float* x, size_t n);
/* core/vec.hpp:36-51 (portable body of vec::Dot, which DotF32 calls,
 * models/qwen35/gguf_dot.hpp:71-75) */
float gufo_oracle_dot_f32(const uint8_t* row, const float* x, size_t n);
/* dequantize then sum in double: GgufProjections' kDouble path,
 * models/qwen35/gguf_projections.cpp:48-54,277-282 */
double gufo_oracle_dot_double(int type, const uint8_t* row, const float* x,
                              size_t n);

/*
 * models/qwen35/gguf_projections.cpp:239-286 (GgufProjections::MatMul).
 * y[t*stride + offset_p + r] = dot(row first[p]+r of part p, x + t*in), where
 * stride = sum of rows[] and offset_p = rows of the parts before p.
 * precision 0 = fused fp32 dots (Precision::kFloat), 1 = dequantize + double
 * (Precision::kDouble).  threads <= 1 runs on the caller.  Returns 0, -1 on a
 * bad argument.
 */
int gufo_oracle_matmul(int n_parts, const uint8_t* const* data, const int* types,
                       const size_t* first, const size_t* rows, size_t in,
                       const float* x, int tokens, float* y, int precision,
                       int threads);

/* models/qwen35/moe.cpp:16-42 (Route) */
void gufo_oracle_route(const float* logits, int experts, int k, int* chosen,
                       float* weights);
/* core/sampling.cpp:327-329: std::max_element, first maximum wins */
int64_t gufo_oracle_argmax(const float* v, size_t n);

/*
 * Grouping tables of models/qwen35/reference.cpp:562-565: for each expert the
 * ascending list of pair ids (t*k+slot) that chose it.
 *   counts[experts], offsets[experts+1], pairs[tokens*k] (pair ids, grouped by
 *   expert ascending, ascending within an expert).  Returns distinct experts.
 */
int gufo_oracle_moe_group(const int* chosen, int tokens, int k, int experts,
                          int* counts, int* offsets, int* pairs);

/*
 * models/qwen35/reference.cpp:514-607 (Reference::Ffn) for the routed experts
 * only (no dense/shared expert): route each token, apply each chosen expert once
 * over the tokens that chose it ([gate|up] -> silu(gate)*up -> down), then the
 * weighted sum in slot order accumulated in double.
 *   gate, up: [experts*ffn rows x hidden], down: [experts*hidden rows x ffn].
 *   logits: tokens x experts.  x: tokens x hidden.  y: tokens x hidden.
 *   chosen/weights (tokens x k) are outputs.  precision as in matmul.
 */
int gufo_oracle_moe_ffn(const uint8_t* gate, int gate_type, const uint8_t* up,
                        int up_type, const uint8_t* down, int down_type,
                        int experts, int hidden, int ffn, const float* logits,
                        const float* x, int tokens, int k, int* chosen,
                        float* weights, float* y, int precision, int threads);

/* core/simd.hpp:82-84 (Silu) */
float gufo_oracle_silu(float x);

/* core/vec.hpp:56-63: out[i] = x[i] * inv * w[i], inv = 1 / sqrt(Dot(x,x)/n + eps), all
 * fp32, Dot in the order of its portable branch (vec.hpp:36-51): eight partial sums by
 * index mod 8, added in order, then the tail.  out may alias x. */
void gufo_oracle_rms_norm(const float* x, const float* w, size_t n, float eps,
                          float* out);

/* The residual add that ends a half layer and the norm that opens the next
 * (models/qwen35/decoder.cpp:504-509): residual = x + delta (delta NULL: x),
 * normed = RmsNorm(residual) * w.  residual may be NULL. */
void gufo_oracle_res_norm(const float* x, const float* delta, const float* w, size_t n,
                          float eps, float* residual, float* normed);

/* The activation between the two products of the dense feed-forward block
 * (models/qwen35/decoder.cpp:511-514 with Silu of :28-33, x * (1 / (1 + e^-x))):
 * act[i] = silu(gate_up[i]) * gate_up[f + i], i < f. */
void gufo_oracle_swiglu(const float* gate_up, size_t f, float* act);

#ifdef __cplusplus
}
#endif
#endif /* GUFO_KQUANT_ORACLE_H_ */
