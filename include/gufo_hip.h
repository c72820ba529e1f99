/*
 * gufo_hip.h - C-ABI of the MI355X (gfx950) backend for gufo-npu's quantized
 * matrix-vector decode path.
 *
 * The library replaces, for this one path, what the reference engine reaches
 * through `qwen35::Projections` (src/models/qwen35/projections.hpp:45-59): its CPU
 * backend `GgufProjections` (src/models/qwen35/gguf_projections.cpp:179-286) and
 * the NPU operator `npu::Q4nxGemv` (src/npu/gemv.hpp:134-158).  Weights are GGUF
 * K-quant blocks exactly as a GGUF file stores them (row-major, Q4_K 144 B,
 * Q5_K 176 B, Q6_K 210 B per 256 values); they are copied to HBM once and stay
 * resident, like the NPU backend keeps its matrices on the device.
 *
 * Conventions
 *   - Every entry point returns a gufo_hip_status (0 = ok) and never throws.
 *     gufo_hip_last_error() gives the message of the calling thread's last
 *     failure.  The C++ adapter (gufo-npu_amd/host/hip_projections.hpp) maps the
 *     codes back to the exception types the reference throws.
 *   - Entry points may be called from several host threads; calls are serialised
 *     on one HIP stream, as GgufProjections serialises products on its pool
 *     (gguf_projections.hpp:14-16).
 *   - "_dev" variants take device pointers, enqueue on the library's stream and
 *     return without waiting; gufo_hip_synchronize() waits.  The others take host
 *     pointers and return when y is complete.
 *   - x is `tokens` rows of `cols` fp32; y is `tokens` rows of fp32, a row being
 *     the parts' outputs concatenated (projections.hpp:8-11).
 */
#ifndef GUFO_HIP_H_
#define GUFO_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ggml tensor type ids, numerically as in GGUF (src/core/gguf.hpp:16-24): the five
 * row types GgufProjections multiplies (gguf_projections.cpp:58-75).  F32 and Q8_0
 * rows (routers, gates, a few projections of real files) go through the dense
 * products only; expert tensors and the prefill GEMM take K-quants. */
enum gufo_hip_type {
  GUFO_HIP_F32 = 0,
  GUFO_HIP_Q8_0 = 8,
  GUFO_HIP_Q4_K = 12,
  GUFO_HIP_Q5_K = 13,
  GUFO_HIP_Q6_K = 14
};

/* Status codes.  The exception each one stands for in the reference:
 *   INVALID_ARGUMENT  std::invalid_argument  partial block, unknown type
 *                     (src/core/quant.cpp:199,224,233)
 *   SHAPE             std::runtime_error     tensor shape mismatch
 *                     (src/models/qwen35/gguf_projections.cpp:43)
 *   LOGIC             std::logic_error       no weights for a stage, no such
 *                     expert (gguf_projections.cpp:214,223,235)
 *   NO_DEVICE         std::runtime_error     backend not available
 *                     (src/npu/gemv_stub.cpp:8-10)
 *   OUT_OF_RANGE      std::out_of_range      token / index out of range
 *                     (src/models/qwen35/decoder.cpp:484)
 */
enum gufo_hip_status {
  GUFO_HIP_OK = 0,
  GUFO_HIP_ERR_NO_DEVICE = 1,
  GUFO_HIP_ERR_NOT_INITIALIZED = 2,
  GUFO_HIP_ERR_INVALID_ARGUMENT = 3,
  GUFO_HIP_ERR_SHAPE = 4,
  GUFO_HIP_ERR_LOGIC = 5,
  GUFO_HIP_ERR_OUT_OF_RANGE = 6,
  GUFO_HIP_ERR_OUT_OF_MEMORY = 7,
  GUFO_HIP_ERR_RUNTIME = 8
};

/* A K-quant matrix resident in HBM.  Replaces gguf::TensorInfo + its mapped data
 * (src/core/gguf.hpp:40-54) as GgufProjections::Rows refers to it
 * (gguf_projections.hpp:41-45). */
typedef struct gufo_hip_matrix gufo_hip_matrix;

/* ---- life cycle ---------------------------------------------------------- */

/* Selects HIP device `device`, checks that it is a gfx950 part, creates the
 * library's stream.  Fails with NO_DEVICE where the reference's stub backend
 * throws at construction (src/npu/gemv_stub.cpp:8-10).  Idempotent. */
int gufo_hip_init(int device);
/* Frees the stream and library-owned scratch.  Matrices must be destroyed first. */
int gufo_hip_shutdown(void);
/* Message of the calling thread's last failing call ("" if none). */
const char* gufo_hip_last_error(void);
/* Device name ("gfx950...") and compute-unit count of the initialised device. */
int gufo_hip_device_info(char* name, size_t name_bytes, int* compute_units);

/* ---- block geometry: quant::BlockBytes / RowBytes (src/core/quant.cpp:202-227) */

/* Bytes of one block of the format (144 / 176 / 210 for the 256-value K-quant
 * super-blocks, 34 for Q8_0's 32 values, 4 for F32); 0 for a type this backend does
 * not take. */
size_t gufo_hip_block_bytes(int ggml_type);
/* Bytes of a row of `cols` values; 0 when cols is not a multiple of 256 (where
 * RowBytes throws std::invalid_argument for a partial block).  This backend walks
 * every row in steps of 256 values, so Q8_0 and F32 rows must be a multiple of 256
 * long too, which is stricter than the reference's 32 and 1. */
size_t gufo_hip_row_bytes(int ggml_type, size_t cols);

/* ---- device memory for callers that keep x / y resident ------------------- */
/* The NPU backend's npu::Buffer (src/npu/gemv.hpp:82-131) in four calls. */

int gufo_hip_malloc(void** device_ptr, size_t bytes);
int gufo_hip_free(void* device_ptr);
int gufo_hip_memcpy_h2d(void* device_dst, const void* host_src, size_t bytes);
int gufo_hip_memcpy_d2h(void* host_dst, const void* device_src, size_t bytes);
/* Waits for everything enqueued on the library's stream. */
int gufo_hip_synchronize(void);

/* ---- matrices ------------------------------------------------------------- */

/* Copies `rows` rows of `cols` values of GGUF blocks (row-major, as stored in the
 * file: row r starts at r * row_bytes, gguf_projections.cpp:262,269) to HBM.
 * A 3-D expert tensor [cols, rows_per_expert, experts] is passed with
 * rows = rows_per_expert * experts; expert e is the row range
 * [e*rows_per_expert, (e+1)*rows_per_expert) (gguf_projections.cpp:230-233).
 * The host bytes may be freed on return. */
int gufo_hip_matrix_create(int ggml_type, const void* host_blocks, size_t rows,
                           size_t cols, gufo_hip_matrix** out);
int gufo_hip_matrix_destroy(gufo_hip_matrix* m);
int gufo_hip_matrix_info(const gufo_hip_matrix* m, int* ggml_type, size_t* rows,
                         size_t* cols, size_t* bytes);

/* ---- the matrix-vector products ------------------------------------------- */

/* GgufProjections::MatMul (gguf_projections.cpp:239-286):
 *   y[t*stride + offset_p + r] = row (first_row[p] + r) of parts[p] . x[t]
 * for r < n_rows[p], t < tokens, with stride = sum of n_rows and offset_p the rows
 * of the parts before p.  All parts share `cols`.  Any tokens >= 0 is accepted;
 * the GEMV kernels carry up to four token columns per pass over the weights.
 * Column t of a multi-token call is bit-identical to a one-token call on x[t]. */
int gufo_hip_gemv(const gufo_hip_matrix* const* parts, const size_t* first_row,
                  const size_t* n_rows, int n_parts, const float* x_host,
                  int tokens, float* y_host);
int gufo_hip_gemv_dev(const gufo_hip_matrix* const* parts, const size_t* first_row,
                      const size_t* n_rows, int n_parts, const float* x_dev,
                      int tokens, float* y_dev);

/* What a product does to its activation rows before multiplying: the elementwise
 * steps Decoder::Step runs on the host between its products
 * (src/models/qwen35/decoder.cpp:493-521), taken into the product's own kernel the way
 * the reference's NPU GEMV takes them as input stages (Prologue,
 * src/npu/gemv.hpp:58-63), so that a decoder layer is four launches with nothing
 * between them.
 *   PLAIN    x[t] as given (cols values).
 *   SWIGLU   x[t] holds [gate | up], 2*cols values, e.g. the y row of the product
 *            before; the activation is silu(gate[i]) * up[i]
 *            (decoder.cpp:511-514, Silu at :28-33; here x / (1 + exp(-x)) in fp32).
 *   RESNORM  the activation is RmsNorm(x[t] + delta[t]) * norm_weight, with
 *            RmsNorm(v)[i] = v[i] * (1 / sqrt(mean(v^2) + eps)) * w[i] in fp32
 *            (src/core/vec.hpp:56-63): the residual add that ends one half of a layer
 *            (decoder.cpp:504-506,519-521) and the norm that opens the next (:493,508).
 *            delta_dev may be NULL (the first layer has nothing to add).  If not NULL,
 *            residual_out_dev receives x + delta (the new residual stream) and
 *            normed_out_dev the normalized rows (for the router and the experts of a
 *            mixture layer, which read the same input); token rows of all four are
 *            cols floats apart, 16-byte aligned, and the two outputs must not overlap
 *            x, delta, the weight, y or each other.
 * Rows of fp32 matrices take PLAIN only.  Column t of a multi-token call stays
 * bit-identical to a one-token call on the same row with every prologue. */
enum gufo_hip_prologue_kind {
  GUFO_HIP_PROLOGUE_PLAIN = 0,
  GUFO_HIP_PROLOGUE_SWIGLU = 1,
  GUFO_HIP_PROLOGUE_RESNORM = 2
};
typedef struct gufo_hip_prologue {
  int kind;
  const float* delta_dev;       /* RESNORM: tokens x cols, or NULL */
  const float* norm_weight_dev; /* RESNORM: cols */
  float eps;                    /* RESNORM: Config::rms_eps */
  float* residual_out_dev;      /* RESNORM: tokens x cols, or NULL */
  float* normed_out_dev;        /* RESNORM: tokens x cols, or NULL */
} gufo_hip_prologue;
/* gufo_hip_gemv_dev with a prologue (NULL: PLAIN). */
int gufo_hip_gemv_fused_dev(const gufo_hip_matrix* const* parts, const size_t* first_row,
                            const size_t* n_rows, int n_parts,
                            const gufo_hip_prologue* prologue, const float* x_dev,
                            int tokens, float* y_dev);

/* The product with the greedy pick inside: index_dev[t] = position, within the
 * concatenated output row, of the first maximum of y[t] (std::max_element's rule,
 * src/core/sampling.cpp:327-329); y itself is never stored.  This is how the reference's
 * NPU decoder reads its draft head (src/models/qwen36_35b_a3b/npu_decoder.cpp:968-973):
 * a head product whose only consumer is max_element.  PLAIN and RESNORM prologues
 * (RESNORM: the output norm in front of the head, decoder.cpp:525-526).  Enqueued only;
 * index_dev is device memory (tokens x int64).  The pick rides inside the product's
 * kernel (each workgroup keeps its best candidate; a small kernel behind it takes the
 * best of those) when the product is one launch (quantized rows of one type,
 * tokens <= 4); otherwise the product goes to library scratch and gufo_hip_argmax_dev's
 * kernels pick. */
int gufo_hip_gemv_argmax_dev(const gufo_hip_matrix* const* parts, const size_t* first_row,
                             const size_t* n_rows, int n_parts,
                             const gufo_hip_prologue* prologue, const float* x_dev,
                             int tokens, int64_t* index_dev);

/* A new matrix holding rows rows_host[0..n) of `src`, in that order: the draft
 * vocabulary's rows of the head (qwen35::DraftVocab, src/models/qwen35/draft_vocab.hpp:7-14;
 * q4nx::PackRows in npu_decoder.cpp:532-544).  A pick over it returns a position i; the
 * token is rows_host[i].  Rows out of range: OUT_OF_RANGE. */
int gufo_hip_matrix_gather_rows(const gufo_hip_matrix* src, const int64_t* rows_host,
                                size_t n, gufo_hip_matrix** out);

/* Greedy pick over logits, std::max_element's rule: the first maximum wins
 * (src/core/sampling.cpp:327-329).  `index` receives the position. */
int gufo_hip_argmax_dev(const float* logits_dev, size_t n, int64_t* index_host);

/* ---- mixture of experts ---------------------------------------------------- */

/* qwen35::Route (src/models/qwen35/moe.cpp:16-42) for `tokens` rows of `experts`
 * logits: softmax in double, the k most probable experts in order of probability
 * (ties to the lower index), weights renormalised with the sum floored at 2^-14.
 * ids and weights are tokens x k. */
int gufo_hip_route_topk(const float* logits_host, int tokens, int experts, int k,
                        int* ids_host, float* weights_host);
int gufo_hip_route_topk_dev(const float* logits_dev, int tokens, int experts, int k,
                            int* ids_dev, float* weights_dev);

/* The grouping of Reference::Ffn (src/models/qwen35/reference.cpp:562-565), done
 * on the device: for ids (tokens x k) writes counts[experts], offsets[experts+1]
 * and pairs[tokens*k] - the pair ids t*k+slot grouped by expert ascending and
 * ascending within an expert - and the number of distinct experts. */
int gufo_hip_moe_group(const int* ids_host, int tokens, int k, int experts,
                       int* counts_host, int* offsets_host, int* pairs_host,
                       int* distinct_host);

/* The routed part of Reference::Ffn / Decoder::MoeFfn (reference.cpp:562-606,
 * decoder.cpp:530-558): tokens are grouped by expert on the device, every distinct
 * expert's gate, up and down rows are streamed once over the tokens that chose it
 * ([gate|up] -> silu(gate)*up -> down), and
 *   y[t] = sum over slots, in slot order, of weights[t][slot] * down_out[t][slot]
 * accumulated in double as reference.cpp:595-606 does.
 * gate, up: experts*ffn rows x hidden; down: experts*hidden rows x ffn. */
int gufo_hip_moe_ffn(const gufo_hip_matrix* gate, const gufo_hip_matrix* up,
                     const gufo_hip_matrix* down, int experts, const float* x_host,
                     int tokens, const int* ids_host, const float* weights_host,
                     int k, float* y_host);
int gufo_hip_moe_ffn_dev(const gufo_hip_matrix* gate, const gufo_hip_matrix* up,
                         const gufo_hip_matrix* down, int experts,
                         const float* x_dev, int tokens, const int* ids_dev,
                         const float* weights_dev, int k, float* y_dev);

/* Decoder::MoeFfn whole, for device-resident callers (src/models/qwen35/decoder.cpp:530-558):
 * the router product (Stage::kRouter: the whole matrices router_parts[0..n), their
 * outputs side by side as the stage's parts are, gguf_projections.cpp:127-131), Route
 * over its first `experts` logits (moe.cpp:16-42), the k chosen experts of every token
 * and their weighted sum.  With shared_dev (tokens x hidden, the shared expert's output)
 * the router parts must have experts + 1 rows together, and the sum starts from
 * shared_dev[t] * SharedExpertScale(logit `experts` of token t) (moe.cpp:44-47: sigmoid
 * in double; decoder.cpp:539-542).  y_dev may be shared_dev.  Five to seven launches,
 * all recordable. */
int gufo_hip_moe_layer_dev(const gufo_hip_matrix* const* router_parts, int n_router_parts,
                           const gufo_hip_matrix* gate, const gufo_hip_matrix* up,
                           const gufo_hip_matrix* down, int experts, int k,
                           const float* x_dev, int tokens, const float* shared_dev,
                           float* y_dev);

/* ---- prefill --------------------------------------------------------------- */

/* MatMul with many tokens, the prefill shape (gguf_projections.cpp:239-286 with
 * tokens = m; NPU analogue src/npu/gemm.hpp:99-105):
 *   c[t*rows + r] = row r of w . a[t],  a given as bf16 (m x cols, row-major),
 * computed on the matrix cores with fp32 accumulation: both operands are converted to
 * fp16 once per call (each weight rounded once; activations beyond +-65504 saturate).
 * w is Q4_K, Q5_K, Q6_K or Q8_0 (MatMul takes the row type of whatever tensor the stage
 * holds, gguf_projections.cpp:251-262); fp32 rows are GUFO_HIP_ERR_INVALID_ARGUMENT. */
int gufo_hip_gemm_bf16(const gufo_hip_matrix* w, const uint16_t* a_bf16_host, size_t m,
                       float* c_host);
int gufo_hip_gemm_bf16_dev(const gufo_hip_matrix* w, const uint16_t* a_bf16_dev, size_t m,
                           float* c_dev);
/* The same for the matrices of one stage (whole, sharing their input), their outputs side
 * by side within a token's row as MatMul lays them out (gguf_projections.cpp:264-283):
 *   c[t*stride + offset_p + r] = row r of parts[p] . a[t],  stride = the sum of the rows.
 * The activations are converted once for all parts. */
int gufo_hip_gemm_bf16_parts_dev(const gufo_hip_matrix* const* parts, int n_parts,
                                 const uint16_t* a_bf16_dev, size_t m, float* c_dev);
/* Keeps w's weights in the form the prefill product multiplies from (fp16, 512 bytes
 * per 256 weights, beside the packed rows) from now until w is destroyed, so that every
 * gufo_hip_gemm_* call on w converts only its activations: the counterpart of the NPU
 * backend keeping each matrix resident in its own layout (src/npu/gemv.hpp:134-145).
 * Results do not change by a bit.  Not while recording. */
int gufo_hip_matrix_prepare_prefill(gufo_hip_matrix* w);
/* gufo_hip_gemm_bf16 and _dev, refusing any w that is not Q4_K (the type of the prefill
 * configuration). */
int gufo_hip_gemm_q4k_bf16(const gufo_hip_matrix* w, const uint16_t* a_bf16_host,
                           size_t m, float* c_host);
int gufo_hip_gemm_q4k_bf16_dev(const gufo_hip_matrix* w, const uint16_t* a_bf16_dev,
                               size_t m, float* c_dev);

/* ---- replaying a fixed sequence of products -------------------------------- */

/* A recorded sequence of "_dev" calls: the counterpart of the NPU backend's
 * npu::Chain, which submits a layer's products as one runlist
 * (src/npu/gemv.hpp:299-331).  Between capture_begin and capture_end the "_dev"
 * product calls made by this thread are recorded (HIP stream capture) instead of
 * run; graph_launch then enqueues the whole sequence with one submission.  Only the
 * "_dev" product entry points may be called while recording, and every scratch
 * size they need must have been seen by an earlier ordinary call (recording cannot
 * allocate).  The buffers named at record time are the ones every replay uses. */
typedef struct gufo_hip_graph gufo_hip_graph;
int gufo_hip_capture_begin(void);
int gufo_hip_capture_end(gufo_hip_graph** out);
int gufo_hip_graph_launch(gufo_hip_graph* graph);
int gufo_hip_graph_destroy(gufo_hip_graph* graph);

/* ---- measurement ----------------------------------------------------------- */

/* HIP events on the library's stream: begin records the start event, end records
 * the stop event, waits for it and returns the milliseconds between them. */
int gufo_hip_timer_begin(void);
int gufo_hip_timer_end(float* milliseconds);
/* A plain streaming read of `bytes` of device memory: the achievable-read-bandwidth
 * probe, as the reference measures its own ceiling (src/npu/device.hpp:58-74).
 * *sink_dev is written only if a lane's xor of its data equals a magic constant
 * (that keeps the loads alive without timing a store). */
int gufo_hip_read_probe_dev(const void* src_dev, size_t bytes, uint32_t* sink_dev);
/* The write-side twin (the reference's bw_memcpy probe, src/npu/device.hpp:58-66):
 * a plain streaming store of a constant over `bytes` of device memory.  Together
 * the two probes calibrate the memory-traffic counters of a profiler run: both move
 * a known number of bytes. */
int gufo_hip_write_probe_dev(void* dst_dev, size_t bytes);

#ifdef __cplusplus
}
#endif
#endif /* GUFO_HIP_H_ */
