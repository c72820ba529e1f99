/*
 * Model-level C interface of the MI355X backend: a GGUF model file opened, its weights
 * in HBM, and the reference's `Projections` calls on it.
 *
 * Where include/gufo_hip.h replaces the arithmetic of GgufProjections, this header
 * replaces the object itself as a consumer sees it: construct from a model file
 * (GgufProjections::GgufProjections(const gguf::File&, Precision),
 * src/models/qwen35/gguf_projections.hpp:27-30), then Apply / ApplyExpert by stage and
 * layer (src/models/qwen35/projections.hpp:45-59).  It is what a binding from another
 * language (ctypes, cgo, JNI) would bind; C++ callers use GgufModel
 * (gufo-npu_amd/host/gguf_model.hpp) directly.  Implemented in libgufo_hip_model.so,
 * which links libgufo_hip.so.
 *
 * Every function returns a gufo_hip_status code (include/gufo_hip.h) unless stated;
 * gufo_model_last_error() gives the message of the calling thread's last failure.  The
 * exception the C++ layer raised maps to the code as in gufo_hip.h: std::runtime_error
 * (unreadable or malformed file, not a Qwen3.5 model, wrong tensor shape, no device)
 * -> RUNTIME, std::invalid_argument -> INVALID_ARGUMENT, std::logic_error (no weights
 * for a stage, no such expert) -> LOGIC, std::out_of_range (layer) -> OUT_OF_RANGE.
 */
#ifndef GUFO_HIP_MODEL_H_
#define GUFO_HIP_MODEL_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* qwen35::Stage (src/models/qwen35/projections.hpp:14-39), same order. */
enum gufo_model_stage {
  GUFO_STAGE_LINEAR_IN = 0,    /* [qkv | z | alpha | beta] */
  GUFO_STAGE_ATTENTION_IN = 1, /* [q and gate | k | v] */
  GUFO_STAGE_MIXER_OUT = 2,    /* ssm_out or attn_output */
  GUFO_STAGE_FFN_IN = 3,       /* [gate | up]: dense FFN or the shared expert */
  GUFO_STAGE_FFN_DOWN = 4,
  GUFO_STAGE_LM_HEAD = 5,
  GUFO_STAGE_ROUTER = 6,       /* [expert logits | shared-expert gate logit] */
  GUFO_STAGE_EXPERT_IN = 7,    /* apply_expert only */
  GUFO_STAGE_EXPERT_DOWN = 8,  /* apply_expert only */
  GUFO_STAGE_MTP_IN = 9        /* nextn.eh_proj */
};

/* qwen35::Config (src/models/qwen35/config.hpp:13-60) as plain fields. */
typedef struct gufo_model_shape {
  int is_moe; /* architecture "qwen35moe" (1) or "qwen35" (0) */
  int layers;
  int mtp_layers;
  int hidden;
  int ffn;
  int vocab;
  float rms_eps;
  int full_attention_interval;
  int heads;
  int kv_heads;
  int head_dim;
  int rope_dim;
  float rope_theta;
  int conv_kernel;
  int linear_key_heads;
  int linear_value_heads;
  int linear_head_dim;
  int experts;
  int experts_used;
  int expert_ffn;
  int shared_expert_ffn;
  int tied_embeddings;
  int has_mtp_layer; /* HasMtpLayer (config.cpp:74-78) */
  int tensors;       /* tensor records in the file */
} gufo_model_shape;

typedef struct gufo_model gufo_model;

const char* gufo_model_last_error(void);

/* Reads the file's header only - gguf::File::Open + ReadConfig + the shape checks of the
 * GgufProjections constructor - without touching a device.  For tools and for hosts
 * that want to validate a file before they commit HBM to it. */
int gufo_model_inspect(const char* path, gufo_model_shape* shape);

/* Opens the file, checks it as gufo_model_inspect does, initialises the library on
 * `device` and copies every projection weight to HBM.  The file stays mapped until
 * gufo_model_close. */
int gufo_model_open(const char* path, int device, gufo_model** out);
int gufo_model_close(gufo_model* model);
int gufo_model_get_shape(const gufo_model* model, gufo_model_shape* shape);
/* Bytes of projection weights resident in HBM. */
uint64_t gufo_model_weight_bytes(const gufo_model* model);

/* StageInputs / StageOutputs (src/models/qwen35/reference.cpp:609-648): values per token
 * row a stage reads and writes; 0 for a stage the layer does not have. */
size_t gufo_model_stage_inputs(const gufo_model* model, int stage, int layer);
size_t gufo_model_stage_outputs(const gufo_model* model, int stage, int layer);

/* The resident matrices behind a stage, in the order of its parts
 * (src/models/qwen35/gguf_projections.cpp:100-175), for callers that keep their rows on
 * the device and drive gufo_hip.h's "_dev" entry points themselves (gufo_hip_gemv_fused_dev,
 * gufo_hip_gemv_argmax_dev, gufo_hip_gemm_bf16_parts_dev, gufo_hip_moe_layer_dev ...).
 * *count receives the number of parts (0 for a stage the layer does not have); with `out`
 * given, `capacity` must hold them.  The handles belong to the model: never destroy them. */
struct gufo_hip_matrix;
int gufo_model_stage_matrices(const gufo_model* model, int stage, int layer,
                              const struct gufo_hip_matrix** out, int capacity, int* count);
/* The expert tensors of a mixture layer (ffn_gate_exps, ffn_up_exps, ffn_down_exps); null
 * for a dense layer.  Any of the three pointers may be null. */
int gufo_model_expert_matrices(const gufo_model* model, int layer,
                               const struct gufo_hip_matrix** gate,
                               const struct gufo_hip_matrix** up,
                               const struct gufo_hip_matrix** down);

/* Projections::Apply: y[t] = W x[t], host pointers, any tokens >= 0.  `layer` is ignored
 * for GUFO_STAGE_LM_HEAD. */
int gufo_model_apply(const gufo_model* model, int stage, int layer, const float* x,
                     int tokens, float* y);
/* Projections::ApplyExpert for GUFO_STAGE_EXPERT_IN / _DOWN of routed expert `expert`. */
int gufo_model_apply_expert(const gufo_model* model, int stage, int layer, int expert,
                            const float* x, int tokens, float* y);

/* The norm weights a decoder keeps beside the products (Decoder's attn_norm,
 * post_attention_norm and output_norm, src/models/qwen35/decoder.cpp:449-454): copies
 * `hidden` floats.  which: 0 attn_norm, 1 post_attention_norm of `layer`; 2 output_norm. */
int gufo_model_norm_weight(const gufo_model* model, int which, int layer, float* out);

#ifdef __cplusplus
}
#endif
#endif /* GUFO_HIP_MODEL_H_ */
