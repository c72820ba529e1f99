/*
 * TEST INFRASTRUCTURE, NOT PRODUCT CODE.  See kquant_oracle.h for what this file
 * is, who may use it and how each function is pinned.
 *
 * Plain C, scalar, fp arithmetic exactly as written (build with
 * -ffp-contract=off).  Paths in comments are under the reference's src/.
 */
#include "kquant_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdatomic.h>
#include <stdlib.h>
#include <string.h>

enum { kSuper = 256, kSub = 32, kPackedScales = 12 };

static uint16_t load_u16(const uint8_t* p) {
  uint16_t v;
  memcpy(&v, p, sizeof v);
  return v;
}

/* core/quant.cpp:129-155.  Sign, 5-bit exponent, 10-bit mantissa; subnormals are
 * renormalised, inf/nan keep their payload. */
float gufo_oracle_half_to_float(uint16_t h) {
  const uint32_t sign = (uint32_t)(h >> 15) << 31;
  const uint32_t e = (h >> 10) & 31u;
  uint32_t m = h & 1023u;
  uint32_t bits;
  if (e == 31u) {
    bits = sign | 0x7F800000u | (m << 13);
  } else if (e != 0u) {
    bits = sign | ((e + 112u) << 23) | (m << 13);
  } else if (m == 0u) {
    bits = sign;
  } else {
    uint32_t exp32 = 113u; /* 127 - 15 + 1 */
    while ((m & 1024u) == 0u) {
      m <<= 1;
      --exp32;
    }
    bits = sign | (exp32 << 23) | ((m & 1023u) << 13);
  }
  float f;
  memcpy(&f, &bits, sizeof f);
  return f;
}

size_t gufo_oracle_block_bytes(int type) {
  switch (type) {
    case GUFO_ORACLE_Q4_K: return 144; /* 2+2+12+128 */
    case GUFO_ORACLE_Q5_K: return 176; /* 2+2+12+32+128 */
    case GUFO_ORACLE_Q6_K: return 210; /* 128+64+16+2 */
    case GUFO_ORACLE_Q8_0: return 34;  /* 2+32 */
    case GUFO_ORACLE_F32: return 4;
    default: return 0;
  }
}

size_t gufo_oracle_block_elements(int type) {
  switch (type) {
    case GUFO_ORACLE_Q4_K:
    case GUFO_ORACLE_Q5_K:
    case GUFO_ORACLE_Q6_K: return kSuper;
    case GUFO_ORACLE_Q8_0: return kSub;
    case GUFO_ORACLE_F32: return 1;
    default: return 0;
  }
}

size_t gufo_oracle_row_bytes(int type, size_t n) {
  const size_t bytes = gufo_oracle_block_bytes(type);
  const size_t elements = gufo_oracle_block_elements(type);
  if (bytes == 0 || n % elements != 0) return 0;
  return n / elements * bytes;
}

/* core/quant.cpp:158-167.  Twelve bytes hold eight 6-bit scales and eight 6-bit
 * mins: the first four of each in the low six bits of bytes 0-3 / 4-7; the last
 * four split into a nibble of bytes 8-11 and the top two bits of bytes 0-7. */
void gufo_oracle_scale_min_k4(size_t j, const uint8_t* s, uint8_t* scale,
                              uint8_t* min) {
  if (j < 4) {
    *scale = s[j] & 0x3F;
    *min = s[4 + j] & 0x3F;
    return;
  }
  const uint8_t tail = s[4 + j]; /* bytes 8..11 */
  *scale = (uint8_t)((tail & 0x0F) | ((s[j - 4] >> 6) << 4));
  *min = (uint8_t)((tail >> 4) | ((s[j] >> 6) << 4));
}

/* The 4- or 5-bit code of value `l` in sub-block `j` of a Q4_K/Q5_K block
 * (core/quant.cpp:49-54,81-88; models/qwen35/gguf_dot.hpp:109-114): nibble j&1 of
 * byte l in the (j/2)-th run of 32 quant bytes; bit j of qh[l] adds 16. */
static int code_k4(const uint8_t* qs, const uint8_t* qh, int j, int l) {
  const uint8_t byte = qs[32 * (j >> 1) + l];
  int v = (j & 1) ? (byte >> 4) : (byte & 0x0F);
  if (qh != NULL && ((qh[l] >> j) & 1)) v += 16;
  return v;
}

/* core/quant.cpp:33-59 (Q4_K) and 62-95 (Q5_K): value = (d*sc)*q - (dmin*m). */
static void dequant_k4(const uint8_t* src, float* dst, size_t blocks, int fifth) {
  const size_t stride = fifth ? 176 : 144;
  for (size_t b = 0; b < blocks; ++b, src += stride, dst += kSuper) {
    const float d = gufo_oracle_half_to_float(load_u16(src));
    const float dmin = gufo_oracle_half_to_float(load_u16(src + 2));
    const uint8_t* packed = src + 4;
    const uint8_t* qh = fifth ? src + 16 : NULL;
    const uint8_t* qs = src + 16 + (fifth ? 32 : 0);
    for (int j = 0; j < 8; ++j) {
      uint8_t sc, m;
      gufo_oracle_scale_min_k4((size_t)j, packed, &sc, &m);
      const float scale = d * (float)sc;
      const float offset = dmin * (float)m;
      for (int l = 0; l < kSub; ++l) {
        dst[kSub * j + l] = scale * (float)code_k4(qs, qh, j, l) - offset;
      }
    }
  }
}

/* The signed 6-bit code (q - 32) of value p (0..127) in half `half` of a Q6_K
 * block (core/quant.cpp:104-118; models/qwen35/gguf_dot.hpp:195-202): with
 * k = p/32 and l = p%32 the low four bits come from ql[l] (k even) or ql[l+32]
 * (k odd), low nibble for k<2 and high nibble otherwise; bits 2k..2k+1 of qh[l]
 * go on top. */
static int code_q6(const uint8_t* ql, const uint8_t* qh, int p) {
  const int k = p >> 5;
  const int l = p & 31;
  const uint8_t byte = ql[l + ((k & 1) ? 32 : 0)];
  const int low = (k < 2) ? (byte & 0x0F) : (byte >> 4);
  const int high = (qh[l] >> (2 * k)) & 3;
  return (low | (high << 4)) - 32;
}

/* core/quant.cpp:98-125: value = d * sc[p/16] * q, evaluated left to right. */
static void dequant_q6(const uint8_t* src, float* dst, size_t blocks) {
  for (size_t b = 0; b < blocks; ++b, src += 210, dst += kSuper) {
    const int8_t* sc = (const int8_t*)(src + 192);
    const float d = gufo_oracle_half_to_float(load_u16(src + 208));
    for (int half = 0; half < 2; ++half) {
      const uint8_t* ql = src + 64 * half;
      const uint8_t* qh = src + 128 + 32 * half;
      for (int p = 0; p < 128; ++p) {
        const float scale = (float)sc[8 * half + p / 16];
        dst[128 * half + p] = d * scale * (float)code_q6(ql, qh, p);
      }
    }
  }
}

/* core/quant.cpp:22-31: fp16 scale times 32 int8. */
static void dequant_q8_0(const uint8_t* src, float* dst, size_t blocks) {
  for (size_t b = 0; b < blocks; ++b, src += 34, dst += kSub) {
    const float d = gufo_oracle_half_to_float(load_u16(src));
    const int8_t* q = (const int8_t*)(src + 2);
    for (int j = 0; j < kSub; ++j) dst[j] = d * (float)q[j];
  }
}

int gufo_oracle_dequantize(int type, const uint8_t* src, float* dst, size_t n) {
  if (gufo_oracle_row_bytes(type, n) == 0 && n != 0) return -1;
  if (type == GUFO_ORACLE_F32) {
    memcpy(dst, src, n * sizeof(float));
    return 0;
  }
  if (type == GUFO_ORACLE_Q8_0) {
    dequant_q8_0(src, dst, n / kSub);
    return 0;
  }
  const size_t blocks = n / kSuper;
  switch (type) {
    case GUFO_ORACLE_Q4_K: dequant_k4(src, dst, blocks, 0); return 0;
    case GUFO_ORACLE_Q5_K: dequant_k4(src, dst, blocks, 1); return 0;
    default: dequant_q6(src, dst, blocks); return 0;
  }
}

/* models/qwen35/gguf_dot.hpp:156-182: per super-block an fp32 sum of
 * (scale_j*q - min_j)*x over sub-blocks in order; block sums added in order. */
static float dot_k4(const uint8_t* row, const float* x, size_t n, int fifth) {
  const size_t stride = fifth ? 176 : 144;
  float total = 0.0f;
  for (size_t b = 0; b < n / kSuper; ++b, row += stride, x += kSuper) {
    const float d = gufo_oracle_half_to_float(load_u16(row));
    const float dmin = gufo_oracle_half_to_float(load_u16(row + 2));
    const uint8_t* qh = fifth ? row + 16 : NULL;
    const uint8_t* qs = row + 16 + (fifth ? 32 : 0);
    float block = 0.0f;
    for (int j = 0; j < 8; ++j) {
      uint8_t sc, m;
      gufo_oracle_scale_min_k4((size_t)j, row + 4, &sc, &m);
      const float scale = d * (float)sc;
      const float offset = dmin * (float)m;
      for (int l = 0; l < kSub; ++l) {
        const float w = scale * (float)code_k4(qs, qh, j, l) - offset;
        block += w * x[kSub * j + l];
      }
    }
    total += block;
  }
  return total;
}

float gufo_oracle_dot_q4_k(const uint8_t* row, const float* x, size_t n) {
  return dot_k4(row, x, n, 0);
}

float gufo_oracle_dot_q5_k(const uint8_t* row, const float* x, size_t n) {
  return dot_k4(row, x, n, 1);
}

/* models/qwen35/gguf_dot.hpp:260-289: codes times x summed per 16 values, times
 * that group's int8 scale into the block sum, times d into the row sum. */
float gufo_oracle_dot_q6_k(const uint8_t* row, const float* x, size_t n) {
  float total = 0.0f;
  for (size_t b = 0; b < n / kSuper; ++b, row += 210, x += kSuper) {
    const int8_t* sc = (const int8_t*)(row + 192);
    const float d = gufo_oracle_half_to_float(load_u16(row + 208));
    float block = 0.0f;
    for (int half = 0; half < 2; ++half) {
      const uint8_t* ql = row + 64 * half;
      const uint8_t* qh = row + 128 + 32 * half;
      for (int g = 0; g < 8; ++g) {
        float group = 0.0f;
        for (int i = 0; i < 16; ++i) {
          const int p = 16 * g + i;
          group += (float)code_q6(ql, qh, p) * x[128 * half + p];
        }
        block += (float)sc[8 * half + g] * group;
      }
    }
    total += d * block;
  }
  return total;
}

/* models/qwen35/gguf_dot.hpp:62-74: per block an fp32 sum of q*x in order, times the
 * block's scale into the row sum. */
float gufo_oracle_dot_q8_0(const uint8_t* row, const float* x, size_t n) {
  float sum = 0.0f;
  for (size_t b = 0; b < n / kSub; ++b, row += 34) {
    const int8_t* q = (const int8_t*)(row + 2);
    float block = 0.0f;
    for (int j = 0; j < kSub; ++j) block += (float)q[j] * x[b * kSub + j];
    sum += gufo_oracle_half_to_float(load_u16(row)) * block;
  }
  return sum;
}

/* core/vec.hpp:36-51: eight interleaved partial sums, added in order, then the tail. */
float gufo_oracle_dot_f32(const uint8_t* row, const float* x, size_t n) {
  float lanes[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  size_t i = 0;
  for (; i + 8 <= n; i += 8) {
    for (int l = 0; l < 8; ++l) {
      float w;
      memcpy(&w, row + 4 * (i + (size_t)l), sizeof w);
      lanes[l] += w * x[i + (size_t)l];
    }
  }
  float total = 0.0f;
  for (int l = 0; l < 8; ++l) total += lanes[l];
  for (; i < n; ++i) {
    float w;
    memcpy(&w, row + 4 * i, sizeof w);
    total += w * x[i];
  }
  return total;
}

static double dot_double_buf(int type, const uint8_t* row, const float* x,
                             size_t n, float* w) {
  gufo_oracle_dequantize(type, row, w, n);
  double sum = 0.0;
  for (size_t i = 0; i < n; ++i) sum += (double)w[i] * x[i];
  return sum;
}

double gufo_oracle_dot_double(int type, const uint8_t* row, const float* x,
                              size_t n) {
  if (gufo_oracle_row_bytes(type, n) == 0) return NAN;
  float* w = (float*)malloc(n * sizeof(float));
  const double sum = dot_double_buf(type, row, x, n, w);
  free(w);
  return sum;
}

static float dot_fused(int type, const uint8_t* row, const float* x, size_t n) {
  switch (type) {
    case GUFO_ORACLE_Q4_K: return dot_k4(row, x, n, 0);
    case GUFO_ORACLE_Q5_K: return dot_k4(row, x, n, 1);
    case GUFO_ORACLE_Q8_0: return gufo_oracle_dot_q8_0(row, x, n);
    case GUFO_ORACLE_F32: return gufo_oracle_dot_f32(row, x, n);
    default: return gufo_oracle_dot_q6_k(row, x, n);
  }
}

/* ---- MatMul: models/qwen35/gguf_projections.cpp:239-286 ------------------ */

enum { kChunkRows = 16 }; /* gguf_projections.cpp:244 */

typedef struct {
  int n_parts;
  const uint8_t* const* data;
  const int* types;
  const size_t* first;
  const size_t* rows;
  size_t in;
  const float* x;
  int tokens;
  float* y;
  int precision;
  size_t stride;
  size_t n_jobs;
  const size_t* first_job; /* n_parts + 1 */
  atomic_size_t next;
} MatMulTask;

static void matmul_job(const MatMulTask* t, size_t job, float* scratch) {
  int p = 0;
  size_t offset = 0;
  while (job >= t->first_job[p + 1]) {
    offset += t->rows[p];
    ++p;
  }
  const int type = t->types[p];
  const size_t row_bytes = gufo_oracle_row_bytes(type, t->in);
  const size_t begin = (job - t->first_job[p]) * kChunkRows;
  size_t end = begin + kChunkRows;
  if (end > t->rows[p]) end = t->rows[p];
  for (size_t r = begin; r < end; ++r) {
    const uint8_t* row = t->data[p] + (t->first[p] + r) * row_bytes;
    if (t->precision == 1) gufo_oracle_dequantize(type, row, scratch, t->in);
    for (int tok = 0; tok < t->tokens; ++tok) {
      const float* xt = t->x + (size_t)tok * t->in;
      float out;
      if (t->precision == 1) {
        double sum = 0.0;
        for (size_t i = 0; i < t->in; ++i) sum += (double)scratch[i] * xt[i];
        out = (float)sum;
      } else {
        out = dot_fused(type, row, xt, t->in);
      }
      t->y[(size_t)tok * t->stride + offset + r] = out;
    }
  }
}

static void* matmul_worker(void* arg) {
  MatMulTask* t = (MatMulTask*)arg;
  float* scratch = (float*)malloc(t->in * sizeof(float));
  for (;;) {
    const size_t job = atomic_fetch_add(&t->next, 1);
    if (job >= t->n_jobs) break;
    matmul_job(t, job, scratch);
  }
  free(scratch);
  return NULL;
}

int gufo_oracle_matmul(int n_parts, const uint8_t* const* data, const int* types,
                       const size_t* first, const size_t* rows, size_t in,
                       const float* x, int tokens, float* y, int precision,
                       int threads) {
  if (n_parts <= 0 || tokens < 0 || in == 0) return -1;
  size_t* first_job = (size_t*)malloc(((size_t)n_parts + 1) * sizeof(size_t));
  MatMulTask task;
  memset(&task, 0, sizeof task);
  first_job[0] = 0;
  for (int p = 0; p < n_parts; ++p) {
    if (gufo_oracle_row_bytes(types[p], in) == 0) { /* unknown type or partial block */
      free(first_job);
      return -1;
    }
    task.stride += rows[p];
    first_job[p + 1] = first_job[p] + (rows[p] + kChunkRows - 1) / kChunkRows;
  }
  task.n_parts = n_parts;
  task.data = data;
  task.types = types;
  task.first = first;
  task.rows = rows;
  task.in = in;
  task.x = x;
  task.tokens = tokens;
  task.y = y;
  task.precision = precision;
  task.n_jobs = first_job[n_parts];
  task.first_job = first_job;
  atomic_init(&task.next, 0);
  if (threads > 64) threads = 64;
  if (threads <= 1 || task.n_jobs <= 1) {
    matmul_worker(&task);
  } else {
    pthread_t ids[64];
    int started = 0;
    for (int i = 0; i < threads - 1; ++i) {
      if (pthread_create(&ids[started], NULL, matmul_worker, &task) == 0) ++started;
    }
    matmul_worker(&task);
    for (int i = 0; i < started; ++i) pthread_join(ids[i], NULL);
  }
  free(first_job);
  return 0;
}

/* ---- Routing: models/qwen35/moe.cpp:16-42 -------------------------------- */

void gufo_oracle_route(const float* logits, int experts, int k, int* chosen,
                       float* weights) {
  double* prob = (double*)malloc((size_t)experts * sizeof(double));
  char* taken = (char*)calloc((size_t)experts, 1);
  float max_logit = logits[0];
  for (int e = 1; e < experts; ++e) {
    if (logits[e] > max_logit) max_logit = logits[e];
  }
  double total = 0.0;
  for (int e = 0; e < experts; ++e) {
    prob[e] = exp((double)logits[e] - (double)max_logit);
    total += prob[e];
  }
  /* k rounds of selection: highest probability not yet taken, the lower index
   * on a tie - the order std::partial_sort produces under moe.cpp:29-32. */
  for (int slot = 0; slot < k; ++slot) {
    int best = -1;
    for (int e = 0; e < experts; ++e) {
      if (taken[e]) continue;
      if (best < 0 || prob[e] > prob[best]) best = e;
    }
    taken[best] = 1;
    chosen[slot] = best;
  }
  double top = 0.0;
  for (int slot = 0; slot < k; ++slot) top += prob[chosen[slot]] / total;
  const double floor_sum = 6.103515625e-5; /* smallest normal fp16, moe.cpp:12 */
  if (top < floor_sum) top = floor_sum;
  for (int slot = 0; slot < k; ++slot) {
    weights[slot] = (float)(prob[chosen[slot]] / total / top);
  }
  free(prob);
  free(taken);
}

int64_t gufo_oracle_argmax(const float* v, size_t n) {
  size_t best = 0;
  for (size_t i = 1; i < n; ++i) {
    if (v[best] < v[i]) best = i;
  }
  return (int64_t)best;
}

float gufo_oracle_silu(float x) { return x / (1.0f + expf(-x)); }

void gufo_oracle_rms_norm(const float* x, const float* w, size_t n, float eps,
                          float* out) {
  float lanes[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  size_t i = 0;
  for (; i + 8 <= n; i += 8) {
    for (int l = 0; l < 8; ++l) lanes[l] += x[i + l] * x[i + l];
  }
  float total = 0.0f;
  for (int l = 0; l < 8; ++l) total += lanes[l];
  for (; i < n; ++i) total += x[i] * x[i];
  const float inv = 1.0f / sqrtf(total / (float)n + eps);
  for (i = 0; i < n; ++i) out[i] = x[i] * inv * w[i];
}

void gufo_oracle_res_norm(const float* x, const float* delta, const float* w, size_t n,
                          float eps, float* residual, float* normed) {
  for (size_t i = 0; i < n; ++i) normed[i] = delta != NULL ? x[i] + delta[i] : x[i];
  if (residual != NULL) memcpy(residual, normed, n * sizeof(float));
  gufo_oracle_rms_norm(normed, w, n, eps, normed);
}

void gufo_oracle_swiglu(const float* gate_up, size_t f, float* act) {
  for (size_t i = 0; i < f; ++i) {
    const float g = gate_up[i];
    const float sigmoid = 1.0f / (1.0f + expf(-g));
    act[i] = g * sigmoid * gate_up[f + i];
  }
}

/* ---- Expert grouping and the routed FFN: reference.cpp:514-607 ----------- */

int gufo_oracle_moe_group(const int* chosen, int tokens, int k, int experts,
                          int* counts, int* offsets, int* pairs) {
  const int n = tokens * k;
  memset(counts, 0, (size_t)experts * sizeof(int));
  for (int i = 0; i < n; ++i) ++counts[chosen[i]];
  offsets[0] = 0;
  int distinct = 0;
  for (int e = 0; e < experts; ++e) {
    offsets[e + 1] = offsets[e] + counts[e];
    if (counts[e] != 0) ++distinct;
  }
  int* cursor = (int*)malloc((size_t)experts * sizeof(int));
  memcpy(cursor, offsets, (size_t)experts * sizeof(int));
  for (int i = 0; i < n; ++i) pairs[cursor[chosen[i]]++] = i;
  free(cursor);
  return distinct;
}

int gufo_oracle_moe_ffn(const uint8_t* gate, int gate_type, const uint8_t* up,
                        int up_type, const uint8_t* down, int down_type,
                        int experts, int hidden, int ffn, const float* logits,
                        const float* x, int tokens, int k, int* chosen,
                        float* weights, float* y, int precision, int threads) {
  if (tokens <= 0 || k <= 0 || k > experts) return -1;
  const size_t d = (size_t)hidden;
  const size_t f = (size_t)ffn;
  const int n = tokens * k;
  for (int t = 0; t < tokens; ++t) {
    gufo_oracle_route(logits + (size_t)t * experts, experts, k, chosen + t * k,
                      weights + t * k);
  }
  int* counts = (int*)malloc((size_t)experts * sizeof(int));
  int* offsets = (int*)malloc(((size_t)experts + 1) * sizeof(int));
  int* pairs = (int*)malloc((size_t)n * sizeof(int));
  gufo_oracle_moe_group(chosen, tokens, k, experts, counts, offsets, pairs);
  float* routed = (float*)malloc((size_t)n * d * sizeof(float));
  float* xs = (float*)malloc((size_t)tokens * d * sizeof(float));
  float* gate_up = (float*)malloc((size_t)tokens * 2 * f * sizeof(float));
  float* act = (float*)malloc((size_t)tokens * f * sizeof(float));
  float* ys = (float*)malloc((size_t)tokens * d * sizeof(float));
  int status = 0;
  for (int e = 0; e < experts && status == 0; ++e) {
    const int m = counts[e];
    if (m == 0) continue;
    const int* slots = pairs + offsets[e];
    for (int r = 0; r < m; ++r) {
      memcpy(xs + (size_t)r * d, x + (size_t)(slots[r] / k) * d, d * sizeof(float));
    }
    const uint8_t* in_data[2] = {gate, up};
    const int in_types[2] = {gate_type, up_type};
    const size_t in_first[2] = {(size_t)e * f, (size_t)e * f};
    const size_t in_rows[2] = {f, f};
    status |= gufo_oracle_matmul(2, in_data, in_types, in_first, in_rows, d, xs, m,
                                 gate_up, precision, threads);
    for (int r = 0; r < m; ++r) {
      const float* g = gate_up + (size_t)r * 2 * f;
      for (size_t i = 0; i < f; ++i) {
        act[(size_t)r * f + i] = gufo_oracle_silu(g[i]) * g[f + i];
      }
    }
    const uint8_t* down_data[1] = {down};
    const int down_types[1] = {down_type};
    const size_t down_first[1] = {(size_t)e * d};
    const size_t down_rows[1] = {d};
    status |= gufo_oracle_matmul(1, down_data, down_types, down_first, down_rows, f,
                                 act, m, ys, precision, threads);
    for (int r = 0; r < m; ++r) {
      memcpy(routed + (size_t)slots[r] * d, ys + (size_t)r * d, d * sizeof(float));
    }
  }
  for (int t = 0; t < tokens; ++t) {
    for (size_t i = 0; i < d; ++i) {
      double acc = 0.0;
      for (int slot = 0; slot < k; ++slot) {
        const size_t s = (size_t)t * k + slot;
        acc += (double)weights[s] * routed[s * d + i];
      }
      y[(size_t)t * d + i] = (float)acc;
    }
  }
  free(counts); free(offsets); free(pairs); free(routed);
  free(xs); free(gate_up); free(act); free(ys);
  return status == 0 ? 0 : -1;
}
