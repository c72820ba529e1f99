// Fused GGUF K-quant matrix-vector product for gfx950 (MI355X).
//
// Computes what GgufProjections::MatMul computes on the CPU
// (src/models/qwen35/gguf_projections.cpp:239-286 of the reference): every output
// is the dot product of one packed weight row with one fp32 activation row,
// y[t*stride + offset + r] = row r . x[t].  Q4_K / Q5_K / Q6_K super-blocks are
// unpacked in registers; nothing is dequantized to memory.
//
// The kernel is bound by the HBM read of the packed weights, so everything else is
// arranged to keep that stream saturated:
//
//   * Persistent waves.  A launch has no more workgroups than are resident at once;
//     every wave walks the rows in a grid-stride loop and holds two or three row
//     visits of weight loads in registers: after the arithmetic of a visit its
//     registers are reloaded with the visit that many steps ahead, so the other
//     visits' loads are in flight during the arithmetic.
//   * Four lanes per super-block, 64 weights per lane, 16 super-blocks per wave
//     pass.  Each lane's share of a block is two or three 16-byte loads (Q6_K
//     blocks are 210 bytes, so those loads are only 2-byte aligned, which gfx950
//     global loads accept).  A pass covers `bpp` consecutive blocks of each of
//     16/bpp consecutive rows, bpp = the largest power of two <= 16 dividing
//     cols/256: one pass is two whole rows for cols = 2048 and eight rows for the
//     512-wide expert down projection.
//   * Integer dot products.  The activation row is quantized once per workgroup
//     into three signed 8-bit limbs per value (a 21-bit integer X with a power-of-
//     two scale per scale group of the weight format: 32 values for Q4_K/Q5_K, 16
//     for Q6_K), staged in LDS in the order the lanes read it, and then held in
//     registers.  The 4/5/6-bit codes are already bytes after unpacking, so a
//     sub-block's sum(code * X) is exact integer arithmetic on v_dot4_i32_i8, 0.75
//     instructions per weight and token instead of a convert and an fma each.  The
//     sub-block sums are converted to fp32 once, scaled (d*sc, the x scale) and
//     accumulated in fp32 across sub-blocks, super-blocks and lanes.  Unit-vector
//     inputs reproduce the dequantized weights bit for bit; for N(0,1) inputs the
//     result is within ~5e-7 (rel-L2) of the double-precision product.
//   * Each decoded weight register is applied to every token column (up to four).
//   * Per-row totals are reduced across lanes with DPP adds in a fixed order.
//
// The arithmetic of a token column does not depend on how many columns travel
// together, so column t of an N-column call equals the one-column call bit for
// bit, and repeated calls give identical bits.
#include "kernels.hpp"
#include "kquant_common.hpp"

namespace gufo {
namespace {

constexpr int kThreads = 256;
constexpr int kWavesPerGroup = kThreads / 64;
constexpr int kBlocksPerPass = 16;  // super-blocks a wave covers per pass (4 lanes each)

// Tuning, by token columns of the launch.  One column leaves registers for three
// row visits of prefetched weights at three waves per SIMD, the occupancy the
// 151,936-row lm_head measured fastest at; more columns hold more quantized
// activations in registers, so they run at lower occupancy and shallower prefetch.
// The macros are for kernel experiments (-D on the hipcc line).
#ifndef GUFO_GEMV_DEPTH
#define GUFO_GEMV_DEPTH 3
#endif
#ifndef GUFO_GEMV_WAVES_PER_EU
#define GUFO_GEMV_WAVES_PER_EU 3
#endif
__host__ __device__ constexpr int DepthFor(int tokens) {
  return tokens <= 2 ? GUFO_GEMV_DEPTH : GUFO_GEMV_DEPTH;
}
__host__ __device__ constexpr int WavesPerSimdFor(int tokens) {
  return tokens == 1 ? GUFO_GEMV_WAVES_PER_EU : 2;
}
// Up to this many token columns keep their quantized activations in registers.
constexpr int kResidentColumns = 2;
// Row groups per workgroup tile of an expert launch (any column count).
constexpr uint32_t kMoeGroupsPerTile = kWavesPerGroup * 3;

int g_compute_units = 256;  // set by SetGemvComputeUnits at library init

struct GemvParams {
  GemvLaunch launch;
  uint32_t start[kMaxGemvParts];  // first flat row of each part
  uint32_t row_bytes;
  uint32_t cols;
  uint32_t bpp_log2;  // blocks of one row per wave pass = 1 << bpp_log2 (<= 16)
  uint32_t passes;    // blocks_per_row >> bpp_log2
  uint32_t n_groups;  // row groups = ceil(total_rows / rows per pass)
};

__device__ __forceinline__ float Fma(float a, float b, float c) {
  return __builtin_fmaf(a, b, c);
}

__device__ __forceinline__ int Dot4(uint32_t codes, uint32_t limbs, int acc) {
  return __builtin_amdgcn_sdot4(static_cast<int>(codes), static_cast<int>(limbs), acc,
                                false);
}

// v / (1 + e^-v) through the hardware's exp2 and reciprocal (about one unit in the last
// place each): every workgroup takes the activation of its whole input row, so the
// library exp and the exact division would cost the wide down projections a
// microsecond.  e^-v overflows to +inf for v < -88.7: 1 / inf = 0, the limit.
__device__ __forceinline__ float Silu(float v) {
  const float e = __builtin_amdgcn_exp2f(v * -1.44269504088896341f);
  return v * __builtin_amdgcn_rcpf(1.0f + e);
}

// ---- the quantized activation row ---------------------------------------------
//
// x = s * X with s a power of two and |X| <= 2^20, X = a0 + 256 a1 + 65536 a2 with
// signed bytes a0, a1 in [-128, 127] and a2 in [-16, 16].  The bytes of four
// consecutive values share a dword per limb, the operand layout of v_dot4_i32_i8.
//
// Per lane (64 values of one super-block):
//   Q4_K/Q5_K  lane p owns sub-blocks 2p and 2p+1: limb[half][limb][8 dwords],
//              xs[half] = s, fx[half] = s * sum(X) (carries the minimum term)
//              = 52 dwords, 13 LDS slots of 16 bytes
//   Q6_K       lane (n, i) owns the four 16-value groups 128n + 32k + 16i:
//              limb[k][limb][4 dwords], xs[k] = s, sx32[k] = 32 * sum(X) (carries
//              the -32 code offset) = 56 dwords, 14 slots
// LDS holds [token][pass][slot][position] x 16 bytes, position = blk_lane*4 + lane
// within the block, so one ds_read_b128 per slot is conflict free.

struct XK4 {
  uint32_t limb[2][3][8];
  float xs[2];
  float fx[2];
};

struct XQ6 {
  uint32_t limb[4][3][4];
  float xs[4];
  int sx32[4];
};

template <int TYPE>
struct XOf {
  using Type = XK4;
};
template <>
struct XOf<kTypeQ6K> {
  using Type = XQ6;
};

template <int TYPE>
__host__ __device__ constexpr int Slots() {
  return TYPE == kTypeQ6K ? 14 : 13;
}

// The power-of-two scale 2^e with gmax * 2^-e in [2^19, 2^20), and its inverse.
// Groups whose largest magnitude is below 2^-107 quantize to zero.
__device__ __forceinline__ void GroupScale(float gmax, float* scale, float* inverse) {
  const uint32_t exponent = (__float_as_uint(gmax) >> 23) & 0xFFu;
  const bool live = exponent >= 20u && exponent < 255u;
  *scale = live ? __uint_as_float((exponent - 19u) << 23) : 0.0f;
  *inverse = live ? __uint_as_float((273u - exponent) << 23) : 0.0f;
}

// Lane exchange inside a quad (DPP quad_perm), for the group-wide max and sum below.
template <int kCtrl>
__device__ __forceinline__ int QuadSwap(int v) {
  return __builtin_amdgcn_mov_dpp(v, kCtrl, 0xF, 0xF, true);
}

// Quantizes the 8 consecutive activations of one thread, given the largest magnitude
// of the whole scale group: two dwords per limb, the scale and the sum of the X.
__device__ __forceinline__ void QuantizeOctet(const float (&v)[8], float gmax,
                                              uint32_t (&limb)[3][2], float* scale,
                                              int* sum) {
  float s, inv;
  GroupScale(gmax, &s, &inv);
  int total = 0;
#pragma unroll
  for (int w = 0; w < 2; ++w) {
    limb[0][w] = 0;
    limb[1][w] = 0;
    limb[2][w] = 0;
  }
#pragma unroll
  for (int c = 0; c < 8; ++c) {
    const int x0 = __float2int_rn(v[c] * inv);
    const int x1 = (x0 + 128) >> 8;
    const int x2 = (x1 + 128) >> 8;
    total += x0;
    const int shift = 8 * (c & 3);
    limb[0][c >> 2] |= static_cast<uint32_t>(x0 & 0xFF) << shift;
    limb[1][c >> 2] |= static_cast<uint32_t>(x1 & 0xFF) << shift;
    limb[2][c >> 2] |= static_cast<uint32_t>(x2 & 0xFF) << shift;
  }
  *scale = s;
  *sum = total;
}

// Where the token columns of one kernel instance live: x[t] is the activation row
// of column t, y[t] the output row.
template <int NTOK>
struct Columns {
  const float* x[NTOK];
  float* y[NTOK];
};

template <int NTOK>
__device__ __forceinline__ const float* ColumnX(const Columns<NTOK>& col, uint32_t t) {
  const float* p = col.x[0];
#pragma unroll
  for (int i = 1; i < NTOK; ++i) {
    if (t == static_cast<uint32_t>(i)) p = col.x[i];
  }
  return p;
}

// ---- cross-lane sum ----------------------------------------------------------------
// Sum over a group of `lanes` (4..64, a power of two) consecutive lanes with DPP adds
// in a fixed order.  The group's last lane ends with the total.
template <int kCtrl, int kRowMask>
__device__ __forceinline__ float DppAdd(float v) {
  const int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), kCtrl, kRowMask, 0xF,
                                                false);
  return v + __int_as_float(moved);
}

__device__ __forceinline__ float GroupTotal(float v, int lanes) {
  v = DppAdd<0xB1, 0xF>(v);                    // quad_perm [1,0,3,2]
  v = DppAdd<0x4E, 0xF>(v);                    // quad_perm [2,3,0,1]
  if (lanes >= 8) v = DppAdd<0x141, 0xF>(v);   // row_half_mirror
  if (lanes >= 16) v = DppAdd<0x140, 0xF>(v);  // row_mirror
  if (lanes >= 32) v = DppAdd<0x142, 0xA>(v);  // row_bcast15 into rows 1 and 3
  if (lanes >= 64) v = DppAdd<0x143, 0xC>(v);  // row_bcast31 into rows 2 and 3
  return v;
}

// ---- what happens to an activation row on its way in -----------------------------------
//   kInPlain    the row as given.
//   kInSwiGlu   the row holds [gate | up] (2*cols values) and the activation is
//               silu(gate) * up, the step between the two products of a feed-forward
//               block (src/models/qwen35/decoder.cpp:511-514,547-549 of the reference).
//   kInResNorm  the activation is RmsNorm(x + delta) * weight: the residual add and the
//               norm that precede the first product of each half of a decoder layer
//               (src/models/qwen35/decoder.cpp:493,504-509; RmsNorm is
//               src/core/vec.hpp:56-63).  Workgroup 0 also stores x + delta and the
//               normalized row for the steps that follow.
constexpr int kInPlain = kProloguePlain;
constexpr int kInSwiGlu = kPrologueSwiGlu;
constexpr int kInResNorm = kPrologueResNorm;

// The 8 consecutive activations one staging thread handles, as loaded.  Fetch only
// issues the loads, so a kernel can have them in flight early; Raw and Values wait for
// them.
template <int kIn>
struct Octet {
  float4 lo[2];
  float4 up[2];      // kInSwiGlu: the up half; kInResNorm: delta
  float4 weight[2];  // kInResNorm: the norm weight

  // `row` is the token's activation row, `at` the first of the 8 values; `delta_row` the
  // token's row of the addend (null: none).
  __device__ __forceinline__ void Fetch(const float* row, uint32_t at, uint32_t cols,
                                        const float* delta_row, const float* norm_weight) {
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      lo[q] = reinterpret_cast<const float4*>(row + at)[q];
      if (kIn == kInSwiGlu) up[q] = reinterpret_cast<const float4*>(row + cols + at)[q];
      if (kIn == kInResNorm) {
        up[q] = delta_row != nullptr ? reinterpret_cast<const float4*>(delta_row + at)[q]
                                     : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        weight[q] = reinterpret_cast<const float4*>(norm_weight + at)[q];
      }
    }
  }

  // kInResNorm: x + delta, the values the norm is taken over.  (x + 0 == x for every x
  // but -0, whose square and whose product are the same as those of +0.)
  __device__ __forceinline__ void Raw(float (&v)[8]) const {
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      v[4 * q + 0] = lo[q].x + up[q].x;
      v[4 * q + 1] = lo[q].y + up[q].y;
      v[4 * q + 2] = lo[q].z + up[q].z;
      v[4 * q + 3] = lo[q].w + up[q].w;
    }
  }

  // The activations.  `inverse_rms` is used by kInResNorm only.
  __device__ __forceinline__ void Values(float (&v)[8], float inverse_rms) const {
    if (kIn == kInResNorm) {
      Raw(v);
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        v[4 * q + 0] = v[4 * q + 0] * inverse_rms * weight[q].x;
        v[4 * q + 1] = v[4 * q + 1] * inverse_rms * weight[q].y;
        v[4 * q + 2] = v[4 * q + 2] * inverse_rms * weight[q].z;
        v[4 * q + 3] = v[4 * q + 3] * inverse_rms * weight[q].w;
      }
      return;
    }
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      float4 f = lo[q];
      if (kIn == kInSwiGlu) {
        const float4 u = up[q];
        f = make_float4(Silu(f.x) * u.x, Silu(f.y) * u.y, Silu(f.z) * u.z, Silu(f.w) * u.w);
      }
      v[4 * q + 0] = f.x;
      v[4 * q + 1] = f.y;
      v[4 * q + 2] = f.z;
      v[4 * q + 3] = f.w;
    }
  }
};

// Token rows of the kInResNorm operands are `cols` floats apart.
template <int kIn>
__device__ __forceinline__ void FetchOctet(Octet<kIn>* piece, const float* row, uint32_t token,
                                           uint32_t at, uint32_t cols,
                                           const GemvPrologue& in) {
  const float* delta_row =
      kIn == kInResNorm && in.delta != nullptr ? in.delta + static_cast<size_t>(token) * cols
                                               : nullptr;
  piece->Fetch(row, at, cols, delta_row, in.norm_weight);
}

// Which token column and which 8 values of it staging piece `u` is.
struct OctetIndex {
  uint32_t token;
  uint32_t block;
  uint32_t piece;  // values 8*piece .. +8 of the block
};

__device__ __forceinline__ OctetIndex IndexOctet(uint32_t u, uint32_t octets_per_token) {
  OctetIndex ix;
  ix.token = u / octets_per_token;
  const uint32_t o = u - ix.token * octets_per_token;
  ix.block = o >> 5;
  ix.piece = o & 31;
  return ix;
}

// Quantizes all token columns into LDS.  A thread takes 8 consecutive values; the two
// (Q6_K, groups of 16) or four (Q4_K/Q5_K, groups of 32) neighbouring threads of a
// scale group agree on its largest magnitude and on sum(X) through quad exchanges.
// The number of 8-value pieces per token is a multiple of 32, so quads are never
// split by the loop bound.
// `first` holds the loads of the thread's first piece (u = threadIdx.x), fetched by the
// caller before it issued its weight loads: memory returns loads in issue order, so
// this way the wait for x does not also wait for the weights.
//
// kInResNorm first takes 1 / rms of every token row.  The sum of squares is formed in an
// order that depends on the row length alone - a thread adds the pieces o = thread,
// thread + 256, ... of a row, the 64 lanes of a wave are added by GroupTotal, the four
// waves in order - so a token's activations, and with them its outputs, are the same
// bits in whichever column of whichever call it travels.  The four wave sums per token
// pass through the 64 bytes of LDS behind the staged rows.
template <int TYPE, int NTOK, int kIn>
__device__ __forceinline__ void StageActivations(const GemvParams& prm,
                                                 const Columns<NTOK>& col,
                                                 const GemvPrologue& in,
                                                 const Octet<kIn>& first, U32x4* lds) {
  constexpr bool kSix = TYPE == kTypeQ6K;
  constexpr uint32_t kSlots = Slots<TYPE>();
  const uint32_t bpp_log2 = prm.bpp_log2;
  const uint32_t positions = 4u << bpp_log2;  // lanes that cover one pass of a row
  const uint32_t octets = prm.launch.blocks_per_row * 32;  // 8-value pieces per token
  float inverse_rms[NTOK];
#pragma unroll
  for (int t = 0; t < NTOK; ++t) inverse_rms[t] = 1.0f;
  if (kIn == kInResNorm) {
    float* wave_sums = reinterpret_cast<float*>(
        lds + static_cast<size_t>(NTOK) * prm.launch.blocks_per_row * 4 * kSlots);
#pragma unroll
    for (int t = 0; t < NTOK; ++t) {
      float squares = 0.0f;
      for (uint32_t o = threadIdx.x; o < octets; o += kThreads) {
        float r[8];
        if (t * octets + o == threadIdx.x) {
          first.Raw(r);
        } else {
          Octet<kIn> piece;
          FetchOctet(&piece, col.x[t], t, o * 8, prm.cols, in);
          piece.Raw(r);
        }
        float of_piece = 0.0f;
#pragma unroll
        for (int c = 0; c < 8; ++c) of_piece = Fma(r[c], r[c], of_piece);
        squares += of_piece;
      }
      squares = GroupTotal(squares, 64);
      if ((threadIdx.x & 63) == 63) wave_sums[t * kWavesPerGroup + (threadIdx.x >> 6)] = squares;
    }
    __syncthreads();
#pragma unroll
    for (int t = 0; t < NTOK; ++t) {
      float total = wave_sums[t * kWavesPerGroup];
#pragma unroll
      for (int w = 1; w < kWavesPerGroup; ++w) total += wave_sums[t * kWavesPerGroup + w];
      inverse_rms[t] = 1.0f / sqrtf(total / static_cast<float>(prm.cols) + in.eps);
    }
  }
  const bool keeps_rows = kIn == kInResNorm && blockIdx.x == 0 && blockIdx.y == 0;
  for (uint32_t u = threadIdx.x; u < NTOK * octets; u += kThreads) {
    const OctetIndex ix = IndexOctet(u, octets);
    const uint32_t t = ix.token;
    const uint32_t block = ix.block;
    const uint32_t piece = ix.piece;
    float inverse = inverse_rms[0];
#pragma unroll
    for (int i = 1; i < NTOK; ++i) {
      if (t == static_cast<uint32_t>(i)) inverse = inverse_rms[i];
    }
    float v[8];
    float r[8];  // kInResNorm: the row before the norm
    if (u == threadIdx.x) {
      first.Values(v, inverse);
      if (kIn == kInResNorm) first.Raw(r);
    } else {
      Octet<kIn> later;
      FetchOctet(&later, ColumnX<NTOK>(col, t), t, block * 256 + piece * 8, prm.cols, in);
      later.Values(v, inverse);
      if (kIn == kInResNorm) later.Raw(r);
    }
    if (keeps_rows) {
      const size_t at = static_cast<size_t>(t) * prm.cols + block * 256 + piece * 8;
      if (in.residual_out != nullptr) {
        reinterpret_cast<float4*>(in.residual_out + at)[0] = make_float4(r[0], r[1], r[2], r[3]);
        reinterpret_cast<float4*>(in.residual_out + at)[1] = make_float4(r[4], r[5], r[6], r[7]);
      }
      if (in.normed_out != nullptr) {
        reinterpret_cast<float4*>(in.normed_out + at)[0] = make_float4(v[0], v[1], v[2], v[3]);
        reinterpret_cast<float4*>(in.normed_out + at)[1] = make_float4(v[4], v[5], v[6], v[7]);
      }
    }
    float gmax = 0.0f;
#pragma unroll
    for (int c = 0; c < 8; ++c) gmax = fmaxf(gmax, fabsf(v[c]));
    gmax = fmaxf(gmax, __int_as_float(QuadSwap<0xB1>(__float_as_int(gmax))));
    if (!kSix) gmax = fmaxf(gmax, __int_as_float(QuadSwap<0x4E>(__float_as_int(gmax))));
    uint32_t limb[3][2];
    float scale;
    int sum;
    QuantizeOctet(v, gmax, limb, &scale, &sum);
    sum += QuadSwap<0xB1>(sum);
    if (!kSix) sum += QuadSwap<0x4E>(sum);

    const uint32_t pass = block >> bpp_log2;
    const uint32_t blk_lane = block & ((1u << bpp_log2) - 1);
    U32x4* base = lds + (static_cast<size_t>(t) * prm.passes + pass) * kSlots * positions +
                  (blk_lane << 2);
    if (kSix) {
      // group = piece/2 = 8n + 2k + i; lane of the block = 2n + i.
      const uint32_t group = piece >> 1;
      const uint32_t half = piece & 1;  // first or second 8 of the 16
      const uint32_t n = group >> 3;
      const uint32_t k = (group & 7) >> 1;
      const uint32_t i = group & 1;
      base += 2 * n + i;
#pragma unroll
      for (int l = 0; l < 3; ++l) {
        U32x2* dst = reinterpret_cast<U32x2*>(base + (k * 3 + l) * positions) + half;
        *dst = U32x2{limb[l][0], limb[l][1]};
      }
      if (half == 0) {
        reinterpret_cast<float*>(base + 12 * positions)[k] = scale;
        reinterpret_cast<int*>(base + 13 * positions)[k] = 32 * sum;
      }
    } else {
      // sub-block j = piece/4; lane of the block = j/2, low or high nibbles = j%2.
      const uint32_t j = piece >> 2;
      const uint32_t quarter = piece & 3;  // which 8 of the 32
      const uint32_t nibble = j & 1;
      base += j >> 1;
#pragma unroll
      for (int l = 0; l < 3; ++l) {
        const uint32_t slot = (nibble * 3 + l) * 2 + (quarter >> 1);
        U32x2* dst = reinterpret_cast<U32x2*>(base + slot * positions) + (quarter & 1);
        *dst = U32x2{limb[l][0], limb[l][1]};
      }
      if (quarter == 0) {
        float* tail = reinterpret_cast<float*>(base + 12 * positions);
        tail[nibble] = scale;
        tail[2 + nibble] = scale * static_cast<float>(sum);
      }
    }
  }
}

__device__ __forceinline__ void LoadX(const U32x4* base, uint32_t positions, XK4* x) {
#pragma unroll
  for (int s = 0; s < 12; ++s) {
    const U32x4 v = base[s * positions];
    const int hl = s >> 1;  // half * 3 + limb
    const int w0 = 4 * (s & 1);
    x->limb[hl / 3][hl % 3][w0 + 0] = v.x;
    x->limb[hl / 3][hl % 3][w0 + 1] = v.y;
    x->limb[hl / 3][hl % 3][w0 + 2] = v.z;
    x->limb[hl / 3][hl % 3][w0 + 3] = v.w;
  }
  const U32x4 tail = base[12 * positions];
  x->xs[0] = __uint_as_float(tail.x);
  x->xs[1] = __uint_as_float(tail.y);
  x->fx[0] = __uint_as_float(tail.z);
  x->fx[1] = __uint_as_float(tail.w);
}

__device__ __forceinline__ void LoadX(const U32x4* base, uint32_t positions, XQ6* x) {
#pragma unroll
  for (int s = 0; s < 12; ++s) {
    const U32x4 v = base[s * positions];
    x->limb[s / 3][s % 3][0] = v.x;
    x->limb[s / 3][s % 3][1] = v.y;
    x->limb[s / 3][s % 3][2] = v.z;
    x->limb[s / 3][s % 3][3] = v.w;
  }
  const U32x4 scales = base[12 * positions];
  const U32x4 sums = base[13 * positions];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    x->xs[k] = __uint_as_float(scales[k]);
    x->sx32[k] = static_cast<int>(sums[k]);
  }
}

// sum over 4*kWords values of code * X, exact: the limbs from the most significant
// down, the accumulator shifted one byte between them.
template <int kWords>
__device__ __forceinline__ int CodeDot(const uint32_t (&codes)[kWords],
                                       const uint32_t (&limb)[3][kWords]) {
  int acc = 0;
#pragma unroll
  for (int w = 0; w < kWords; ++w) acc = Dot4(codes[w], limb[2][w], acc);
  acc <<= 8;
#pragma unroll
  for (int w = 0; w < kWords; ++w) acc = Dot4(codes[w], limb[1][w], acc);
  acc <<= 8;
#pragma unroll
  for (int w = 0; w < kWords; ++w) acc = Dot4(codes[w], limb[0][w], acc);
  return acc;
}

// ---- one lane's share of a super-block: raw bytes, decode, multiply-accumulate ---

// Q4_K / Q5_K.  Lane p (0..3) takes the p-th run of 32 quant bytes: sub-block 2p in
// the low nibbles, 2p+1 in the high nibbles; Q5_K adds bit 2p / 2p+1 of qh[l] as the
// fifth bit.  weight = (d*sc_j)*q - (dmin*m_j), so a sub-block contributes
// (d*sc_j) * sum(q*x) - (dmin*m_j) * sum(x).
template <bool kFifthBit>
struct RawK4 {
  U32x4 header;  // d, dmin, 12 packed scale bytes
  U32x4 qs[2];
  U32x4 qh[2];

  __device__ __forceinline__ void Load(const uint8_t* blk, int lane4) {
    header = Load16(blk);
    const uint8_t* run = blk + 16 + (kFifthBit ? 32 : 0) + 32 * lane4;
    qs[0] = Load16(run);
    qs[1] = Load16(run + 16);
    if (kFifthBit) {
      qh[0] = Load16(blk + 16);
      qh[1] = Load16(blk + 32);
    }
  }

  template <int NTOK, typename XSource>
  __device__ __forceinline__ void Mac(int lane4, const XSource& source,
                                      float (&acc)[NTOK]) const {
    const int p = lane4;
    const float d = HalfBitsToFloat(header.x & 0xFFFFu);
    const float dmin = HalfBitsToFloat(header.x >> 16);
    uint32_t sc0, m0, sc1, m1;
    ScaleMinK4(header.y, header.z, header.w, 2 * p, &sc0, &m0);
    ScaleMinK4(header.y, header.z, header.w, 2 * p + 1, &sc1, &m1);
    const float scale0 = d * static_cast<float>(sc0);
    const float scale1 = d * static_cast<float>(sc1);
    const float min0 = dmin * static_cast<float>(m0);
    const float min1 = dmin * static_cast<float>(m1);
    uint32_t lo[8];
    uint32_t hi[8];
#pragma unroll
    for (int w = 0; w < 8; ++w) {
      const uint32_t q = qs[w >> 2][w & 3];
      lo[w] = q & 0x0F0F0F0Fu;
      hi[w] = (q >> 4) & 0x0F0F0F0Fu;
      if (kFifthBit) {
        const uint32_t h = qh[w >> 2][w & 3];
        lo[w] |= ((h >> (2 * p)) & 0x01010101u) << 4;
        hi[w] |= ((h >> (2 * p + 1)) & 0x01010101u) << 4;
      }
    }
#pragma unroll
    for (int t = 0; t < NTOK; ++t) {
      const XK4 x = source.Get(t);
      const float dot_lo = static_cast<float>(CodeDot<8>(lo, x.limb[0])) * x.xs[0];
      const float dot_hi = static_cast<float>(CodeDot<8>(hi, x.limb[1])) * x.xs[1];
      float part = scale0 * dot_lo;
      part = Fma(-min0, x.fx[0], part);
      part = Fma(scale1, dot_hi, part);
      part = Fma(-min1, x.fx[1], part);
      acc[t] += part;
    }
  }
};

// Q6_K.  Lane (n, i) = (lane/2, lane%2) reads ql[64n+16i..+16), ql[64n+32+16i..+16)
// and qh[32n+16i..+16) and so owns values 128n + 32k + 16i + c for k < 4, c < 16:
// code = 4 low bits from the first (k even) or second (k odd) ql run, low nibble for
// k < 2 and high nibble otherwise, plus bits 2k..2k+1 of qh.
// weight = d * sc[8n + 2k + i] * (code - 32).
struct RawQ6 {
  U32x4 a;
  U32x4 b;
  U32x4 h;
  U32x2 scales;  // this half's eight int8 scales
  uint32_t d;

  __device__ __forceinline__ void Load(const uint8_t* blk, int lane4) {
    const int n = lane4 >> 1;
    const int i = lane4 & 1;
    a = Load16Align2(blk + 64 * n + 16 * i);
    b = Load16Align2(blk + 64 * n + 32 + 16 * i);
    h = Load16Align2(blk + 128 + 32 * n + 16 * i);
    scales = Load8Align2(blk + 192 + 8 * n);
    d = Load2(blk + 208);
  }

  template <int NTOK, typename XSource>
  __device__ __forceinline__ void Mac(int lane4, const XSource& source,
                                      float (&acc)[NTOK]) const {
    const int i = lane4 & 1;
    uint32_t codes[4][4];
    float scale[4];
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      codes[0][w] = (a[w] & 0x0F0F0F0Fu) | ((h[w] << 4) & 0x30303030u);
      codes[1][w] = (b[w] & 0x0F0F0F0Fu) | ((h[w] << 2) & 0x30303030u);
      codes[2][w] = ((a[w] >> 4) & 0x0F0F0F0Fu) | (h[w] & 0x30303030u);
      codes[3][w] = ((b[w] >> 4) & 0x0F0F0F0Fu) | ((h[w] >> 2) & 0x30303030u);
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t word = k < 2 ? scales.x : scales.y;
      const uint32_t shift = 8 * (((2 * k) & 3) + i);
      scale[k] = static_cast<float>(static_cast<int>(word << (24u - shift)) >> 24);
    }
    const float df = HalfBitsToFloat(d);
#pragma unroll
    for (int t = 0; t < NTOK; ++t) {
      const XQ6 x = source.Get(t);
      float block = 0.0f;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int dot = CodeDot<4>(codes[k], x.limb[k]) - x.sx32[k];
        block = Fma(scale[k], static_cast<float>(dot) * x.xs[k], block);
      }
      acc[t] = Fma(df, block, acc[t]);
    }
  }
};

// Q8_0.  256 values are eight blocks of 34 bytes (fp16 scale, 32 int8).  Lane p owns
// blocks 2p and 2p+1 - values 64p .. 64p+63, the split Q4_K's sub-blocks 2p, 2p+1 have,
// so the activation layout is XK4's - at bytes 68p .. 68p+67 of the 272.  The int8
// weights are dot4 operands as they are.  |sum of 32 q*X| can pass 2^31, so the three
// limbs are summed apart (each below 2^19) and joined in fp32.
struct RawQ8 {
  U32x4 q[2][2];
  uint32_t d[2];

  __device__ __forceinline__ void Load(const uint8_t* blk, int lane4) {
    const uint8_t* mine = blk + 68 * lane4;
    d[0] = Load2(mine);
    q[0][0] = Load16Align2(mine + 2);
    q[0][1] = Load16Align2(mine + 18);
    d[1] = Load2(mine + 34);
    q[1][0] = Load16Align2(mine + 36);
    q[1][1] = Load16Align2(mine + 52);
  }

  __device__ __forceinline__ static float BlockDot(const U32x4 (&codes)[2],
                                                   const uint32_t (&limb)[3][8]) {
    float joined = 0.0f;
#pragma unroll
    for (int l = 2; l >= 0; --l) {
      int acc = 0;
#pragma unroll
      for (int w = 0; w < 8; ++w) acc = Dot4(codes[w >> 2][w & 3], limb[l][w], acc);
      joined = Fma(joined, 256.0f, static_cast<float>(acc));
    }
    return joined;
  }

  template <int NTOK, typename XSource>
  __device__ __forceinline__ void Mac(int /*lane4*/, const XSource& source,
                                      float (&acc)[NTOK]) const {
    const float scale0 = HalfBitsToFloat(d[0]);
    const float scale1 = HalfBitsToFloat(d[1]);
#pragma unroll
    for (int t = 0; t < NTOK; ++t) {
      const XK4 x = source.Get(t);
      float part = scale0 * (BlockDot(q[0], x.limb[0]) * x.xs[0]);
      part = Fma(scale1, BlockDot(q[1], x.limb[1]) * x.xs[1], part);
      acc[t] += part;
    }
  }
};

template <int TYPE>
struct RawOf {
  using Type = RawK4<TYPE == kTypeQ5K>;
};
template <>
struct RawOf<kTypeQ80> {
  using Type = RawQ8;
};
template <>
struct RawOf<kTypeQ6K> {
  using Type = RawQ6;
};

// Where a visit's arithmetic takes the quantized activations of token column t
// from: registers (one or two columns: loaded once per pass, reused by every row
// visit) or LDS (three or four columns would not leave registers for the weight
// prefetch, so each visit reads them again).
template <typename X, int NTOK>
struct ResidentX {
  X x[NTOK];
  __device__ __forceinline__ const X& Get(int t) const { return x[t]; }
};

template <typename X>
struct LdsX {
  const U32x4* base;       // this lane's position in column 0 of the current pass
  uint32_t column_stride;  // 16-byte units between token columns
  uint32_t positions;
  __device__ __forceinline__ X Get(int t) const {
    X x;
    LoadX(base + static_cast<size_t>(t) * column_stride, positions, &x);
    return x;
  }
};

// ---- the product ---------------------------------------------------------------------

// One workgroup's share.  Row group g (16 >> bpp_log2 consecutive flat rows) is
// visited by one wave; this wave takes groups g_first, g_first + g_stride, ... below
// g_end.  part_shift is added to every part's row pointer: the byte offset of an
// expert inside its 3-D tensor (the parts of one launch share the expert stride).
// With kPick no output is stored: best[t] collects this lane's best output of column t.
template <int TYPE, int NTOK, int kIn, bool kPick = false>
__device__ __forceinline__ void GemvBody(const GemvParams& prm, const Columns<NTOK>& col,
                                         const GemvPrologue& in, size_t part_shift,
                                         uint32_t g_first, uint32_t g_stride, uint32_t g_end,
                                         U32x4* lds, Best* best = nullptr) {
  using Raw = typename RawOf<TYPE>::Type;
  using X = typename XOf<TYPE>::Type;
  constexpr int kBlockBytes = BlockBytes(TYPE);
  constexpr uint32_t kSlots = Slots<TYPE>();
  constexpr int kDepth = DepthFor(NTOK);  // row visits of weight loads held in registers

  const int lane = threadIdx.x & 63;
  const uint32_t bpp_log2 = prm.bpp_log2;
  const uint32_t bpp = 1u << bpp_log2;
  const uint32_t rpp = kBlocksPerPass >> bpp_log2;
  const int lanes_per_row = 4 << bpp_log2;
  const int lane4 = lane & 3;
  const uint32_t blk_lane = (lane >> 2) & (bpp - 1);
  const uint32_t row_lane = lane >> (2 + bpp_log2);
  const uint32_t position = (blk_lane << 2) + lane4;
  const uint32_t positions = 4u << bpp_log2;
  const uint32_t passes = prm.passes;

  // State of the kDepth visits in flight: where the lane's row starts, where its
  // output goes, and the raw bytes of the next block to consume.
  Raw raw[kDepth];
  const uint8_t* row_base[kDepth];
  uint32_t y_index[kDepth];
  bool valid[kDepth];

  const uint8_t* const base0 =
      prm.launch.part[0].rows + part_shift + static_cast<size_t>(blk_lane) * kBlockBytes;
  const uint32_t y_offset0 = prm.launch.part[0].y_offset;
  const bool one_part = prm.launch.n_parts == 1;
  auto locate = [&](int d, uint32_t group) {
    const uint32_t flat = group * rpp + row_lane;
    valid[d] = group < g_end && flat < prm.launch.total_rows;
    if (one_part) {
      row_base[d] = base0 + static_cast<size_t>(flat) * prm.row_bytes;
      y_index[d] = y_offset0 + flat;
      return;
    }
    const uint8_t* base = prm.launch.part[0].rows;
    uint32_t start = 0;
    uint32_t y_offset = y_offset0;
#pragma unroll
    for (int p = 1; p < kMaxGemvParts; ++p) {
      if (p < static_cast<int>(prm.launch.n_parts) && flat >= prm.start[p]) {
        base = prm.launch.part[p].rows;
        start = prm.start[p];
        y_offset = prm.launch.part[p].y_offset;
      }
    }
    row_base[d] = base + part_shift + static_cast<size_t>(flat - start) * prm.row_bytes +
                  static_cast<size_t>(blk_lane) * kBlockBytes;
    y_index[d] = y_offset + (flat - start);
  };
  auto issue = [&](int d, uint32_t pass) {
    if (valid[d]) {
      raw[d].Load(row_base[d] + static_cast<size_t>(pass) * bpp * kBlockBytes, lane4);
    }
  };

  // The thread's first piece of x, then the first weight loads, then the staging:
  // both latencies overlap, and the wait for x does not wait for the weights.
  Octet<kIn> first_piece;
  {
    const uint32_t octets = prm.launch.blocks_per_row * 32;
    if (threadIdx.x < NTOK * octets) {
      const OctetIndex ix = IndexOctet(threadIdx.x, octets);
      FetchOctet(&first_piece, ColumnX<NTOK>(col, ix.token), ix.token,
                 ix.block * 256 + ix.piece * 8, prm.cols, in);
    }
  }
#pragma unroll
  for (int d = 0; d < kDepth; ++d) {
    locate(d, g_first + d * g_stride);
    issue(d, 0);
  }

  StageActivations<TYPE, NTOK, kIn>(prm, col, in, first_piece, lds);
  __syncthreads();

  constexpr bool kResident = NTOK <= kResidentColumns;
  ResidentX<X, kResident ? NTOK : 1> resident;
  LdsX<X> streamed;
  streamed.column_stride = passes * kSlots * positions;
  streamed.positions = positions;
  float acc[kDepth][NTOK];
  uint32_t group0 = g_first;  // group of visit 0 of the current iteration
  uint32_t pass = 0;
  while (group0 < g_end) {
    if (pass == 0) {
#pragma unroll
      for (int d = 0; d < kDepth; ++d) {
#pragma unroll
        for (int t = 0; t < NTOK; ++t) acc[d][t] = 0.0f;
      }
    }
    const U32x4* pass_base = lds + static_cast<size_t>(pass) * kSlots * positions + position;
    if (kResident) {
      if (passes > 1 || group0 == g_first) {
#pragma unroll
        for (int t = 0; t < (kResident ? NTOK : 1); ++t) {
          LoadX(pass_base + static_cast<size_t>(t) * streamed.column_stride, positions,
                &resident.x[t]);
        }
      }
    } else {
      streamed.base = pass_base;
    }
    const bool last_pass = pass + 1 == passes;
    const uint32_t next_pass = last_pass ? 0 : pass + 1;
    const uint32_t next_group0 = last_pass ? group0 + kDepth * g_stride : group0;
#pragma unroll
    for (int d = 0; d < kDepth; ++d) {
      // The arithmetic of this visit, then the loads of the visit that takes over its
      // registers: kDepth - 1 visits stay in flight meanwhile.
      if (valid[d]) {
        if (kResident) {
          raw[d].template Mac<NTOK>(lane4, resident, acc[d]);
        } else {
          raw[d].template Mac<NTOK>(lane4, streamed, acc[d]);
        }
      }
      if (last_pass) {
#pragma unroll
        for (int t = 0; t < NTOK; ++t) {
          const float total = GroupTotal(acc[d][t], lanes_per_row);
          if (valid[d] && (lane & (lanes_per_row - 1)) == lanes_per_row - 1) {
            if (kPick) {
              best[t] = Better(best[t], Best{total, y_index[d]});
            } else {
              col.y[t][y_index[d]] = total;
            }
          }
        }
        locate(d, next_group0 + d * g_stride);
      }
      issue(d, next_pass);
    }
    pass = next_pass;
    group0 = next_group0;
  }
}

// Dense product: token t reads x + t*cols and writes y + t*y_stride; the waves of
// the whole grid share the row groups round robin.
// With kInSwiGlu token t's [gate | up] row is x + t*2*cols.
template <int TYPE, int NTOK, int kIn>
__global__ __launch_bounds__(kThreads)
__attribute__((amdgpu_waves_per_eu(WavesPerSimdFor(NTOK)))) void KquantGemvKernel(
    const GemvParams prm, const GemvPrologue in, const float* __restrict__ x,
    float* __restrict__ y) {
  extern __shared__ __align__(16) U32x4 lds[];
  Columns<NTOK> col;
  const size_t x_row_floats = kIn == kInSwiGlu ? 2 * static_cast<size_t>(prm.cols) : prm.cols;
#pragma unroll
  for (int t = 0; t < NTOK; ++t) {
    col.x[t] = x + static_cast<size_t>(t) * x_row_floats;
    col.y[t] = y + static_cast<size_t>(t) * prm.launch.y_stride;
  }
  const uint32_t wave = blockIdx.x * kWavesPerGroup + (threadIdx.x >> 6);
  GemvBody<TYPE, NTOK, kIn>(prm, col, in, 0, wave, gridDim.x * kWavesPerGroup, prm.n_groups,
                            lds);
}

// The dense product with the greedy pick inside: no y.  Every lane keeps the best output
// it formed per token; the workgroup's best goes to pick.partial[t][blockIdx.x], and
// GemvPickFinalKernel, launched behind it, takes the best of those (at most 768 per
// token).  Better is a total order, so the result does not depend on how the rows were
// spread over lanes and workgroups.  (Finishing inside this kernel - the last workgroup
// to arrive, found with a device-scope counter, reduces - was built and measured: the
// device-scope fences it needs around the counter made the 151,936-row head 77 us
// against 50 us, as each fence writes back and invalidates an L2 that is per XCD.)
template <int TYPE, int NTOK, int kIn>
__global__ __launch_bounds__(kThreads)
__attribute__((amdgpu_waves_per_eu(WavesPerSimdFor(NTOK)))) void KquantGemvPickKernel(
    const GemvParams prm, const GemvPrologue in, const float* __restrict__ x,
    const GemvPick pick) {
  extern __shared__ __align__(16) U32x4 lds[];
  Columns<NTOK> col;
#pragma unroll
  for (int t = 0; t < NTOK; ++t) {
    col.x[t] = x + static_cast<size_t>(t) * prm.cols;
    col.y[t] = nullptr;
  }
  Best best[NTOK];
#pragma unroll
  for (int t = 0; t < NTOK; ++t) best[t] = Best{-INFINITY, kNoIndex};
  const uint32_t wave = blockIdx.x * kWavesPerGroup + (threadIdx.x >> 6);
  GemvBody<TYPE, NTOK, kIn, true>(prm, col, in, 0, wave, gridDim.x * kWavesPerGroup,
                                  prm.n_groups, lds, best);

  // The staged activations are dead once every wave has left the loop; their LDS now
  // carries the wave results (NTOK x 4 candidates).
  __syncthreads();
  Best* wave_best = reinterpret_cast<Best*>(lds);
#pragma unroll
  for (int t = 0; t < NTOK; ++t) {
    const Best of_wave = WaveBest(best[t]);
    if ((threadIdx.x & 63) == 0) wave_best[t * kWavesPerGroup + (threadIdx.x >> 6)] = of_wave;
  }
  __syncthreads();
  Best* partial = static_cast<Best*>(pick.partial);
  if (threadIdx.x < NTOK) {
    Best of_group = wave_best[threadIdx.x * kWavesPerGroup];
#pragma unroll
    for (int w = 1; w < kWavesPerGroup; ++w) {
      of_group = Better(of_group, wave_best[threadIdx.x * kWavesPerGroup + w]);
    }
    partial[threadIdx.x * gridDim.x + blockIdx.x] = of_group;
  }
}

// The best of the `groups` candidates of token blockIdx.x -> pick.index / pick.value.
__global__ __launch_bounds__(kThreads) void GemvPickFinalKernel(const GemvPick pick,
                                                                uint32_t groups) {
  __shared__ Best wave_best[kWavesPerGroup];
  const uint32_t t = blockIdx.x;
  const Best* partial = static_cast<const Best*>(pick.partial) + t * groups;
  Best mine{-INFINITY, kNoIndex};
  for (uint32_t i = threadIdx.x; i < groups; i += kThreads) mine = Better(mine, partial[i]);
  mine = WaveBest(mine);
  if ((threadIdx.x & 63) == 0) wave_best[threadIdx.x >> 6] = mine;
  __syncthreads();
  if (threadIdx.x == 0) {
    Best all = wave_best[0];
#pragma unroll
    for (int w = 1; w < kWavesPerGroup; ++w) all = Better(all, wave_best[w]);
    // Nothing but -inf and NaN: max_element returns the first element.
    pick.index[t] = all.index == kNoIndex ? 0 : static_cast<int64_t>(all.index);
    if (pick.value != nullptr) pick.value[t] = all.value;
  }
}

// Expert product: blockIdx.y names a segment, i.e. one routed expert and up to four
// of the (token, slot) pairs that chose it; blockIdx.x a tile of the expert's row
// groups.  The expert's rows are streamed once for all of the segment's pairs.
// Column t reads the activation row of its pair (the token's x, or with kSwiGlu the
// pair's [gate | up] row) and writes the pair's output row.
template <int TYPE, int NTOK, bool kSwiGlu>
__device__ __forceinline__ void MoeSegmentBody(const GemvParams& prm,
                                               const MoeGemvArgs& moe,
                                               const MoeSegment& seg, U32x4* lds) {
  Columns<NTOK> col;
#pragma unroll
  for (int t = 0; t < NTOK; ++t) {
    const uint32_t pair = static_cast<uint32_t>(seg.pair[t]);
    const size_t x_row = kSwiGlu ? pair : pair / moe.k;
    col.x[t] = moe.x + x_row * moe.x_row_floats;
    col.y[t] = moe.y + static_cast<size_t>(pair) * prm.launch.y_stride;
  }
  const size_t shift = static_cast<size_t>(seg.expert) * moe.expert_bytes;
  const uint32_t first = blockIdx.x * kMoeGroupsPerTile;
  const uint32_t end = min(first + kMoeGroupsPerTile, prm.n_groups);
  GemvBody<TYPE, NTOK, kSwiGlu ? kInSwiGlu : kInPlain>(
      prm, col, GemvPrologue{}, shift, first + (threadIdx.x >> 6), kWavesPerGroup, end, lds);
}

// kMaxTok bounds the pairs of a segment (the launch's token count, at most four):
// a one-token call compiles only the one-column body and keeps its registers.
template <int TYPE, bool kSwiGlu, int kMaxTok>
__global__ __launch_bounds__(kThreads)
__attribute__((amdgpu_waves_per_eu(WavesPerSimdFor(kMaxTok)))) void KquantMoeGemvKernel(
    const GemvParams prm, const MoeGemvArgs moe) {
  extern __shared__ __align__(16) U32x4 lds[];
  const uint32_t s = blockIdx.y;
  MoeSegment seg;
  if (moe.direct_ids != nullptr) {
    // An ungrouped one-token call: segment s is slot s.
    seg.expert = moe.direct_ids[s];
    if (seg.expert < 0 || seg.expert >= moe.experts) return;
    seg.n_pairs = 1;
#pragma unroll
    for (int t = 0; t < kMaxGemvTokens; ++t) seg.pair[t] = static_cast<int32_t>(s);
  } else {
    if (s >= static_cast<uint32_t>(moe.tables->n_segments)) return;
    seg = moe.segments[s];
  }
  if (kMaxTok == 1 || seg.n_pairs == 1) {
    MoeSegmentBody<TYPE, 1, kSwiGlu>(prm, moe, seg, lds);
  } else if (kMaxTok >= 2 && seg.n_pairs == 2) {
    MoeSegmentBody<TYPE, kMaxTok >= 2 ? 2 : 1, kSwiGlu>(prm, moe, seg, lds);
  } else if (kMaxTok >= 3 && seg.n_pairs == 3) {
    MoeSegmentBody<TYPE, kMaxTok >= 3 ? 3 : 1, kSwiGlu>(prm, moe, seg, lds);
  } else {
    MoeSegmentBody<TYPE, kMaxTok >= 4 ? 4 : 1, kSwiGlu>(prm, moe, seg, lds);
  }
}

// ---- host side -------------------------------------------------------------------------

size_t LdsBytes(int type, uint32_t blocks_per_row, int tokens) {
  const size_t slots = type == kTypeQ6K ? Slots<kTypeQ6K>() : Slots<kTypeQ4K>();
  return static_cast<size_t>(tokens) * blocks_per_row * 4 * slots * 16;
}

bool ValidLaunch(int type, const GemvLaunch& launch) {
  return BlockBytes(type) != 0 && launch.n_parts >= 1 &&
         launch.n_parts <= kMaxGemvParts && launch.blocks_per_row != 0;
}

void PlanGemv(int type, const GemvLaunch& launch, GemvParams* prm) {
  prm->launch = launch;
  const uint32_t nb = launch.blocks_per_row;
  prm->row_bytes = nb * BlockBytes(type);
  prm->cols = nb * 256;
  // Blocks of a row per wave pass: the largest power of two (up to 16) dividing nb, so
  // that no lane idles.  (Measured alternative for rows with an odd factor, e.g. 2560 =
  // 10 blocks as 2 blocks x 5 passes: one padded pass of 16 block slots with 6 idle gives
  // more, shorter work items but ran 20-60% slower at every column count.)
  uint32_t bpp_log2 = 0;
  while (bpp_log2 < 4 && (nb & ((2u << bpp_log2) - 1)) == 0) ++bpp_log2;
  prm->bpp_log2 = bpp_log2;
  prm->passes = nb >> bpp_log2;
  const uint32_t rpp = kBlocksPerPass >> bpp_log2;
  prm->n_groups = (launch.total_rows + rpp - 1) / rpp;
  uint32_t start = 0;
  for (uint32_t p = 0; p < static_cast<uint32_t>(kMaxGemvParts); ++p) {
    prm->start[p] = start;
    if (p < launch.n_parts) start += launch.part[p].n_rows;
  }
}

// Kernels whose LDS need may exceed the 64 KB default are allowed the full LDS of a
// gfx950 compute unit.
template <typename Kernel>
hipError_t AllowLargeLds(Kernel kernel, size_t lds_bytes) {
  if (lds_bytes <= 64 * 1024) return hipSuccess;
  return hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                             hipFuncAttributeMaxDynamicSharedMemorySize,
                             static_cast<int>(kGemvMaxLdsBytes));
}

struct DenseCall {
  GemvParams prm;
  GemvPrologue in;
  const float* x;
  float* y;
  dim3 grid;
  size_t lds_bytes;
  hipStream_t stream;
};

template <int TYPE, int NTOK, int kIn>
hipError_t LaunchDense(const DenseCall& call) {
  const hipError_t status = AllowLargeLds(KquantGemvKernel<TYPE, NTOK, kIn>, call.lds_bytes);
  if (status != hipSuccess) return status;
  hipLaunchKernelGGL((KquantGemvKernel<TYPE, NTOK, kIn>), call.grid, dim3(kThreads),
                     call.lds_bytes, call.stream, call.prm, call.in, call.x, call.y);
  return hipGetLastError();
}

template <int TYPE, int NTOK>
hipError_t LaunchColumns(const DenseCall& call) {
  switch (call.in.kind) {
    case kInPlain: return LaunchDense<TYPE, NTOK, kInPlain>(call);
    case kInSwiGlu: return LaunchDense<TYPE, NTOK, kInSwiGlu>(call);
    case kInResNorm: return LaunchDense<TYPE, NTOK, kInResNorm>(call);
    default: return hipErrorInvalidValue;
  }
}

template <int TYPE>
hipError_t LaunchTyped(const DenseCall& call, int tokens) {
  switch (tokens) {
    case 1: return LaunchColumns<TYPE, 1>(call);
    case 2: return LaunchColumns<TYPE, 2>(call);
    case 3: return LaunchColumns<TYPE, 3>(call);
    case 4: return LaunchColumns<TYPE, 4>(call);
    default: return hipErrorInvalidValue;
  }
}

template <int TYPE, int NTOK, int kIn>
hipError_t LaunchPick(const DenseCall& call, const GemvPick& pick) {
  const hipError_t status =
      AllowLargeLds(KquantGemvPickKernel<TYPE, NTOK, kIn>, call.lds_bytes);
  if (status != hipSuccess) return status;
  hipLaunchKernelGGL((KquantGemvPickKernel<TYPE, NTOK, kIn>), call.grid, dim3(kThreads),
                     call.lds_bytes, call.stream, call.prm, call.in, call.x, pick);
  hipLaunchKernelGGL(GemvPickFinalKernel, dim3(NTOK), dim3(kThreads), 0, call.stream, pick,
                     call.grid.x);
  return hipGetLastError();
}

template <int TYPE, int NTOK>
hipError_t LaunchPickColumns(const DenseCall& call, const GemvPick& pick) {
  return call.in.kind == kInResNorm ? LaunchPick<TYPE, NTOK, kInResNorm>(call, pick)
                                    : LaunchPick<TYPE, NTOK, kInPlain>(call, pick);
}

template <int TYPE>
hipError_t LaunchPickTyped(const DenseCall& call, const GemvPick& pick, int tokens) {
  switch (tokens) {
    case 1: return LaunchPickColumns<TYPE, 1>(call, pick);
    case 2: return LaunchPickColumns<TYPE, 2>(call, pick);
    case 3: return LaunchPickColumns<TYPE, 3>(call, pick);
    case 4: return LaunchPickColumns<TYPE, 4>(call, pick);
    default: return hipErrorInvalidValue;
  }
}

template <int TYPE, bool kSwiGlu, int kMaxTok>
hipError_t LaunchMoeKernel(const GemvParams& prm, const MoeGemvArgs& moe, dim3 grid,
                           size_t lds_bytes, hipStream_t stream) {
  const hipError_t status =
      AllowLargeLds(KquantMoeGemvKernel<TYPE, kSwiGlu, kMaxTok>, lds_bytes);
  if (status != hipSuccess) return status;
  hipLaunchKernelGGL((KquantMoeGemvKernel<TYPE, kSwiGlu, kMaxTok>), grid, dim3(kThreads),
                     lds_bytes, stream, prm, moe);
  return hipGetLastError();
}

template <int TYPE>
hipError_t LaunchMoeTyped(const GemvParams& prm, const MoeGemvArgs& moe, bool swiglu,
                          bool one_token, dim3 grid, size_t lds_bytes, hipStream_t stream) {
  if (swiglu) {
    return one_token ? LaunchMoeKernel<TYPE, true, 1>(prm, moe, grid, lds_bytes, stream)
                     : LaunchMoeKernel<TYPE, true, 4>(prm, moe, grid, lds_bytes, stream);
  }
  return one_token ? LaunchMoeKernel<TYPE, false, 1>(prm, moe, grid, lds_bytes, stream)
                   : LaunchMoeKernel<TYPE, false, 4>(prm, moe, grid, lds_bytes, stream);
}

}  // namespace

void SetGemvComputeUnits(int compute_units) {
  if (compute_units > 0) g_compute_units = compute_units;
}

int DeviceComputeUnits() { return g_compute_units; }

int GemvMaxTokens(int type, uint32_t blocks_per_row) {
  if (type == kTypeF32) return kMaxGemvTokens;  // no staging in LDS
  const size_t per_token = LdsBytes(type, blocks_per_row, 1);
  if (per_token == 0) return 0;
  const size_t fit = kGemvMaxLdsBytes / per_token;
  return static_cast<int>(fit < static_cast<size_t>(kMaxGemvTokens) ? fit : kMaxGemvTokens);
}

hipError_t LaunchGemv(int type, const GemvLaunch& launch, const float* x, int tokens,
                      float* y, hipStream_t stream) {
  return LaunchGemvFused(type, launch, GemvPrologue{}, x, tokens, y, stream);
}

namespace {

// Checks a dense launch and fills everything of `call` but its output.
hipError_t PlanDense(int type, const GemvLaunch& launch, const GemvPrologue& in,
                     const float* x, int tokens, hipStream_t stream, DenseCall* call) {
  if (!ValidLaunch(type, launch) || tokens < 1 ||
      tokens > GemvMaxTokens(type, launch.blocks_per_row)) {
    return hipErrorInvalidValue;
  }
  if (in.kind == kInResNorm && in.norm_weight == nullptr) return hipErrorInvalidValue;
  call->in = in;
  call->x = x;
  call->y = nullptr;
  call->stream = stream;
  // kInResNorm keeps the four wave sums of every token behind the staged rows.
  call->lds_bytes = LdsBytes(type, launch.blocks_per_row, tokens) +
                    (in.kind == kInResNorm ? kMaxGemvTokens * kWavesPerGroup * sizeof(float) : 0);
  if (call->lds_bytes > kGemvMaxLdsBytes) return hipErrorInvalidValue;
  PlanGemv(type, launch, &call->prm);
  uint32_t blocks = (call->prm.n_groups + kWavesPerGroup - 1) / kWavesPerGroup;
  // Persistent: no more workgroups than are resident at once.
  const uint32_t resident =
      static_cast<uint32_t>(g_compute_units) * WavesPerSimdFor(tokens);
  if (blocks > resident) blocks = resident;
  call->grid = dim3(blocks);
  return hipSuccess;
}

}  // namespace

size_t GemvPickPartialBytes(int tokens) {
  return static_cast<size_t>(tokens > 0 ? tokens : 0) * g_compute_units *
         WavesPerSimdFor(1) * sizeof(Best);
}

hipError_t LaunchGemvPick(int type, const GemvLaunch& launch, const GemvPrologue& in,
                          const float* x, int tokens, const GemvPick& pick,
                          hipStream_t stream) {
  if (in.kind != kInPlain && in.kind != kInResNorm) return hipErrorInvalidValue;
  if (pick.partial == nullptr || pick.index == nullptr || launch.total_rows == 0) {
    return hipErrorInvalidValue;
  }
  DenseCall call;
  const hipError_t status = PlanDense(type, launch, in, x, tokens, stream, &call);
  if (status != hipSuccess) return status;
  switch (type) {
    case kTypeQ4K: return LaunchPickTyped<kTypeQ4K>(call, pick, tokens);
    case kTypeQ5K: return LaunchPickTyped<kTypeQ5K>(call, pick, tokens);
    case kTypeQ6K: return LaunchPickTyped<kTypeQ6K>(call, pick, tokens);
    case kTypeQ80: return LaunchPickTyped<kTypeQ80>(call, pick, tokens);
    default: return hipErrorInvalidValue;
  }
}

hipError_t LaunchGemvFused(int type, const GemvLaunch& launch, const GemvPrologue& in,
                           const float* x, int tokens, float* y, hipStream_t stream) {
  if (type == kTypeF32) {
    // The fp32 kernel reads x as it goes and has no staging step to fuse into.
    if (in.kind != kInPlain) return hipErrorInvalidValue;
    return LaunchGemvF32(launch, x, tokens, y, stream);
  }
  DenseCall call;
  const hipError_t status = PlanDense(type, launch, in, x, tokens, stream, &call);
  if (status != hipSuccess) return status;
  if (launch.total_rows == 0) return hipSuccess;
  call.y = y;
  switch (type) {
    case kTypeQ4K: return LaunchTyped<kTypeQ4K>(call, tokens);
    case kTypeQ5K: return LaunchTyped<kTypeQ5K>(call, tokens);
    case kTypeQ6K: return LaunchTyped<kTypeQ6K>(call, tokens);
    case kTypeQ80: return LaunchTyped<kTypeQ80>(call, tokens);
    default: return hipErrorInvalidValue;
  }
}

hipError_t LaunchMoeGemv(int type, const GemvLaunch& launch, const MoeGemvArgs& moe,
                         bool swiglu, uint32_t max_segments, int max_pairs,
                         hipStream_t stream) {
  // Expert tensors are K-quants (the reference's models hold them as Q4_K .. Q6_K).
  if (type != kTypeQ4K && type != kTypeQ5K && type != kTypeQ6K) return hipErrorInvalidValue;
  if (!ValidLaunch(type, launch) || max_pairs < 1 ||
      GemvMaxTokens(type, launch.blocks_per_row) < kMaxGemvTokens) {
    return hipErrorInvalidValue;
  }
  if (launch.total_rows == 0 || max_segments == 0) return hipSuccess;
  GemvParams prm;
  PlanGemv(type, launch, &prm);
  // Sized for the widest segment the launch can hold; narrower ones use less of it.
  const bool one_token = max_pairs == 1;
  const size_t lds_bytes =
      LdsBytes(type, launch.blocks_per_row, one_token ? 1 : kMaxGemvTokens);
  const dim3 grid((prm.n_groups + kMoeGroupsPerTile - 1) / kMoeGroupsPerTile, max_segments);
  switch (type) {
    case kTypeQ4K:
      return LaunchMoeTyped<kTypeQ4K>(prm, moe, swiglu, one_token, grid, lds_bytes, stream);
    case kTypeQ5K:
      return LaunchMoeTyped<kTypeQ5K>(prm, moe, swiglu, one_token, grid, lds_bytes, stream);
    default:
      return LaunchMoeTyped<kTypeQ6K>(prm, moe, swiglu, one_token, grid, lds_bytes, stream);
  }
}

}  // namespace gufo
