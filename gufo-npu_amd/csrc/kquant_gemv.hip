// Fused GGUF K-quant matrix-vector product for gfx950 (MI355X).
//
// Computes what GgufProjections::MatMul computes on the CPU
// (src/models/qwen35/gguf_projections.cpp:239-286 of the reference): every output
// is the dot product of one packed weight row with one fp32 activation row,
// y[t*stride + offset + r] = row r . x[t].  Q4_K / Q5_K / Q6_K super-blocks are
// unpacked in registers; nothing is dequantized to memory.
//
// Work decomposition (wave64):
//   * A super-block (256 weights) is decoded by 8 consecutive lanes, 32 weights
//     each, so that every lane's share of the quant bytes is one or three
//     contiguous vector loads and consecutive lanes read consecutive addresses.
//   * A wave pass covers 8 super-blocks: `bpp` consecutive blocks of each of
//     8/bpp consecutive rows, bpp = the largest power of two <= 8 dividing
//     cols/256.  For cols = 2048 one pass is exactly one row; for the 512-wide
//     expert down projection it is four rows.
//   * The activation rows (all token columns) are staged in LDS once per
//     workgroup and K-chunk together with the sums of every 8 consecutive values,
//     which carry the Q4_K/Q5_K minimum term and Q6_K's -32 code offset.
//   * Each weight register is decoded once and applied to every token column.
//   * Per-row totals are reduced with wavefront shuffles in a fixed order.
//
// The arithmetic per token column does not depend on how many columns travel
// together, so column t of an N-column call equals the one-column call bit for
// bit.
#include "kernels.hpp"
#include "kquant_common.hpp"

namespace gufo {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;
constexpr int kVisits = 4;  // row groups each wave owns within a workgroup
constexpr int kLdsBudget = 48 * 1024;
// LDS floats per staged super-block and token: 256 values + 32 sums of 8.
constexpr int kLdsFloatsPerBlock = 256 + 32;

struct GemvParams {
  GemvLaunch launch;
  uint32_t row_bytes;
  uint32_t cols;
  uint32_t bpp_log2;      // blocks of one row per wave pass = 1 << bpp_log2
  uint32_t rows_per_wg;   // kVisits * kWaves * (8 >> bpp_log2)
  uint32_t chunk_blocks;  // super-blocks of x staged at a time
};

__device__ __forceinline__ float Fma(float a, float b, float c) {
  return __builtin_fmaf(a, b, c);
}

// Sum of four byte codes times four activations, added to acc.
__device__ __forceinline__ float Dot4Bytes(uint32_t codes, float4 x, float acc) {
  acc = Fma(Byte0(codes), x.x, acc);
  acc = Fma(Byte1(codes), x.y, acc);
  acc = Fma(Byte2(codes), x.z, acc);
  acc = Fma(Byte3(codes), x.w, acc);
  return acc;
}

// ---- Q4_K / Q5_K ------------------------------------------------------------
// Lane `sub` (0..7) of a block takes 16 of the 128 quant bytes: run p = sub/2 of
// 32 bytes (sub-blocks 2p from the low nibbles and 2p+1 from the high nibbles),
// half h = sub%2 of that run, i.e. values 16h..16h+15 of both sub-blocks.
// weight = (d*sc_j)*q - (dmin*m_j), so a sub-block contributes
// (d*sc_j) * sum(q*x) - (dmin*m_j) * sum(x).
template <bool kFifthBit, int NTOK>
__device__ __forceinline__ void MacK4(const uint8_t* blk, int sub, const float* xb,
                                      const float* sb, int x_stride, int s_stride,
                                      float (&acc)[NTOK]) {
  const int p = sub >> 1;
  const int h = sub & 1;
  const U32x4 hdr = Load16(blk);
  const U32x4 q = Load16(blk + 16 + (kFifthBit ? 32 : 0) + 32 * p + 16 * h);
  U32x4 high = {0, 0, 0, 0};
  if (kFifthBit) high = Load16(blk + 16 + 16 * h);

  const float d = HalfBitsToFloat(hdr.x & 0xFFFFu);
  const float dmin = HalfBitsToFloat(hdr.x >> 16);
  uint32_t sc0, m0, sc1, m1;
  ScaleMinK4(hdr.y, hdr.z, hdr.w, 2 * p, &sc0, &m0);
  ScaleMinK4(hdr.y, hdr.z, hdr.w, 2 * p + 1, &sc1, &m1);
  const float scale0 = d * static_cast<float>(sc0);
  const float scale1 = d * static_cast<float>(sc1);
  const float min0 = dmin * static_cast<float>(m0);
  const float min1 = dmin * static_cast<float>(m1);

  uint32_t lo[4];
  uint32_t hi[4];
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    lo[w] = q[w] & 0x0F0F0F0Fu;
    hi[w] = (q[w] >> 4) & 0x0F0F0F0Fu;
    if (kFifthBit) {
      lo[w] |= ((high[w] >> (2 * p)) & 0x01010101u) << 4;
      hi[w] |= ((high[w] >> (2 * p + 1)) & 0x01010101u) << 4;
    }
  }
#pragma unroll
  for (int t = 0; t < NTOK; ++t) {
    const float4* xl =
        reinterpret_cast<const float4*>(xb + t * x_stride + 64 * p + 16 * h);
    const float4* xh = xl + 8;  // +32 values
    float dot_lo = 0.0f;
    float dot_hi = 0.0f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      dot_lo = Dot4Bytes(lo[w], xl[w], dot_lo);
      dot_hi = Dot4Bytes(hi[w], xh[w], dot_hi);
    }
    const float* s = sb + t * s_stride + 8 * p + 2 * h;
    const float sum_lo = s[0] + s[1];
    const float sum_hi = s[4] + s[5];
    float part = scale0 * dot_lo;
    part = Fma(-min0, sum_lo, part);
    part = Fma(scale1, dot_hi, part);
    part = Fma(-min1, sum_hi, part);
    acc[t] += part;
  }
}

// ---- Q6_K -------------------------------------------------------------------
// Lane `sub` (0..7): half n = sub/4 of the block (128 values), eighth i = sub%4.
// It reads ql[64n+8i..+8), ql[64n+32+8i..+8) and qh[32n+8i..+8) and so owns
// values 128n + 32k + 8i + c for k < 4, c < 8: code = 4 low bits from the first
// (k even) or second (k odd) ql run, low nibble for k < 2 and high nibble
// otherwise, plus bits 2k..2k+1 of qh.  weight = d * sc[8n + 2k + i/2] * (code-32).
template <int NTOK>
__device__ __forceinline__ void MacQ6K(const uint8_t* blk, int sub, const float* xb,
                                       const float* sb, int x_stride, int s_stride,
                                       float (&acc)[NTOK]) {
  const int n = sub >> 2;
  const int i = sub & 3;
  const U32x2 a = Load8Align2(blk + 64 * n + 8 * i);
  const U32x2 b = Load8Align2(blk + 64 * n + 32 + 8 * i);
  const U32x2 hq = Load8Align2(blk + 128 + 32 * n + 8 * i);
  const U32x2 sc8 = Load8Align2(blk + 192 + 8 * n);
  const float d = HalfBitsToFloat(Load2(blk + 208));

  uint32_t codes[4][2];
  float scale[4];
#pragma unroll
  for (int w = 0; w < 2; ++w) {
    codes[0][w] = (a[w] & 0x0F0F0F0Fu) | ((hq[w] << 4) & 0x30303030u);
    codes[1][w] = (b[w] & 0x0F0F0F0Fu) | ((hq[w] << 2) & 0x30303030u);
    codes[2][w] = ((a[w] >> 4) & 0x0F0F0F0Fu) | (hq[w] & 0x30303030u);
    codes[3][w] = ((b[w] >> 4) & 0x0F0F0F0Fu) | ((hq[w] >> 2) & 0x30303030u);
  }
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    // int8 scale number 2k + i/2 of this half's eight.
    const uint32_t word = k < 2 ? sc8.x : sc8.y;
    const int shift = 8 * (((2 * k) & 3) + (i >> 1));
    const int sc = static_cast<int>(word << (24 - shift)) >> 24;
    scale[k] = static_cast<float>(sc);
  }
#pragma unroll
  for (int t = 0; t < NTOK; ++t) {
    const float* xt = xb + t * x_stride + 128 * n + 8 * i;
    const float* st = sb + t * s_stride + 16 * n + i;
    float block = 0.0f;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float4* xv = reinterpret_cast<const float4*>(xt + 32 * k);
      float group = Dot4Bytes(codes[k][0], xv[0], 0.0f);
      group = Dot4Bytes(codes[k][1], xv[1], group);
      group = Fma(-32.0f, st[4 * k], group);
      block = Fma(scale[k], group, block);
    }
    acc[t] = Fma(d, block, acc[t]);
  }
}

template <int TYPE, int NTOK>
__device__ __forceinline__ void MacBlock(const uint8_t* blk, int sub, const float* xb,
                                         const float* sb, int x_stride, int s_stride,
                                         float (&acc)[NTOK]) {
  if (TYPE == kTypeQ4K) {
    MacK4<false, NTOK>(blk, sub, xb, sb, x_stride, s_stride, acc);
  } else if (TYPE == kTypeQ5K) {
    MacK4<true, NTOK>(blk, sub, xb, sb, x_stride, s_stride, acc);
  } else {
    MacQ6K<NTOK>(blk, sub, xb, sb, x_stride, s_stride, acc);
  }
}

// Where the token columns of one kernel instance live: x[t] is the activation row
// of column t, y[t] the output row (the kernel adds part.y_offset + r).
template <int NTOK>
struct Columns {
  const float* x[NTOK];
  float* y[NTOK];
};

__device__ __forceinline__ float Silu(float v) { return v / (1.0f + expf(-v)); }

// One workgroup's share of the product.  kSwiGlu: x[t] points at a [gate | up] row
// of 2*cols values and the activation staged in LDS is silu(gate) * up, the step
// between an expert's two products (src/models/qwen35/decoder.cpp:547-549 of the
// reference).  part_shift is added to every part's row pointer (the byte offset
// of an expert's rows inside a 3-D tensor).
template <int TYPE, int NTOK, bool kSwiGlu>
__device__ __forceinline__ void GemvBody(const GemvParams& prm,
                                         const Columns<NTOK>& col,
                                         const size_t* part_shift, float* lds) {
  constexpr int kBlockBytes = BlockBytes(TYPE);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int bpp_log2 = static_cast<int>(prm.bpp_log2);
  const int bpp = 1 << bpp_log2;
  const int rpp = 8 >> bpp_log2;
  const int sub = lane & 7;
  const int blk_lane = (lane >> 3) & (bpp - 1);
  const int row_lane = lane >> (3 + bpp_log2);
  const int lanes_per_row = 8 << bpp_log2;

  const uint32_t nb = prm.launch.blocks_per_row;
  const uint32_t chunk = prm.chunk_blocks;
  const int x_stride = static_cast<int>(chunk) * 256;
  const int s_stride = static_cast<int>(chunk) * 32;
  float* lds_x = lds;
  float* lds_s = lds + NTOK * x_stride;

  // The rows this lane works on, one per visit.
  const uint8_t* row_ptr[kVisits];
  uint32_t y_index[kVisits];
  bool valid[kVisits];
  const uint32_t wg_row0 = blockIdx.x * prm.rows_per_wg;
#pragma unroll
  for (int v = 0; v < kVisits; ++v) {
    const uint32_t row = wg_row0 + (v * kWaves + wave) * rpp + row_lane;
    uint32_t rest = row;
    bool found = false;
    row_ptr[v] = prm.launch.part[0].rows;
    y_index[v] = 0;
#pragma unroll
    for (int p = 0; p < kMaxGemvParts; ++p) {
      if (p < static_cast<int>(prm.launch.n_parts) && !found) {
        const GemvPart part = prm.launch.part[p];
        if (rest < part.n_rows) {
          row_ptr[v] = part.rows + (part_shift != nullptr ? part_shift[p] : 0) +
                       static_cast<size_t>(rest) * prm.row_bytes;
          y_index[v] = part.y_offset + rest;
          found = true;
        } else {
          rest -= part.n_rows;
        }
      }
    }
    valid[v] = found && row < prm.launch.total_rows;
  }

  float acc[kVisits][NTOK];
#pragma unroll
  for (int v = 0; v < kVisits; ++v) {
#pragma unroll
    for (int t = 0; t < NTOK; ++t) acc[v][t] = 0.0f;
  }

  for (uint32_t c0 = 0; c0 < nb; c0 += chunk) {
    const uint32_t cb = min(chunk, nb - c0);
    if (c0 != 0) __syncthreads();
    // Stage x[t][c0*256 .. (c0+cb)*256) and the sums of every 8 values.
    const uint32_t units = cb * 32;  // groups of 8 values per token
    for (uint32_t u = tid; u < NTOK * units; u += kThreads) {
      const uint32_t t = u / units;
      const uint32_t g = u - t * units;
      const float4* src =
          reinterpret_cast<const float4*>(col.x[t] + static_cast<size_t>(c0) * 256 + g * 8);
      float4 v0 = src[0];
      float4 v1 = src[1];
      if (kSwiGlu) {
        const float4* up = reinterpret_cast<const float4*>(
            col.x[t] + prm.cols + static_cast<size_t>(c0) * 256 + g * 8);
        const float4 u0 = up[0];
        const float4 u1 = up[1];
        v0 = make_float4(Silu(v0.x) * u0.x, Silu(v0.y) * u0.y, Silu(v0.z) * u0.z,
                         Silu(v0.w) * u0.w);
        v1 = make_float4(Silu(v1.x) * u1.x, Silu(v1.y) * u1.y, Silu(v1.z) * u1.z,
                         Silu(v1.w) * u1.w);
      }
      float4* dst = reinterpret_cast<float4*>(lds_x + t * x_stride + g * 8);
      dst[0] = v0;
      dst[1] = v1;
      lds_s[t * s_stride + g] =
          ((v0.x + v0.y) + (v0.z + v0.w)) + ((v1.x + v1.y) + (v1.z + v1.w));
    }
    __syncthreads();

    const uint32_t passes = cb >> bpp_log2;
#pragma unroll
    for (int v = 0; v < kVisits; ++v) {
      if (!valid[v]) continue;
      const uint8_t* base =
          row_ptr[v] + static_cast<size_t>(c0 + blk_lane) * kBlockBytes;
      for (uint32_t it = 0; it < passes; ++it) {
        const uint32_t b = it * bpp + blk_lane;  // block within the chunk
        MacBlock<TYPE, NTOK>(base + static_cast<size_t>(it) * bpp * kBlockBytes, sub,
                             lds_x + b * 256, lds_s + b * 32, x_stride, s_stride,
                             acc[v]);
      }
    }
  }

#pragma unroll
  for (int v = 0; v < kVisits; ++v) {
#pragma unroll
    for (int t = 0; t < NTOK; ++t) {
      const float total = GroupSum(acc[v][t], lanes_per_row);
      if (valid[v] && (lane & (lanes_per_row - 1)) == 0) {
        col.y[t][y_index[v]] = total;
      }
    }
  }
}

// Dense product: token t reads x + t*cols and writes y + t*y_stride.
template <int TYPE, int NTOK>
__global__ __launch_bounds__(kThreads) void KquantGemvKernel(
    const GemvParams prm, const float* __restrict__ x, float* __restrict__ y) {
  extern __shared__ __align__(16) float lds[];
  Columns<NTOK> col;
#pragma unroll
  for (int t = 0; t < NTOK; ++t) {
    col.x[t] = x + static_cast<size_t>(t) * prm.cols;
    col.y[t] = y + static_cast<size_t>(t) * prm.launch.y_stride;
  }
  GemvBody<TYPE, NTOK, false>(prm, col, nullptr, lds);
}

// Expert product: blockIdx.y names a segment, i.e. one routed expert and up to
// four of the (token, slot) pairs that chose it.  The expert's rows are streamed
// once for all of them.  Column t reads the activation row of its pair (the
// token's x, or with kSwiGlu the pair's [gate | up] row) and writes the pair's
// output row.
template <int TYPE, int NTOK, bool kSwiGlu>
__device__ __forceinline__ void MoeSegmentBody(const GemvParams& prm,
                                               const MoeGemvArgs& moe,
                                               const MoeSegment& seg, float* lds) {
  Columns<NTOK> col;
#pragma unroll
  for (int t = 0; t < NTOK; ++t) {
    const uint32_t pair = static_cast<uint32_t>(seg.pair[t]);
    const size_t x_row = kSwiGlu ? pair : pair / moe.k;
    col.x[t] = moe.x + x_row * moe.x_row_floats;
    col.y[t] = moe.y + static_cast<size_t>(pair) * prm.launch.y_stride;
  }
  size_t shift[kMaxGemvParts];
#pragma unroll
  for (int p = 0; p < kMaxGemvParts; ++p) {
    shift[p] = static_cast<size_t>(seg.expert) * moe.expert_bytes[p];
  }
  GemvBody<TYPE, NTOK, kSwiGlu>(prm, col, shift, lds);
}

template <int TYPE, bool kSwiGlu>
__global__ __launch_bounds__(kThreads) void KquantMoeGemvKernel(const GemvParams prm,
                                                                const MoeGemvArgs moe) {
  extern __shared__ __align__(16) float lds[];
  const uint32_t s = blockIdx.y;
  if (s >= static_cast<uint32_t>(moe.tables->n_segments)) return;
  const MoeSegment seg = moe.segments[s];
  switch (seg.n_pairs) {
    case 1: MoeSegmentBody<TYPE, 1, kSwiGlu>(prm, moe, seg, lds); break;
    case 2: MoeSegmentBody<TYPE, 2, kSwiGlu>(prm, moe, seg, lds); break;
    case 3: MoeSegmentBody<TYPE, 3, kSwiGlu>(prm, moe, seg, lds); break;
    default: MoeSegmentBody<TYPE, 4, kSwiGlu>(prm, moe, seg, lds); break;
  }
}

template <int TYPE>
hipError_t LaunchTyped(const GemvParams& prm, const float* x, int tokens, float* y,
                       dim3 grid, size_t lds_bytes, hipStream_t stream) {
  switch (tokens) {
    case 1:
      hipLaunchKernelGGL((KquantGemvKernel<TYPE, 1>), grid, dim3(kThreads), lds_bytes,
                         stream, prm, x, y);
      break;
    case 2:
      hipLaunchKernelGGL((KquantGemvKernel<TYPE, 2>), grid, dim3(kThreads), lds_bytes,
                         stream, prm, x, y);
      break;
    case 3:
      hipLaunchKernelGGL((KquantGemvKernel<TYPE, 3>), grid, dim3(kThreads), lds_bytes,
                         stream, prm, x, y);
      break;
    case 4:
      hipLaunchKernelGGL((KquantGemvKernel<TYPE, 4>), grid, dim3(kThreads), lds_bytes,
                         stream, prm, x, y);
      break;
    default:
      return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

// Fills the launch geometry for `tokens` columns; returns the dynamic LDS bytes.
size_t PlanGemv(int type, const GemvLaunch& launch, int tokens, GemvParams* prm) {
  prm->launch = launch;
  const uint32_t nb = launch.blocks_per_row;
  prm->row_bytes = nb * BlockBytes(type);
  prm->cols = nb * 256;
  uint32_t bpp_log2 = 0;
  while (bpp_log2 < 3 && (nb & ((2u << bpp_log2) - 1)) == 0) ++bpp_log2;
  prm->bpp_log2 = bpp_log2;
  prm->rows_per_wg = kVisits * kWaves * (8u >> bpp_log2);
  // As many super-blocks of x per chunk as the LDS budget holds, in multiples of
  // 8 (every bpp divides 8), or the whole row when it fits.
  uint32_t chunk = kLdsBudget / (tokens * kLdsFloatsPerBlock * 4);
  chunk = chunk / 8 * 8;
  if (chunk >= nb) chunk = nb;
  prm->chunk_blocks = chunk;
  return static_cast<size_t>(tokens) * chunk * kLdsFloatsPerBlock * sizeof(float);
}

bool ValidLaunch(int type, const GemvLaunch& launch) {
  return BlockBytes(type) != 0 && launch.n_parts >= 1 &&
         launch.n_parts <= kMaxGemvParts && launch.blocks_per_row != 0;
}

template <int TYPE>
hipError_t LaunchMoeTyped(const GemvParams& prm, const MoeGemvArgs& moe, bool swiglu,
                          dim3 grid, size_t lds_bytes, hipStream_t stream) {
  if (swiglu) {
    hipLaunchKernelGGL((KquantMoeGemvKernel<TYPE, true>), grid, dim3(kThreads),
                       lds_bytes, stream, prm, moe);
  } else {
    hipLaunchKernelGGL((KquantMoeGemvKernel<TYPE, false>), grid, dim3(kThreads),
                       lds_bytes, stream, prm, moe);
  }
  return hipGetLastError();
}

}  // namespace

hipError_t LaunchGemv(int type, const GemvLaunch& launch, const float* x, int tokens,
                      float* y, hipStream_t stream) {
  if (!ValidLaunch(type, launch) || tokens < 1 || tokens > kMaxGemvTokens) {
    return hipErrorInvalidValue;
  }
  if (launch.total_rows == 0) return hipSuccess;
  GemvParams prm;
  const size_t lds_bytes = PlanGemv(type, launch, tokens, &prm);
  const dim3 grid((launch.total_rows + prm.rows_per_wg - 1) / prm.rows_per_wg);
  switch (type) {
    case kTypeQ4K: return LaunchTyped<kTypeQ4K>(prm, x, tokens, y, grid, lds_bytes, stream);
    case kTypeQ5K: return LaunchTyped<kTypeQ5K>(prm, x, tokens, y, grid, lds_bytes, stream);
    default: return LaunchTyped<kTypeQ6K>(prm, x, tokens, y, grid, lds_bytes, stream);
  }
}

hipError_t LaunchMoeGemv(int type, const GemvLaunch& launch, const MoeGemvArgs& moe,
                         bool swiglu, uint32_t max_segments, hipStream_t stream) {
  if (!ValidLaunch(type, launch)) return hipErrorInvalidValue;
  if (launch.total_rows == 0 || max_segments == 0) return hipSuccess;
  GemvParams prm;
  // Sized for the widest segment (four columns); narrower ones use less of it.
  const size_t lds_bytes = PlanGemv(type, launch, kMaxGemvTokens, &prm);
  const dim3 grid((launch.total_rows + prm.rows_per_wg - 1) / prm.rows_per_wg,
                  max_segments);
  switch (type) {
    case kTypeQ4K: return LaunchMoeTyped<kTypeQ4K>(prm, moe, swiglu, grid, lds_bytes, stream);
    case kTypeQ5K: return LaunchMoeTyped<kTypeQ5K>(prm, moe, swiglu, grid, lds_bytes, stream);
    default: return LaunchMoeTyped<kTypeQ6K>(prm, moe, swiglu, grid, lds_bytes, stream);
  }
}

}  // namespace gufo
