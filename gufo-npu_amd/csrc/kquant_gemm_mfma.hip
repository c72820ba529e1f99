// Prefill projection on the matrix cores: C[t][r] = row r of a Q4_K matrix . a[t]
// for many tokens, a given as bf16.  This is GgufProjections::MatMul with
// tokens = m (src/models/qwen35/gguf_projections.cpp:239-286 of the reference), the
// shape the reference's NPU serves with its prefill GEMM (src/npu/gemm.hpp:99-105).
//
// The weights are never dequantized to memory.  What the matrix cores multiply are
// exact 16-bit operands:
//
//   weight[r][k] = d * (sc_j * q) - dmin * m_j        (j = sub-block of k)
//
//   * sc_j * q is an integer <= 63 * 15 = 945, exact in fp16 (11-bit significand) -
//     it would not be in bf16 (8 bits), and rounding the dequantized weight itself to
//     bf16 costs 1.7e-3 relative L2 on this workload, above the 1e-3 this kernel is
//     held to.  The bf16 activations convert to fp16 without loss (8-bit significand;
//     magnitudes below 2^-24 flush, far below anything that matters).
//   * v_mfma_f32_32x32x16_f16 accumulates sum_k (sc*q) * a over one super-block (16
//     instructions) in fp32; the block scale d, one value per weight row = per lane
//     of the accumulator layout, is applied once per super-block with one fma per
//     accumulator register.
//   * The minimum term needs sum over each sub-block of a, S[t][j].  A pre-pass
//     writes the activations as fp16 together with S split in two fp16 halves
//     (hi + lo, 22 bits), so the term is one more MFMA per super-block: K = 16 =
//     8 sub-blocks x {hi, lo} against the 6-bit minimums m_j, scaled by dmin.
//
// Decomposition: a workgroup of 4 waves computes 128 tokens x 128 weight rows.  The
// activation tile of one super-block (128 x 272 fp16) is staged in LDS and shared;
// each wave owns 32 weight rows, reads their packed blocks straight into registers
// one super-block ahead, converts them to operand fragments on the fly (a byte
// permute and one packed fp16 fma per two weights) and multiplies them with the four
// 32-token tiles.
#include "kernels.hpp"
#include "kquant_common.hpp"

namespace gufo {
namespace {

typedef _Float16 Half8 __attribute__((ext_vector_type(8)));
typedef _Float16 Half2 __attribute__((ext_vector_type(2)));
typedef float Float16v __attribute__((ext_vector_type(16)));

constexpr int kGemmThreads = 256;
constexpr int kTileTokens = 128;  // BM
constexpr int kTileRows = 128;    // BN
constexpr int kBlockHalfs = 272;  // 256 activations + 8 sub-block sums hi + 8 lo
constexpr int kLdsPitch = 280;    // halfs per token row in LDS: 560 B, an odd number of
                                  // 16-byte units, so 8 consecutive rows hit 8 bank groups
constexpr int kQ4Block = 144;

// ---- pre-pass: bf16 activations -> fp16 + sub-block sums ------------------------
// out[t][b][0..255] = a[t][256 b + i] as fp16, out[t][b][256 + j] = hi(S_j),
// out[t][b][264 + j] = lo(S_j), S_j = sum of the 32 activations of sub-block j (fp32).
// One wave per (token, super-block); lane l converts values 4l..4l+3.
__global__ __launch_bounds__(256) void PrepareActivations(const uint16_t* __restrict__ a,
                                                          uint32_t tokens, uint32_t nb,
                                                          _Float16* __restrict__ out) {
  const uint32_t item = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= tokens * nb) return;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t t = item / nb;
  const uint32_t b = item - t * nb;
  const U32x2 raw =
      *reinterpret_cast<const U32x2*>(a + (static_cast<size_t>(t) * nb + b) * 256 + 4 * lane);
  float v[4];
  v[0] = __uint_as_float(raw.x << 16);
  v[1] = __uint_as_float(raw.x & 0xFFFF0000u);
  v[2] = __uint_as_float(raw.y << 16);
  v[3] = __uint_as_float(raw.y & 0xFFFF0000u);
  _Float16* dst = out + (static_cast<size_t>(t) * nb + b) * kBlockHalfs;
  Half2 h01 = {static_cast<_Float16>(v[0]), static_cast<_Float16>(v[1])};
  Half2 h23 = {static_cast<_Float16>(v[2]), static_cast<_Float16>(v[3])};
  U32x2 packed = {__builtin_bit_cast(uint32_t, h01), __builtin_bit_cast(uint32_t, h23)};
  *reinterpret_cast<U32x2*>(dst + 4 * lane) = packed;
  // Sub-block j = lanes 8j..8j+7: sum in a fixed order.
  float s = (v[0] + v[1]) + (v[2] + v[3]);
  s += __shfl_xor(s, 1, 64);
  s += __shfl_xor(s, 2, 64);
  s += __shfl_xor(s, 4, 64);
  if ((lane & 7) == 0) {
    const _Float16 hi = static_cast<_Float16>(s);
    const _Float16 lo = static_cast<_Float16>(s - static_cast<float>(hi));
    dst[256 + (lane >> 3)] = hi;
    dst[264 + (lane >> 3)] = lo;
  }
}

// ---- the product ------------------------------------------------------------------

// One weight row's packed super-block as this lane reads it.  Lane (n, u) = (lane%32,
// lane/32) owns, of each MFMA step s (16 k-values), the 8 values k = 16 s + 8 u .. +8
// of row n: sub-block s/2, bytes 32 (s/4) + 16 (s%2) + 8 u .. +8 of qs, low nibbles
// for even s/2 and high nibbles for odd.  Over a block that is 8 pieces of 8 bytes.
struct PackedRow {
  U32x4 header;     // d, dmin, 12 scale bytes
  U32x2 piece[8];   // piece[2 p + h] = qs[32 p + 16 h + 8 u .. +8)

  __device__ __forceinline__ void Load(const uint8_t* blk, uint32_t u) {
    header = Load16(blk);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      piece[i] = *reinterpret_cast<const U32x2*>(blk + 16 + 32 * (i >> 1) + 16 * (i & 1) + 8 * u);
    }
  }
  __device__ __forceinline__ void Clear() {
    header = U32x4{0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < 8; ++i) piece[i] = U32x2{0, 0};
  }
};

// Two 4-bit codes (bytes b0, b1 of `nibbles`, each 0..15) times the integer scale, as
// two exact fp16: (1024 + q) * sc - 1024 * sc with 0x6400 | q = 1024 + q.
__device__ __forceinline__ uint32_t ScaledPair(uint32_t nibbles, uint32_t selector,
                                               Half2 scale, Half2 offset) {
  const uint32_t biased = __builtin_amdgcn_perm(0x64646464u, nibbles, selector);
  const Half2 h = __builtin_bit_cast(Half2, biased);
  const Half2 r = __builtin_elementwise_fma(h, scale, offset);
  return __builtin_bit_cast(uint32_t, r);
}

// The B operand of step s: 8 values (sc_j * q) as fp16 for this lane.
__device__ __forceinline__ Half8 WeightFragment(const PackedRow& row, int s,
                                                const uint32_t (&sc)[8]) {
  const int j = s >> 1;                       // sub-block
  const U32x2 bytes = row.piece[2 * (s >> 2) + (s & 1)];
  const uint32_t shift = (j & 1) ? 4 : 0;
  const uint32_t n0 = (bytes.x >> shift) & 0x0F0F0F0Fu;
  const uint32_t n1 = (bytes.y >> shift) & 0x0F0F0F0Fu;
  const _Float16 scale = static_cast<_Float16>(static_cast<float>(sc[j]));
  const Half2 scale2 = {scale, scale};
  const _Float16 off = static_cast<_Float16>(-1024.0f * static_cast<float>(sc[j]));
  const Half2 off2 = {off, off};
  // perm selectors: result bytes [3..0] = [0x64, q_hi, 0x64, q_lo]; source 1 (nibbles)
  // holds bytes 0-3, source 0 (the constant) bytes 4-7.
  U32x4 out;
  out.x = ScaledPair(n0, 0x04010400u, scale2, off2);  // codes 0, 1
  out.y = ScaledPair(n0, 0x04030402u, scale2, off2);  // codes 2, 3
  out.z = ScaledPair(n1, 0x04010400u, scale2, off2);  // codes 4, 5
  out.w = ScaledPair(n1, 0x04030402u, scale2, off2);  // codes 6, 7
  return __builtin_bit_cast(Half8, out);
}

__global__ __launch_bounds__(kGemmThreads) void KquantGemmKernel(
    const uint8_t* __restrict__ w, uint32_t rows, uint32_t nb,
    const _Float16* __restrict__ a16, uint32_t tokens, float* __restrict__ c) {
  extern __shared__ __align__(16) _Float16 tile[];  // kTileTokens x kLdsPitch
  const uint32_t tid = threadIdx.x;
  const uint32_t lane = tid & 63;
  const uint32_t wave = tid >> 6;
  const uint32_t n = lane & 31;
  const uint32_t u = lane >> 5;
  const uint32_t token0 = blockIdx.y * kTileTokens;
  const uint32_t row = blockIdx.x * kTileRows + wave * 32 + n;
  const bool row_valid = row < rows;
  const uint8_t* row_ptr = w + static_cast<size_t>(row_valid ? row : 0) * nb * kQ4Block;

  Float16v acc[4];
#pragma unroll
  for (int m = 0; m < 4; ++m) {
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[m][i] = 0.0f;
  }

  PackedRow next;
  if (row_valid) {
    next.Load(row_ptr, u);
  } else {
    next.Clear();
  }

  for (uint32_t b = 0; b < nb; ++b) {
    const PackedRow cur = next;
    if (b + 1 < nb && row_valid) next.Load(row_ptr + static_cast<size_t>(b + 1) * kQ4Block, u);

    // Stage the activation tile of this super-block: 128 rows of 272 halfs = 34 pieces
    // of 16 bytes per row.
    __syncthreads();
    for (uint32_t i = tid; i < kTileTokens * 34; i += kGemmThreads) {
      const uint32_t t = i / 34;
      const uint32_t piece = i - t * 34;
      U32x4 v = {0, 0, 0, 0};
      if (token0 + t < tokens) {
        v = *reinterpret_cast<const U32x4*>(
            a16 + (static_cast<size_t>(token0 + t) * nb + b) * kBlockHalfs + piece * 8);
      }
      *reinterpret_cast<U32x4*>(tile + t * kLdsPitch + piece * 8) = v;
    }
    __syncthreads();

    const float d = HalfBitsToFloat(cur.header.x & 0xFFFFu);
    const float dmin = HalfBitsToFloat(cur.header.x >> 16);
    uint32_t sc[8];
    uint32_t mn[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      ScaleMinK4(cur.header.y, cur.header.z, cur.header.w, j, &sc[j], &mn[j]);
    }

    Float16v part[4];
#pragma unroll
    for (int m = 0; m < 4; ++m) {
#pragma unroll
      for (int i = 0; i < 16; ++i) part[m][i] = 0.0f;
    }
#pragma unroll
    for (int s = 0; s < 16; ++s) {
      const Half8 bf = WeightFragment(cur, s, sc);
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        const Half8 af = *reinterpret_cast<const Half8*>(tile + (m * 32 + n) * kLdsPitch +
                                                         16 * s + 8 * u);
        part[m] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, bf, part[m], 0, 0, 0);
      }
    }
    // The minimum term: k = 8 u + j pairs m_j with hi(S_j) (u = 0) or lo(S_j) (u = 1).
    Half8 mins;
#pragma unroll
    for (int j = 0; j < 8; ++j) mins[j] = static_cast<_Float16>(static_cast<float>(mn[j]));
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const Half8 sums = *reinterpret_cast<const Half8*>(tile + (m * 32 + n) * kLdsPitch + 256 +
                                                         8 * u);
      Float16v zero;
#pragma unroll
      for (int i = 0; i < 16; ++i) zero[i] = 0.0f;
      const Float16v min_part = __builtin_amdgcn_mfma_f32_32x32x16_f16(sums, mins, zero, 0, 0, 0);
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        acc[m][i] = __builtin_fmaf(d, part[m][i], acc[m][i]);
        acc[m][i] = __builtin_fmaf(-dmin, min_part[i], acc[m][i]);
      }
    }
  }

  // Accumulator register i of tile m holds token 8 (i/4) + 4 u + i%4 and weight row n.
  if (row_valid) {
#pragma unroll
    for (int m = 0; m < 4; ++m) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const uint32_t t = token0 + m * 32 + 8 * (i >> 2) + 4 * u + (i & 3);
        if (t < tokens) c[static_cast<size_t>(t) * rows + row] = acc[m][i];
      }
    }
  }
}

}  // namespace

size_t GemmWorkspaceBytes(size_t tokens, uint32_t blocks_per_row) {
  return tokens * blocks_per_row * kBlockHalfs * sizeof(_Float16);
}

hipError_t LaunchGemmQ4K(const uint8_t* w, uint32_t rows, uint32_t blocks_per_row,
                         const uint16_t* a_bf16, size_t tokens, void* workspace, float* c,
                         hipStream_t stream) {
  if (rows == 0 || tokens == 0) return hipSuccess;
  if (blocks_per_row == 0 || tokens > 0x7FFFFFFFull / blocks_per_row) {
    return hipErrorInvalidValue;
  }
  _Float16* a16 = static_cast<_Float16*>(workspace);
  const uint32_t items = static_cast<uint32_t>(tokens) * blocks_per_row;
  hipLaunchKernelGGL(PrepareActivations, dim3((items + 3) / 4), dim3(256), 0, stream, a_bf16,
                     static_cast<uint32_t>(tokens), blocks_per_row, a16);
  hipError_t status = hipGetLastError();
  if (status != hipSuccess) return status;
  const size_t lds_bytes = static_cast<size_t>(kTileTokens) * kLdsPitch * sizeof(_Float16);
  static bool allowed = false;
  if (!allowed) {
    status = hipFuncSetAttribute(reinterpret_cast<const void*>(KquantGemmKernel),
                                 hipFuncAttributeMaxDynamicSharedMemorySize,
                                 static_cast<int>(lds_bytes));
    if (status != hipSuccess) return status;
    allowed = true;
  }
  const dim3 grid((rows + kTileRows - 1) / kTileRows,
                  static_cast<uint32_t>((tokens + kTileTokens - 1) / kTileTokens));
  hipLaunchKernelGGL(KquantGemmKernel, grid, dim3(kGemmThreads), lds_bytes, stream, w, rows,
                     blocks_per_row, a16, static_cast<uint32_t>(tokens), c);
  return hipGetLastError();
}

}  // namespace gufo
