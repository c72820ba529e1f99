// Prefill projection on the matrix cores: C[t][r] = row r of a Q4_K matrix . a[t]
// for many tokens, a given as bf16.  This is GgufProjections::MatMul with
// tokens = m (src/models/qwen35/gguf_projections.cpp:239-286 of the reference), the
// shape the reference's NPU serves with its prefill GEMM (src/npu/gemm.hpp:99-105).
//
// The weights are dequantized in the kernel, in registers, to 16-bit operands and
// never written to memory:
//
//   weight[r][k] = d * sc_j * q - dmin * m_j          (j = sub-block of k)
//
//   * 16-bit means fp16, not bf16: rounding the dequantized weight to bf16 (8-bit
//     significand) costs 1.7e-3 relative L2 on this workload, above the 1e-3 this
//     kernel is held to; fp16 (11 bits) costs 1.4e-4.  The bf16 activations convert
//     to fp16 without loss (a pre-pass; magnitudes above 65504 saturate, below 2^-24
//     flush).
//   * The 4-bit code becomes the fp16 number 1024 + q by a byte permute
//     (0x6400 | q), and one fp32 fma with fp16 input and fp16 result
//     (v_fma_mix) produces the weight with a single rounding:
//     (1024 + q) * (d sc_j) - (1024 d sc_j + dmin m_j).  d sc_j is exact in fp32
//     (11 x 6 bits); the offset is rounded to fp32 once per sub-block, 2^-14 of a
//     quantization step.
//   * v_mfma_f32_32x32x16_f16 accumulates in fp32 over the whole row.
//
// Decomposition: a workgroup of 4 waves computes 128 tokens x 128 weight rows, two
// workgroups to a CU.  The activation tile of half a super-block (128 tokens x 128
// fp16 = 32 KB) goes from global memory straight into LDS (global_load_lds_dwordx4),
// double-buffered, one half ahead of the matrix cores; each wave owns 32 weight rows,
// reads their packed blocks into registers one super-block ahead, builds the operand
// fragments on the fly and multiplies them with the four 32-token tiles.
//
// The matrix instruction does not care which k a lane's 8 values belong to as long as
// both operands agree, so k is dealt to lanes the way the packed block likes it: of
// each 64 values (32 bytes of codes: low nibbles one sub-block, high nibbles the
// next), lane half u owns bytes 16 u .. 16 u + 15 - one 16-byte load - and its four
// steps take (low, first 8), (low, second 8), (high, first 8), (high, second 8).
//
// Workgroups are numbered so that each of the 8 XCDs (which take workgroups
// round-robin) owns a band of weight-row tiles - its slice of the packed matrix
// stays in that XCD's L2 - and walks the token tiles in order, so the workgroups
// running together share activation tiles.
#include <type_traits>

#include "kernels.hpp"
#include "kquant_common.hpp"

namespace gufo {
namespace {

typedef _Float16 Half8 __attribute__((ext_vector_type(8)));
typedef _Float16 Half2 __attribute__((ext_vector_type(2)));
typedef float Float16v __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(3))) void* LdsPointer;

constexpr int kGemmThreads = 256;
constexpr int kGemmWaves = kGemmThreads / 64;
constexpr int kTileTokens = 128;
constexpr int kTileRows = 32 * kGemmWaves;
constexpr int kRowBytes = 256;                            // one token's half super-block as fp16
constexpr int kStageBytes = kTileTokens * kRowBytes;      // 32 KB
constexpr int kCopiesPerWave = kStageBytes / 1024 / kGemmWaves;  // 1 KB per wave instruction
constexpr int kQ4Block = 144;
constexpr int kXcds = 8;

// ---- pre-pass: bf16 activations -> fp16, same [token][k] layout -------------------
__global__ __launch_bounds__(256) void PrepareActivations(const U32x4* __restrict__ a,
                                                          size_t octets,
                                                          U32x4* __restrict__ out) {
  const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= octets) return;
  const U32x4 raw = a[i];
  const uint32_t in[4] = {raw.x, raw.y, raw.z, raw.w};
  uint32_t packed[4];
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    float lo = __uint_as_float(in[p] << 16);
    float hi = __uint_as_float(in[p] & 0xFFFF0000u);
    lo = __builtin_fminf(__builtin_fmaxf(lo, -65504.0f), 65504.0f);
    hi = __builtin_fminf(__builtin_fmaxf(hi, -65504.0f), 65504.0f);
    const Half2 h = {static_cast<_Float16>(lo), static_cast<_Float16>(hi)};
    packed[p] = __builtin_bit_cast(uint32_t, h);
  }
  out[i] = U32x4{packed[0], packed[1], packed[2], packed[3]};
}

// ---- the product ------------------------------------------------------------------

// Where the 16-byte piece p (0..15) of token row t sits inside the row's 256 bytes of
// LDS: slot p ^ Swizzle(t).  Rows are one bank sweep apart, so the slot alone decides
// the banks; a wave reads piece (c | 2 u) of rows n = 0..31, and the xor makes the 16
// slots of rows n..n+15 (either u) and of rows n..n+7 (both u) all different.
__device__ __forceinline__ uint32_t Swizzle(uint32_t t) {
  return (t & 1u) | (((t >> 1) & 3u) << 2) | (((t >> 3) & 1u) << 1);
}

// One weight row's packed super-block as this lane reads it: lane (n, u) = (lane % 32,
// lane / 32) takes bytes 16 u .. 16 u + 15 of each 32 bytes of codes of row n.
struct PackedRow {
  U32x4 header;     // d, dmin, 12 scale bytes
  U32x4 codes[4];   // codes[p] = qs[32 p + 16 u .. +16)

  __device__ __forceinline__ void Load(const uint8_t* blk, uint32_t u) {
    header = Load16(blk);
#pragma unroll
    for (int p = 0; p < 4; ++p) codes[p] = Load16(blk + 16 + 32 * p + 16 * u);
  }
};

// Two 4-bit codes (bytes of `nibbles` picked by `selector`, each 0..15) dequantized to
// two fp16: the permute builds 0x6400 | q = 1024 + q, the fma runs in fp32.
__device__ __forceinline__ uint32_t DequantPair(uint32_t nibbles, uint32_t selector, float scale,
                                                float offset) {
  const uint32_t biased = __builtin_amdgcn_perm(0x64646464u, nibbles, selector);
  const Half2 h = __builtin_bit_cast(Half2, biased);
  Half2 r;
  r[0] = static_cast<_Float16>(__builtin_fmaf(static_cast<float>(h[0]), scale, offset));
  r[1] = static_cast<_Float16>(__builtin_fmaf(static_cast<float>(h[1]), scale, offset));
  return __builtin_bit_cast(uint32_t, r);
}

// Step s = 4 p + 2 high + half of a super-block: this lane's 8 dequantized values,
// k = 64 p + 32 high + 16 u + 8 half .. +8 of sub-block 2 p + high.
__device__ __forceinline__ Half8 WeightFragment(const PackedRow& row, int s,
                                                const float (&scale)[8],
                                                const float (&offset)[8]) {
  const int p = s >> 2;
  const int j = s >> 1;
  const uint32_t b0 = (s & 1) ? row.codes[p].z : row.codes[p].x;
  const uint32_t b1 = (s & 1) ? row.codes[p].w : row.codes[p].y;
  const uint32_t shift = (j & 1) ? 4 : 0;
  const uint32_t n0 = (b0 >> shift) & 0x0F0F0F0Fu;
  const uint32_t n1 = (b1 >> shift) & 0x0F0F0F0Fu;
  // perm selectors: result bytes [3..0] = [0x64, q_hi, 0x64, q_lo]; source 1 (nibbles)
  // holds bytes 0-3, source 0 (the constant) bytes 4-7.
  U32x4 out;
  out.x = DequantPair(n0, 0x04010400u, scale[j], offset[j]);  // codes 0, 1
  out.y = DequantPair(n0, 0x04030402u, scale[j], offset[j]);  // codes 2, 3
  out.z = DequantPair(n1, 0x04010400u, scale[j], offset[j]);  // codes 4, 5
  out.w = DequantPair(n1, 0x04030402u, scale[j], offset[j]);  // codes 6, 7
  return __builtin_bit_cast(Half8, out);
}

// The 16-byte piece of a token's half super-block that step s (0..7 within the half)
// reads for lane half u = 0; lane half 1 reads the piece 2 further.
__device__ __forceinline__ constexpr uint32_t StepPiece(int s) {
  return 8u * ((s >> 2) & 1) + 4u * ((s >> 1) & 1) + (s & 1);
}

struct GemmShape {
  uint32_t rows;
  uint32_t nb;           // super-blocks per row
  uint32_t tokens;
  uint32_t row_tiles;
  uint32_t token_tiles;
  uint32_t band;         // weight-row tiles per band
  uint32_t per_xcd;      // workgroups each XCD takes
  uint32_t total;        // bands * token_tiles * band
};

// Waits until at most `pending` of this wave's vector-memory operations are
// outstanding (they retire in order).
template <int kPending>
__device__ __forceinline__ void WaitVectorMemory() {
  if constexpr (kPending == 0) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  } else {
    static_assert(kPending == 5, "one packed row is 5 loads");
    asm volatile("s_waitcnt vmcnt(5)" ::: "memory");
  }
}

// The workgroup barrier alone.  __syncthreads() adds a release fence that drains every
// vector-memory operation of the wave, the weight prefetch included; here the waits
// that matter are explicit: each wave waits for its own copies into LDS before the
// barrier, and has consumed its LDS reads of the other stage by then.
__device__ __forceinline__ void TileBarrier() {
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// Two workgroups share a CU (2 x 64 KB of LDS, 2 waves per SIMD).
__global__ __launch_bounds__(kGemmThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void
KquantGemmKernel(const uint8_t* __restrict__ w, const uint8_t* __restrict__ a16,
                 float* __restrict__ c, GemmShape shape) {
  extern __shared__ __align__(1024) uint8_t stages[];  // 2 x kStageBytes
  // Workgroup -> tile.  XCD x takes positions [x per_xcd, (x+1) per_xcd) of the order
  // (band, token tile, row tile within the band).
  const uint32_t position = (blockIdx.x % kXcds) * shape.per_xcd + blockIdx.x / kXcds;
  if (position >= shape.total) return;
  const uint32_t within = position % shape.band;
  const uint32_t token_tile = (position / shape.band) % shape.token_tiles;
  const uint32_t row_tile = position / (shape.band * shape.token_tiles) * shape.band + within;
  if (row_tile >= shape.row_tiles) return;

  const uint32_t tid = threadIdx.x;
  const uint32_t lane = tid & 63;
  const uint32_t wave = tid >> 6;
  const uint32_t n = lane & 31;
  const uint32_t u = lane >> 5;
  const uint32_t nb = shape.nb;
  const uint32_t token0 = token_tile * kTileTokens;
  const uint32_t row = row_tile * kTileRows + wave * 32 + n;
  const bool row_valid = row < shape.rows;
  const uint8_t* row_ptr = w + static_cast<size_t>(row_valid ? row : shape.rows - 1) * nb * kQ4Block;

  // Copies global -> LDS.  Wave instruction i of this wave fills the 1 KB holding token
  // rows 4 c .. 4 c + 3 (c = wave * kCopiesPerWave + i); lane l supplies LDS slot l % 16
  // of row 4 c + l / 16, that is piece slot ^ Swizzle(row) of the token's half block.
  // Rows past the last token repeat it; their products are not stored.
  uint32_t copy_piece[kCopiesPerWave];  // in 16-byte pieces from a16, half block 0
#pragma unroll
  for (int i = 0; i < kCopiesPerWave; ++i) {
    const uint32_t t = 4 * (wave * kCopiesPerWave + i) + (lane >> 4);
    const uint32_t token = min(token0 + t, shape.tokens - 1);
    copy_piece[i] = token * (nb * 32) + ((lane & 15u) ^ Swizzle(t & 15u));
  }
  auto copy_stage = [&](uint32_t half_block, uint32_t stage) {
#pragma unroll
    for (int i = 0; i < kCopiesPerWave; ++i) {
      const uint8_t* src = a16 + (static_cast<size_t>(copy_piece[i]) + half_block * 16) * 16;
      uint8_t* dst = stages + stage * kStageBytes + (wave * kCopiesPerWave + i) * 1024;
      __builtin_amdgcn_global_load_lds(src, (LdsPointer)dst, 16, 0, 0);
    }
  };

  Float16v acc[4];
#pragma unroll
  for (int m = 0; m < 4; ++m) {
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[m][i] = 0.0f;
  }

  copy_stage(0, 0);
  PackedRow next;
  next.Load(row_ptr, u);

  // This lane's activation fragment of step s, token tile m: piece StepPiece(s) | 2 u of
  // row 32 m + n, at slot StepPiece(s) ^ flip.
  const uint32_t flip = Swizzle(n & 15u) ^ (u << 1);
  const uint32_t read_base = n * kRowBytes;

  PackedRow cur;
  float scale[8];
  float offset[8];

  // One half super-block: 8 steps on `stage`, both operands one step ahead of the
  // matrix cores - while step s multiplies, the activation fragments of step s + 1 are
  // on their way from LDS and its weight fragment is being dequantized.
  auto multiply_half = [&](uint32_t stage, auto half_tag) {
    constexpr int kHalf = decltype(half_tag)::value;
    const uint8_t* tile = stages + stage * kStageBytes + read_base;
    Half8 af[4];
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      af[m] = *reinterpret_cast<const Half8*>(tile + ((StepPiece(0) ^ flip) << 4) +
                                              m * 32 * kRowBytes);
    }
    Half8 bf = WeightFragment(cur, 8 * kHalf, scale, offset);
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      Half8 af_next[4];
      Half8 bf_next;
      if (s + 1 < 8) {
        const uint8_t* at = tile + ((StepPiece(s + 1) ^ flip) << 4);
#pragma unroll
        for (int m = 0; m < 4; ++m) {
          af_next[m] = *reinterpret_cast<const Half8*>(at + m * 32 * kRowBytes);
        }
      }
      // Nothing moves across: the reads of step s + 1 are issued before step s multiplies.
      __builtin_amdgcn_sched_barrier(0);
      if (s + 1 < 8) bf_next = WeightFragment(cur, 8 * kHalf + s + 1, scale, offset);
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[m], bf, acc[m], 0, 0, 0);
      }
      // Within the step: each matrix instruction followed by a quarter of the next
      // weight fragment's dequantization.
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      if (s + 1 < 8) {
#pragma unroll
        for (int m = 0; m < 4; ++m) af[m] = af_next[m];
        bf = bf_next;
      }
    }
  };

  for (uint32_t b = 0; b < nb; ++b) {
    const bool more = b + 1 < nb;
    // First half.  Everything in flight (stage 0's copies, this block's weights) has
    // landed, for every wave, and every wave is done reading stage 1.
    WaitVectorMemory<0>();
    TileBarrier();
    cur = next;
    copy_stage(2 * b + 1, 1);
    __builtin_amdgcn_sched_barrier(0);  // the wait below counts on this issue order
    if (more) next.Load(row_ptr + static_cast<size_t>(b + 1) * kQ4Block, u);
    const float d = HalfBitsToFloat(cur.header.x & 0xFFFFu);
    const float dmin = HalfBitsToFloat(cur.header.x >> 16);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      uint32_t sc, mn;
      ScaleMinK4(cur.header.y, cur.header.z, cur.header.w, j, &sc, &mn);
      scale[j] = d * static_cast<float>(sc);
      offset[j] = __builtin_fmaf(-dmin, static_cast<float>(mn), -1024.0f * scale[j]);
    }
    multiply_half(0, std::integral_constant<int, 0>{});

    // Second half.  Stage 1's copies were issued before the next block's weights, which
    // may stay in flight.
    if (more) {
      WaitVectorMemory<5>();
    } else {
      WaitVectorMemory<0>();
    }
    TileBarrier();
    if (more) copy_stage(2 * b + 2, 0);
    multiply_half(1, std::integral_constant<int, 1>{});
  }

  // Accumulator register i of tile m holds token 8 (i/4) + 4 u + i%4 and weight row n.
  if (row_valid) {
#pragma unroll
    for (int m = 0; m < 4; ++m) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const uint32_t t = token0 + m * 32 + 8 * (i >> 2) + 4 * u + (i & 3);
        if (t < shape.tokens) c[static_cast<size_t>(t) * shape.rows + row] = acc[m][i];
      }
    }
  }
}

}  // namespace

size_t GemmWorkspaceBytes(size_t tokens, uint32_t blocks_per_row) {
  return tokens * blocks_per_row * 256 * sizeof(_Float16);
}

hipError_t LaunchGemmQ4K(const uint8_t* w, uint32_t rows, uint32_t blocks_per_row,
                         const uint16_t* a_bf16, size_t tokens, void* workspace, float* c,
                         hipStream_t stream) {
  if (rows == 0 || tokens == 0) return hipSuccess;
  // Activation pieces are addressed with 32 bits.
  if (blocks_per_row == 0 || tokens > 0x7FFFFFFFull / (32ull * blocks_per_row)) {
    return hipErrorInvalidValue;
  }
  const size_t octets = tokens * blocks_per_row * 32;
  hipLaunchKernelGGL(PrepareActivations, dim3(static_cast<uint32_t>((octets + 255) / 256)),
                     dim3(256), 0, stream, reinterpret_cast<const U32x4*>(a_bf16), octets,
                     static_cast<U32x4*>(workspace));
  hipError_t status = hipGetLastError();
  if (status != hipSuccess) return status;

  constexpr size_t lds_bytes = 2 * kStageBytes;
  GemmShape shape;
  shape.rows = rows;
  shape.nb = blocks_per_row;
  shape.tokens = static_cast<uint32_t>(tokens);
  shape.row_tiles = (rows + kTileRows - 1) / kTileRows;
  shape.token_tiles = static_cast<uint32_t>((tokens + kTileTokens - 1) / kTileTokens);
  shape.band = (shape.row_tiles + kXcds - 1) / kXcds;
  const uint32_t bands = (shape.row_tiles + shape.band - 1) / shape.band;
  shape.total = bands * shape.token_tiles * shape.band;
  shape.per_xcd = (shape.total + kXcds - 1) / kXcds;
  hipLaunchKernelGGL(KquantGemmKernel, dim3(shape.per_xcd * kXcds), dim3(kGemmThreads), lds_bytes,
                     stream, w, static_cast<const uint8_t*>(workspace), c, shape);
  return hipGetLastError();
}

}  // namespace gufo
