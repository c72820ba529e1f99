// Prefill projection on the matrix cores: C[t][r] = row r of a quantized matrix . a[t]
// for many tokens, a given as bf16.  This is GgufProjections::MatMul with
// tokens = m (src/models/qwen35/gguf_projections.cpp:239-286 of the reference), the
// shape the reference's NPU serves with its prefill GEMM (src/npu/gemm.hpp:99-105).
//
// Two launches.  A pre-pass turns both operands into fp16 once per call; the product
// kernel then only moves 16-bit operands and issues matrix instructions, whatever the
// row type was (Q4_K, Q5_K, Q6_K, Q8_0).  For Q4_K, the type of the prefill
// configuration, the pre-pass is written around the packed block:
//
//   weight[r][k] = d * sc_j * q - dmin * m_j          (j = sub-block of k)
//
//   * 16-bit means fp16, not bf16: rounding the dequantized weight to bf16 (8-bit
//     significand) costs 1.7e-3 relative L2 on this workload, above the 1e-3 this
//     kernel is held to; fp16 (11 bits) costs 1.4e-4.  The bf16 activations convert
//     to fp16 without loss (magnitudes above 65504 saturate, below 2^-24 flush).
//   * The 4-bit code becomes the fp16 number 1024 + q by a byte permute
//     (0x6400 | q), and one fp32 fma with fp16 input and fp16 result
//     (v_fma_mix) produces the weight with a single rounding:
//     (1024 + q) * (d sc_j) - (1024 d sc_j + dmin m_j).  d sc_j is exact in fp32
//     (11 x 6 bits); the offset is rounded to fp32 once per sub-block, 2^-14 of a
//     quantization step.
//   * v_mfma_f32_32x32x16_f16 accumulates in fp32 over the whole row.
//   * Dequantizing once instead of inside the product kernel: with 4096 tokens every
//     weight is used by 32 token tiles, and built in registers each time (the first
//     version of this kernel) the conversion took as many issue cycles as the matrix
//     instructions themselves: 124-133 us.  Written once as fp16 (25 MB for 6144 x 2048,
//     5 us) the product kernel has no arithmetic left but the matrix instructions.
//
// Decomposition: one persistent workgroup of 4 waves per CU - one wave per SIMD - walks
// its share of the 128-token x 256-row tiles.  Each wave owns 64 weight rows (two groups
// of 32) and multiplies them with the four 32-token tiles: 8 matrix instructions per
// step of 16 k for 4 LDS reads and 2 global loads.  (Eight waves of 32 rows each, two per
// SIMD, read every activation fragment from LDS twice as often: 109 us against 101.)
// The activations of half a super-block (128 tokens x 128 fp16 = 32 KB, a "stage") go
// from global memory straight into LDS (global_load_lds_dwordx4) into a ring of four
// stages, three halves ahead of the matrix cores - across tile boundaries too, so the
// copies of a tile's first halves and the stores of the previous tile's results overlap.
// The weight operand of a half (2 groups x 8 steps x 16 bytes per lane) comes from the
// pre-pass's array straight into registers, one half ahead.
//
// The matrix instruction does not care which k a lane's 8 values belong to as long as
// both operands agree, so k is dealt to lanes the way the packed block likes it: of
// each 64 values (32 bytes of codes: low nibbles one sub-block, high nibbles the
// next), lane half u owns bytes 16 u .. 16 u + 15 - one 16-byte load - and its four
// steps take (low, first 8), (low, second 8), (high, first 8), (high, second 8).  The
// pre-pass stores each (32 rows, super-block, step) as the 64 lanes' 16 bytes in lane
// order, 1 KB, so the product kernel's loads are whole cache lines.
//
// Tiles are ordered (band of row tiles, token tile, row tile within the band) and the
// order is cut in 8 pieces, one per XCD (workgroups go to XCDs round-robin): an XCD's
// slice of the fp16 matrix (3 of the 24 row tiles, 3 MB) stays in its L2 while it walks
// the token tiles, and the workgroups running together share activation tiles.
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
constexpr int kWaveGroups = 2;                            // groups of 32 weight rows per wave
constexpr int kTileGroups = kWaveGroups * kGemmWaves;     // groups of 32 weight rows per tile
constexpr int kTileTokens = 128;
constexpr int kTileRows = 32 * kTileGroups;
constexpr int kRowBytes = 256;                            // one token's half super-block as fp16
constexpr int kStageBytes = kTileTokens * kRowBytes;      // 32 KB
constexpr int kStages = 4;                                // the copies run kStages - 1 halves ahead
constexpr int kCopiesPerWave = kStageBytes / 1024 / kGemmWaves;  // 1 KB per wave instruction
constexpr int kStepsPerHalf = 8;
constexpr int kStepBytes = 64 * 16;                       // one step's fragments of 32 rows
constexpr int kHalfBytes = kStepsPerHalf * kStepBytes;    // 8 KB per 32 rows and half super-block
constexpr int kXcds = 8;

// ---- pre-pass ---------------------------------------------------------------------

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

// scale = d sc_j and offset = -(1024 d sc_j + dmin m_j) of sub-block j.
__device__ __forceinline__ void SubBlockAffine(const U32x4& header, int j, float* scale,
                                               float* offset) {
  const float d = HalfBitsToFloat(header.x & 0xFFFFu);
  const float dmin = HalfBitsToFloat(header.x >> 16);
  uint32_t sc, mn;
  ScaleMinK4(header.y, header.z, header.w, j, &sc, &mn);
  *scale = d * static_cast<float>(sc);
  *offset = __builtin_fmaf(-dmin, static_cast<float>(mn), -1024.0f * *scale);
}

// Step s = 4 p + q, q = 2 high + half, of a super-block: this lane's 8 dequantized
// values, k = 64 p + 32 high + 16 u + 8 half .. +8, of sub-block j = 2 p + high, whose
// scale and offset the caller passes.  `codes` = qs[32 p + 16 u .. +16): the lane's 16
// bytes of the 64 values 64 p .. 64 p + 63.
__device__ __forceinline__ U32x4 WeightFragment(const U32x4& codes, int q, float scale,
                                                float offset) {
  const uint32_t b0 = (q & 1) ? codes.z : codes.x;
  const uint32_t b1 = (q & 1) ? codes.w : codes.y;
  const uint32_t shift = (q & 2) ? 4 : 0;
  const uint32_t n0 = (b0 >> shift) & 0x0F0F0F0Fu;
  const uint32_t n1 = (b1 >> shift) & 0x0F0F0F0Fu;
  // perm selectors: result bytes [3..0] = [0x64, q_hi, 0x64, q_lo]; source 1 (nibbles)
  // holds bytes 0-3, source 0 (the constant) bytes 4-7.
  U32x4 out;
  out.x = DequantPair(n0, 0x04010400u, scale, offset);  // codes 0, 1
  out.y = DequantPair(n0, 0x04030402u, scale, offset);  // codes 2, 3
  out.z = DequantPair(n1, 0x04010400u, scale, offset);  // codes 4, 5
  out.w = DequantPair(n1, 0x04030402u, scale, offset);  // codes 6, 7
  return out;
}

// The other row types: the 8 weights k0 .. k0 + 7 (k0 a multiple of 8) of the 256 values
// that start at `blk`, in fp32.  Eight such neighbours share a sub-block in every format,
// and their codes are 8 consecutive bytes.  Each weight is exact in fp32 or rounded once
// (the K-quant formulas of src/core/quant.cpp:61-133 of the reference, Q8_0 of :22-31).
template <int TYPE>
__device__ __forceinline__ void DequantEight(const uint8_t* blk, uint32_t k0, float (&out)[8]) {
  if constexpr (TYPE == kTypeQ5K) {
    // d, dmin | 12 scale bytes | qh[32] | qs[128]: value k of the 64 values 64 p .. is the
    // low (k % 64 < 32) or high nibble of qs[32 p + k % 32] plus 16 x bit (2 p + high) of
    // qh[k % 32].
    const uint32_t p = k0 >> 6;
    const uint32_t high = (k0 >> 5) & 1u;
    const uint32_t l = k0 & 31u;
    const U32x4 header = Load16(blk);
    float scale, offset;
    {
      const float d = HalfBitsToFloat(header.x & 0xFFFFu);
      const float dmin = HalfBitsToFloat(header.x >> 16);
      uint32_t sc, mn;
      ScaleMinK4(header.y, header.z, header.w, static_cast<int>(2 * p + high), &sc, &mn);
      scale = d * static_cast<float>(sc);
      offset = -dmin * static_cast<float>(mn);
    }
    const U32x2 qs = Load8Align2(blk + 48 + 32 * p + l);
    const U32x2 qh = Load8Align2(blk + 16 + l);
    const uint32_t codes[2] = {qs.x >> (4 * high), qs.y >> (4 * high)};
    const uint32_t fifth[2] = {qh.x >> (2 * p + high), qh.y >> (2 * p + high)};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t q = ((codes[i >> 2] >> (8 * (i & 3))) & 15u) +
                         (((fifth[i >> 2] >> (8 * (i & 3))) & 1u) << 4);
      out[i] = __builtin_fmaf(static_cast<float>(q), scale, offset);
    }
  } else if constexpr (TYPE == kTypeQ6K) {
    // ql[128] | qh[64] | int8 scales[16] | d: of each 128 values, quarter c (32 values)
    // takes the low (c < 2) or high nibble of ql[64 n + 32 (c & 1) + l] and bits 2 c,
    // 2 c + 1 of qh[32 n + l]; scale 8 n + 2 c + l / 16.
    const uint32_t n = k0 >> 7;
    const uint32_t c = (k0 >> 5) & 3u;
    const uint32_t l = k0 & 31u;
    const U32x2 ql = Load8Align2(blk + 64 * n + 32 * (c & 1u) + l);
    const U32x2 qh = Load8Align2(blk + 128 + 32 * n + l);
    const int sc = static_cast<int8_t>(blk[192 + 8 * n + 2 * c + (l >> 4)]);
    const float d = HalfBitsToFloat(Load2(blk + 208));
    const uint32_t low[2] = {ql.x >> (4 * (c >> 1)), ql.y >> (4 * (c >> 1))};
    const uint32_t top[2] = {qh.x >> (2 * c), qh.y >> (2 * c)};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int q = static_cast<int>(((low[i >> 2] >> (8 * (i & 3))) & 15u) |
                                     (((top[i >> 2] >> (8 * (i & 3))) & 3u) << 4)) - 32;
      out[i] = d * static_cast<float>(sc * q);  // 11 x 13 bits: exact
    }
  } else {
    static_assert(TYPE == kTypeQ80, "Q5_K, Q6_K or Q8_0");
    // Eight blocks of d | 32 int8.
    const uint8_t* sub = blk + 34 * (k0 >> 5);
    const float d = HalfBitsToFloat(Load2(sub));
    const U32x2 q = Load8Align2(sub + 2 + (k0 & 31u));
    const uint32_t words[2] = {q.x, q.y};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int v = static_cast<int8_t>((words[i >> 2] >> (8 * (i & 3))) & 0xFFu);
      out[i] = d * static_cast<float>(v);  // 11 x 8 bits: exact
    }
  }
}

// Eight fp32 weights as one fragment: fp16, round to nearest, magnitudes above 65504
// saturate.
__device__ __forceinline__ U32x4 PackFragment(const float (&v)[8]) {
  uint32_t packed[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float lo = __builtin_fminf(__builtin_fmaxf(v[2 * i], -65504.0f), 65504.0f);
    const float hi = __builtin_fminf(__builtin_fmaxf(v[2 * i + 1], -65504.0f), 65504.0f);
    const Half2 h = {static_cast<_Float16>(lo), static_cast<_Float16>(hi)};
    packed[i] = __builtin_bit_cast(uint32_t, h);
  }
  return U32x4{packed[0], packed[1], packed[2], packed[3]};
}

// Both operands as fp16, one launch.  Every wave of workgroups [0, weight_groups)
// dequantizes a quarter (64 values, 4 steps) of one super-block of one group of 32 rows
// into fragments: w16[((group * nb + block) * 16 + step) * 64 + lane] (16 bytes each);
// rows past the matrix repeat its last row, their products are not stored.  The other
// workgroups convert 256 octets of activations each (bf16 -> fp16, same [token][k]
// layout).
template <int TYPE>
__global__ __launch_bounds__(256) void PrepareOperands(
    const U32x4* __restrict__ a, size_t octets, U32x4* __restrict__ a16,
    uint32_t weight_groups, const uint8_t* __restrict__ w, uint32_t rows, uint32_t nb,
    uint32_t row_groups, U32x4* __restrict__ w16) {
  if (blockIdx.x >= weight_groups) {
    const size_t i = static_cast<size_t>(blockIdx.x - weight_groups) * 256 + threadIdx.x;
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
    a16[i] = U32x4{packed[0], packed[1], packed[2], packed[3]};
    return;
  }
  const uint32_t quarter_unit = blockIdx.x * 4 + (threadIdx.x >> 6);
  const uint32_t unit = quarter_unit >> 2;  // (group, block)
  const uint32_t p = quarter_unit & 3;      // values 64 p .. 64 p + 63: steps 4 p .. 4 p + 3
  if (unit >= row_groups * nb) return;
  const uint32_t group = unit / nb;
  const uint32_t block = unit - group * nb;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t n = lane & 31;
  const uint32_t u = lane >> 5;
  const uint32_t r = min(group * 32 + n, rows - 1);
  const uint8_t* blk = w + (static_cast<size_t>(r) * nb + block) * BlockBytes(TYPE);
  U32x4* out = w16 + (static_cast<size_t>(unit) * 16 + 4 * p) * 64 + lane;
  if constexpr (TYPE == kTypeQ4K) {
    const U32x4 header = Load16(blk);
    const U32x4 codes = Load16(blk + 16 + 32 * p + 16 * u);
#pragma unroll
    for (int high = 0; high < 2; ++high) {
      float scale, offset;
      SubBlockAffine(header, 2 * p + high, &scale, &offset);
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        out[(2 * high + half) * 64] = WeightFragment(codes, 2 * high + half, scale, offset);
      }
    }
  } else {
    // Step 4 p + q holds k = 64 p + 32 (q / 2) + 16 u + 8 (q % 2) .. + 8, the order the
    // packed Q4_K block suggested; the activation side reads its pieces to match.
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      float v[8];
      DequantEight<TYPE>(blk, 64 * p + 32 * (q >> 1) + 16 * u + 8 * (q & 1), v);
      out[q * 64] = PackFragment(v);
    }
  }
}

// ---- the product ------------------------------------------------------------------

// Where the 16-byte piece p (0..15) of token row t sits inside the row's 256 bytes of
// LDS: slot p ^ Swizzle(t).  Rows are one bank sweep apart, so the slot alone decides
// the banks; a wave reads piece (c | 2 u) of rows n = 0..31, and the xor makes the 16
// slots of rows n..n+15 (either u) and of rows n..n+7 (both u) all different.
__device__ __forceinline__ uint32_t Swizzle(uint32_t t) {
  return (t & 1u) | (((t >> 1) & 3u) << 2) | (((t >> 3) & 1u) << 1);
}

// This lane's weight operand of one half super-block: the fragments of its 8 steps.
//
// The loads are issued from inline assembly and waited for by WaitForFragments below, not
// by the compiler: its own bookkeeping falls back to draining every vector-memory
// operation - the copies into LDS that are meant to stay in flight included - once the
// stores of a finished tile are pending in the same loop.
struct Fragments {
  U32x4 step[kWaveGroups][kStepsPerHalf];

  // `at[g]` is this lane's 16 bytes of step 0 of the wave's row group g; the steps are
  // kStepBytes apart.  The fields hold nothing until WaitForFragments has returned.
  // The load of step kStep of row group kGroup alone: the product kernel deals the sixteen
  // loads of a half one by one between the matrix instructions of the half before.
  template <int kGroup, int kStep>
  __device__ __forceinline__ void StartLoadOne(const uint8_t* const (&at)[kWaveGroups]) {
    static_assert(kGroup >= 0 && kGroup < kWaveGroups && kStep >= 0 && kStep < kStepsPerHalf, "");
    const uint8_t* base = at[kGroup] + (kStep / 4) * 4 * kStepBytes;  // the offset field reaches 4 KB
    U32x4& to = step[kGroup][kStep];
    if constexpr (kStep % 4 == 0) {
      asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(to) : "v"(base) : "memory");
    } else if constexpr (kStep % 4 == 1) {
      asm volatile("global_load_dwordx4 %0, %1, off offset:1024" : "=v"(to) : "v"(base) : "memory");
    } else if constexpr (kStep % 4 == 2) {
      asm volatile("global_load_dwordx4 %0, %1, off offset:2048" : "=v"(to) : "v"(base) : "memory");
    } else {
      asm volatile("global_load_dwordx4 %0, %1, off offset:3072" : "=v"(to) : "v"(base) : "memory");
    }
  }

  // Load number kIndex (0..15) of a half, in the order the product kernel issues them.
  template <int kIndex>
  __device__ __forceinline__ void StartLoadNumber(const uint8_t* const (&at)[kWaveGroups]) {
    StartLoadOne<kIndex % kWaveGroups, kIndex / kWaveGroups>(at);
  }

  template <int kIndex = 0>
  __device__ __forceinline__ void StartLoad(const uint8_t* const (&at)[kWaveGroups]) {
    if constexpr (kIndex < kWaveGroups * kStepsPerHalf) {
      StartLoadNumber<kIndex>(at);
      StartLoad<kIndex + 1>(at);
    }
  }
};
static_assert(kStepBytes == 1024 && kStepsPerHalf == 8, "the offsets above");

// Waits until f's loads have landed: until at most the kCopiesPerWave copies into LDS
// that every StartLoad is followed by are outstanding (operations retire in order, loads,
// copies and stores alike, so everything older has landed too).  Ties the fields to the
// wait so that no use of them moves above it.
__device__ __forceinline__ void WaitForFragments(Fragments& f) {
  static_assert(kCopiesPerWave == 8 && kWaveGroups == 2, "update the literal and the lists below");
  asm volatile("s_waitcnt vmcnt(8)"
               : "+v"(f.step[0][0]), "+v"(f.step[0][1]), "+v"(f.step[0][2]), "+v"(f.step[0][3]),
                 "+v"(f.step[0][4]), "+v"(f.step[0][5]), "+v"(f.step[0][6]), "+v"(f.step[0][7])
               :
               : "memory");
  // (An asm statement takes 30 operands at most; the second group is tied to the point
  // behind the wait by a statement of its own.)
  asm volatile(""
               : "+v"(f.step[1][0]), "+v"(f.step[1][1]), "+v"(f.step[1][2]), "+v"(f.step[1][3]),
                 "+v"(f.step[1][4]), "+v"(f.step[1][5]), "+v"(f.step[1][6]), "+v"(f.step[1][7])
               :
               : "memory");
}

// The byte address inside LDS of a pointer into the stage ring.
__device__ __forceinline__ uint32_t LdsAddress(const uint8_t* p) {
  return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((LdsPointer)p));
}

// This lane's activation operands of one step: its 16 bytes of the four 32-token tiles
// (32 token rows = 8 KB apart).  Read and waited for from inline assembly for the same
// reason as the weights: the wait is a count the compiler does not find.
struct ActivationFragments {
  U32x4 tile[4];

  template <int kTile>
  __device__ __forceinline__ void StartReadOne(uint32_t at) {
    static_assert(32 * kRowBytes == 8192, "the offsets below");
    if constexpr (kTile == 0) {
      asm volatile("ds_read_b128 %0, %1" : "=v"(tile[0]) : "v"(at) : "memory");
    } else if constexpr (kTile == 1) {
      asm volatile("ds_read_b128 %0, %1 offset:8192" : "=v"(tile[1]) : "v"(at) : "memory");
    } else if constexpr (kTile == 2) {
      asm volatile("ds_read_b128 %0, %1 offset:16384" : "=v"(tile[2]) : "v"(at) : "memory");
    } else {
      static_assert(kTile == 3, "four tiles");
      asm volatile("ds_read_b128 %0, %1 offset:24576" : "=v"(tile[3]) : "v"(at) : "memory");
    }
  }

  __device__ __forceinline__ void StartRead(uint32_t at) {
    StartReadOne<0>(at);
    StartReadOne<1>(at);
    StartReadOne<2>(at);
    StartReadOne<3>(at);
  }
};

// Waits until every LDS read issued so far has returned.
__device__ __forceinline__ void WaitForActivations(ActivationFragments& f) {
  asm volatile("s_waitcnt lgkmcnt(0)"
               : "+v"(f.tile[0]), "+v"(f.tile[1]), "+v"(f.tile[2]), "+v"(f.tile[3])
               :
               : "memory");
}

// The 16-byte piece of a token's half super-block that step s (0..7 within the half)
// reads for lane half u = 0; lane half 1 reads the piece 2 further.
__device__ __forceinline__ constexpr uint32_t StepPiece(int s) {
  return 8u * ((s >> 2) & 1) + 4u * ((s >> 1) & 1) + (s & 1);
}

struct GemmShape {
  uint32_t rows;
  uint32_t c_stride;     // floats between the token rows of c
  uint32_t nb;           // super-blocks per row
  uint32_t tokens;
  uint32_t row_tiles;
  uint32_t token_tiles;
  uint32_t band;         // weight-row tiles per band; the last band may hold fewer
  uint32_t per_xcd;      // consecutive tiles of the order each XCD takes
  uint32_t total;        // row_tiles * token_tiles
};

struct TileCoord {
  uint32_t token_tile;
  uint32_t row_tile;
};

// Tile number `position` of the order (band, token tile, row tile within the band).
__device__ __forceinline__ TileCoord DecodeTile(const GemmShape& shape, uint32_t position) {
  const uint32_t full_bands = shape.row_tiles / shape.band;
  const uint32_t in_full = full_bands * shape.token_tiles * shape.band;
  uint32_t width = shape.band;
  uint32_t band_index = position / (shape.band * shape.token_tiles);
  uint32_t local = position - band_index * shape.band * shape.token_tiles;
  if (position >= in_full) {  // the narrower last band
    width = shape.row_tiles - full_bands * shape.band;
    band_index = full_bands;
    local = position - in_full;
  }
  TileCoord tile;
  tile.token_tile = local / width;
  tile.row_tile = band_index * shape.band + (local - tile.token_tile * width);
  return tile;
}

// The workgroup barrier alone.  __syncthreads() adds a release fence that drains every
// vector-memory operation of the wave, the prefetches included; here the waits that
// matter are explicit: each wave waits for its own copies into LDS before the barrier,
// and has consumed its LDS reads of the stage about to be refilled by then.
__device__ __forceinline__ void TileBarrier() {
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// One workgroup per CU (the stage ring takes 128 KB of LDS): one wave per SIMD, which
// leaves it the whole register file - 128 accumulator registers, two sets of 64 for the
// weight fragments.
//
// The stream: this workgroup's tiles one after the other, each 2 nb halves.  Per wave,
// every half issues the same vector-memory operations in the same order - after the
// barrier the stores of the tile the half before completed (if any), then the weight
// fragments of half h + 1 (16 loads), then the copies of half h + 3 (kCopiesPerWave
// instructions) - and, after its matrix instructions, waits until only those copies may
// still be in flight: the fragments of half h + 1 have then landed, and with them
// everything older, the copies of half h + 1 among it.  Past the end of the stream the
// loads and copies repeat the last half into registers and a stage nobody uses, so the
// count never changes.
__global__ __launch_bounds__(kGemmThreads) __attribute__((amdgpu_waves_per_eu(1, 1))) void
KquantGemmKernel(const uint8_t* __restrict__ w16, const uint8_t* __restrict__ a16,
                 float* __restrict__ c, GemmShape shape) {
  extern __shared__ __align__(1024) uint8_t stages[];  // kStages x kStageBytes

  // This workgroup's tiles: positions first, first + stride, ... of its XCD's piece.
  const uint32_t xcd = blockIdx.x % kXcds;
  const uint32_t in_xcd = blockIdx.x / kXcds;
  const uint32_t stride = gridDim.x / kXcds;
  const uint32_t first = xcd * shape.per_xcd + in_xcd;
  if (in_xcd >= shape.per_xcd || first >= shape.total) return;
  const uint32_t reach = min(shape.per_xcd - in_xcd, shape.total - first);
  const uint32_t n_tiles = (reach + stride - 1) / stride;

  const uint32_t tid = threadIdx.x;
  const uint32_t lane = tid & 63;
  const uint32_t wave = tid >> 6;
  const uint32_t n = lane & 31;
  const uint32_t u = lane >> 5;
  const uint32_t nb = shape.nb;
  const uint32_t total_halves = 2 * n_tiles * nb;

  // ---- copies global -> LDS ----
  // Wave instruction i of this wave fills the 1 KB holding token rows 4 c .. 4 c + 3 of
  // a stage (c = wave * kCopiesPerWave + i); lane l supplies LDS slot l % 16 of row
  // 4 c + l / 16, that is piece slot ^ Swizzle(row) of the token's half block.  Rows
  // past the last token repeat it; their products are not stored.
  uint32_t copy_offset[kCopiesPerWave];  // bytes from a16 + 256 * (half within the tile)
  // (Every lambda below is inlined by force: one left as a call would take the
  // accumulators and the fragments it captures by reference out of their registers.)
  auto aim_copies = [&](uint32_t token_tile) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < kCopiesPerWave; ++i) {
      const uint32_t t = 4 * (wave * kCopiesPerWave + i) + (lane >> 4);
      const uint32_t token = min(token_tile * kTileTokens + t, shape.tokens - 1);
      copy_offset[i] = token * (nb * 512) + (((lane & 15u) ^ Swizzle(t & 15u)) << 4);
    }
  };
  // Past the end of the stream the last half is copied again, into a stage nobody reads
  // any more: every half issues the same operations, which keeps the wait a constant.
  uint32_t copy_half = 0;    // stream half the next copy brings in
  uint32_t copy_within = 0;  // the same, within its tile
  uint32_t copy_tile = 0;    // index into this workgroup's tiles
  struct CopyPlan {
    const uint8_t* source[kCopiesPerWave];
    uint8_t* stage;
  };
  // Where the copies of the next half read and write; moves on to the half after it.
  auto plan_next_copy = [&]() __attribute__((always_inline)) {
    CopyPlan plan;
    const uint8_t* base = a16 + static_cast<size_t>(copy_within) * kRowBytes;
#pragma unroll
    for (int i = 0; i < kCopiesPerWave; ++i) plan.source[i] = base + copy_offset[i];
    plan.stage = stages + (copy_half % kStages) * kStageBytes + wave * kCopiesPerWave * 1024;
    if (++copy_half < total_halves && ++copy_within == 2 * nb) {
      copy_within = 0;
      ++copy_tile;
      aim_copies(DecodeTile(shape, first + copy_tile * stride).token_tile);
    }
    return plan;
  };
  auto start_copy = [&](const CopyPlan& plan, int i) __attribute__((always_inline)) {
    __builtin_amdgcn_global_load_lds(plan.source[i], (LdsPointer)(plan.stage + i * 1024), 16, 0, 0);
  };
  auto start_copies = [&](const CopyPlan& plan) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < kCopiesPerWave; ++i) start_copy(plan, i);
  };

  // ---- weight fragments, one half ahead ----
  // Past the end of the stream the last half is loaded again and never used.
  // This lane's 16 bytes of step 0 of the next half to load, in the wave's first row
  // group; the fragments of its other groups follow group_bytes apart.
  const uint8_t* load_ptr = nullptr;
  const size_t group_bytes = static_cast<size_t>(nb) * 2 * kHalfBytes;
  uint32_t load_half = 0;
  uint32_t load_within = 0;
  uint32_t load_tile = 0;
  auto aim_loads = [&](uint32_t row_tile) __attribute__((always_inline)) {
    const size_t group = static_cast<size_t>(row_tile) * kTileGroups + wave * kWaveGroups;
    load_ptr = w16 + group * group_bytes + lane * 16;
  };
  struct LoadPlan {
    const uint8_t* at[kWaveGroups];
  };
  // Where the fragments of the next half are; moves on to the half after it.
  auto plan_next_load = [&]() __attribute__((always_inline)) {
    LoadPlan plan;
#pragma unroll
    for (int g = 0; g < kWaveGroups; ++g) plan.at[g] = load_ptr + g * group_bytes;
    if (++load_half < total_halves) {
      load_ptr += kHalfBytes;
      if (++load_within == 2 * nb) {
        load_within = 0;
        ++load_tile;
        aim_loads(DecodeTile(shape, first + load_tile * stride).row_tile);
      }
    }
    return plan;
  };

  Float16v acc[kWaveGroups][4];
  auto clear_acc = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int g = 0; g < kWaveGroups; ++g) {
#pragma unroll
      for (int m = 0; m < 4; ++m) {
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[g][m][i] = 0.0f;
      }
    }
  };
  clear_acc();

  // This lane's activation fragment of step s, token tile m: piece StepPiece(s) | 2 u of
  // row 32 m + n, at slot StepPiece(s) ^ flip.
  const uint32_t flip = Swizzle(n & 15u) ^ (u << 1);
  const uint32_t read_base = n * kRowBytes;

  // The constant-index members behind indices that are constants only once the step loop
  // is unrolled.
  auto start_read_one = [&](ActivationFragments& f, int m, uint32_t at)
                            __attribute__((always_inline)) {
    switch (m) {
      case 0: f.template StartReadOne<0>(at); break;
      case 1: f.template StartReadOne<1>(at); break;
      case 2: f.template StartReadOne<2>(at); break;
      default: f.template StartReadOne<3>(at); break;
    }
  };
  auto start_load_number = [&](Fragments& f, const LoadPlan& at, int index)
                               __attribute__((always_inline)) {
    switch (index) {
      case 0: f.template StartLoadNumber<0>(at.at); break;
      case 1: f.template StartLoadNumber<1>(at.at); break;
      case 2: f.template StartLoadNumber<2>(at.at); break;
      case 3: f.template StartLoadNumber<3>(at.at); break;
      case 4: f.template StartLoadNumber<4>(at.at); break;
      case 5: f.template StartLoadNumber<5>(at.at); break;
      case 6: f.template StartLoadNumber<6>(at.at); break;
      case 7: f.template StartLoadNumber<7>(at.at); break;
      case 8: f.template StartLoadNumber<8>(at.at); break;
      case 9: f.template StartLoadNumber<9>(at.at); break;
      case 10: f.template StartLoadNumber<10>(at.at); break;
      case 11: f.template StartLoadNumber<11>(at.at); break;
      case 12: f.template StartLoadNumber<12>(at.at); break;
      case 13: f.template StartLoadNumber<13>(at.at); break;
      case 14: f.template StartLoadNumber<14>(at.at); break;
      default: f.template StartLoadNumber<15>(at.at); break;
    }
  };

  // One half super-block: 8 steps of 8 matrix instructions on the stage of stream half
  // `half`.  A wave is alone on its SIMD, so whatever it issues between two matrix
  // instructions is covered by the first of them (32 cycles in the matrix core), and
  // whatever it issues in a block of its own is not.  Hence one memory instruction behind
  // each matrix instruction: behind the first four of step s the LDS reads of step s + 1's
  // activation fragments, behind the last four a quarter of the half's vector-memory
  // operations - the next half's weight fragments over steps 0-3, the copies of the half
  // three ahead over steps 4-7 (two a step).  The wait at the top of a step is then for
  // reads that were issued at least four matrix instructions earlier.
  // (Left to the compiler, the LDS waits become lgkmcnt(0) right behind the reads on every
  // second step: a whole LDS latency in front of the matrix instructions.)
  auto multiply_half = [&](uint32_t half, const Fragments& weights, Fragments& later,
                           const LoadPlan& later_at, const CopyPlan& copies)
                           __attribute__((always_inline)) {
    const uint32_t tile = LdsAddress(stages + (half % kStages) * kStageBytes + read_base);
    ActivationFragments af[2];
    af[0].StartRead(tile + ((StepPiece(0) ^ flip) << 4));
#pragma unroll
    for (int s = 0; s < kStepsPerHalf; ++s) {
      WaitForActivations(af[s & 1]);
#pragma unroll
      for (int j = 0; j < 4 * kWaveGroups; ++j) {
        const int g = j % kWaveGroups;
        const int m = j / kWaveGroups;
        acc[g][m] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
            __builtin_bit_cast(Half8, af[s & 1].tile[m]),
            __builtin_bit_cast(Half8, weights.step[g][s]), acc[g][m], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (j < 4) {
          // Into the registers step s - 1 multiplied from: its last matrix instruction was
          // issued before this step's first.
          if (s + 1 < kStepsPerHalf) {
            start_read_one(af[(s + 1) & 1], j, tile + ((StepPiece(s + 1) ^ flip) << 4));
          }
        } else if (s < 4) {
          start_load_number(later, later_at, 4 * s + (j - 4));
        } else if (j - 4 < 2) {
          start_copy(copies, 2 * (s - 4) + (j - 4));
        }
        __builtin_amdgcn_sched_barrier(0);  // the wait of the half counts on this issue order
      }
    }
  };

  // ---- the tile being multiplied ----
  uint32_t tile_index = 0;
  uint32_t half_within = 0;
  TileCoord tile = DecodeTile(shape, first);
  // With the activations as the first operand, accumulator register i of row group g,
  // token tile m holds token 32 m + 8 (i/4) + 4 u + i%4 and weight row 32 g + n of this
  // wave's 64: a store instruction writes, for two tokens (u = 0, 1), 32 consecutive
  // floats of their rows of c each - whole 128-byte lines when the matrix has a multiple
  // of 32 rows.
  auto finish_tile = [&]() __attribute__((always_inline)) {
    const uint32_t row0 = tile.row_tile * kTileRows + wave * (32 * kWaveGroups);
    const uint32_t token_first = tile.token_tile * kTileTokens;
    const bool whole = row0 + 32 * kWaveGroups <= shape.rows &&
                       token_first + kTileTokens <= shape.tokens;
    auto store_all = [&](auto check) __attribute__((always_inline)) {
#pragma unroll
      for (int g = 0; g < kWaveGroups; ++g) {
        const uint32_t row = row0 + 32 * g + n;
#pragma unroll
        for (int m = 0; m < 4; ++m) {
          const uint32_t t0 = token_first + m * 32 + 4 * u;
          float* at = c + static_cast<size_t>(t0) * shape.c_stride + row;
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const uint32_t dt = 8 * (i >> 2) + (i & 3);
            if (!decltype(check)::value || (t0 + dt < shape.tokens && row < shape.rows)) {
              at[static_cast<size_t>(dt) * shape.c_stride] = acc[g][m][i];
            }
          }
        }
      }
    };
    if (whole) {
      store_all(std::false_type{});
    } else {
      store_all(std::true_type{});
    }
    clear_acc();
    if (++tile_index < n_tiles) tile = DecodeTile(shape, first + tile_index * stride);
  };

  // Stream half h on `now` (landed), with `later` taking the fragments of half h + 1.
  // Between the StartLoad of a set of fragments and its wait there is straight-line code
  // only - no branch, no loop edge - so the compiler has no reason to copy registers the
  // loads have not written yet: the stores of a finished tile and the bookkeeping of the
  // two streams, which branch, come first.
  bool tile_complete = false;  // the half before was the last of its tile
  auto run_half = [&](uint32_t h, const Fragments& now, Fragments& later)
                      __attribute__((always_inline)) {
    TileBarrier();
    if (tile_complete) {
      finish_tile();
      tile_complete = false;
    }
    if (++half_within == 2 * nb) {
      half_within = 0;
      tile_complete = true;
    }
    const LoadPlan fragments_at = plan_next_load();
    const CopyPlan copies = plan_next_copy();
    __builtin_amdgcn_sched_barrier(0);
    multiply_half(h, now, later, fragments_at, copies);
    WaitForFragments(later);
  };

  // ---- prologue: the operations the steady state would have issued before half 0 ----
  aim_copies(tile.token_tile);
  aim_loads(tile.row_tile);
  Fragments even, odd;
  start_copies(plan_next_copy());       // half 0
  start_copies(plan_next_copy());       // half 1 (a tile has at least two halves)
  {
    const LoadPlan fragments_at = plan_next_load();  // half 0
    const CopyPlan copies = plan_next_copy();        // half 2
    even.StartLoad(fragments_at.at);
    start_copies(copies);
  }
  WaitForFragments(even);
  for (uint32_t h = 0; h < total_halves; h += 2) {
    run_half(h, even, odd);
    run_half(h + 1, odd, even);
  }
  finish_tile();
}

}  // namespace

namespace {

// The pre-pass over `octets` activation octets (none: a null `a_bf16`) and, when `w` is
// given, over the weights.
hipError_t LaunchPrepare(int type, const uint8_t* w, uint32_t rows, uint32_t blocks_per_row,
                         const uint16_t* a_bf16, size_t octets, uint8_t* a16, uint8_t* w16,
                         hipStream_t stream) {
  const uint32_t row_tiles = (rows + kTileRows - 1) / kTileRows;
  const uint32_t row_groups = row_tiles * kTileGroups;
  const uint32_t act_groups = a_bf16 != nullptr ? static_cast<uint32_t>((octets + 255) / 256) : 0;
  // One workgroup (4 waves) per (32 rows, super-block): a wave per quarter.
  const uint32_t weight_groups = w != nullptr ? row_groups * blocks_per_row : 0;
  if (weight_groups + act_groups == 0) return hipSuccess;
  auto prepare = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3(weight_groups + act_groups), dim3(256), 0, stream,
                       reinterpret_cast<const U32x4*>(a_bf16), octets,
                       reinterpret_cast<U32x4*>(a16), weight_groups, w, rows, blocks_per_row,
                       row_groups, reinterpret_cast<U32x4*>(w16));
  };
  switch (type) {
    case kTypeQ4K: prepare(PrepareOperands<kTypeQ4K>); break;
    case kTypeQ5K: prepare(PrepareOperands<kTypeQ5K>); break;
    case kTypeQ6K: prepare(PrepareOperands<kTypeQ6K>); break;
    default: prepare(PrepareOperands<kTypeQ80>); break;
  }
  return hipGetLastError();
}

}  // namespace

size_t GemmActivationBytes(size_t tokens, uint32_t blocks_per_row) {
  return (tokens * blocks_per_row * 512 + 255) & ~static_cast<size_t>(255);
}

// The fragments of every 32 rows of every row tile.
size_t GemmWeightBytes(uint32_t rows, uint32_t blocks_per_row) {
  const size_t row_tiles = (static_cast<size_t>(rows) + kTileRows - 1) / kTileRows;
  return row_tiles * kTileGroups * blocks_per_row * 2 * kHalfBytes;
}

bool GemmTakesType(int type) {
  return type == kTypeQ4K || type == kTypeQ5K || type == kTypeQ6K || type == kTypeQ80;
}

hipError_t LaunchGemmPrepareWeights(int type, const uint8_t* w, uint32_t rows,
                                    uint32_t blocks_per_row, void* fragments,
                                    hipStream_t stream) {
  if (!GemmTakesType(type) || blocks_per_row == 0) return hipErrorInvalidValue;
  if (rows == 0) return hipSuccess;
  return LaunchPrepare(type, w, rows, blocks_per_row, nullptr, 0, nullptr,
                       static_cast<uint8_t*>(fragments), stream);
}

hipError_t LaunchGemm(int type, const uint8_t* w, uint32_t rows, uint32_t blocks_per_row,
                      const void* fragments, const uint16_t* a_bf16, size_t tokens,
                      void* workspace, float* c, uint32_t c_stride, hipStream_t stream) {
  if (!GemmTakesType(type) || c_stride < rows) return hipErrorInvalidValue;
  if (rows == 0 || tokens == 0) return hipSuccess;
  // Activation bytes are addressed with 32 bits.
  if (blocks_per_row == 0 || tokens > 0xFFFFFFFFull / (512ull * blocks_per_row)) {
    return hipErrorInvalidValue;
  }
  const size_t octets = tokens * blocks_per_row * 32;
  uint8_t* a16 = static_cast<uint8_t*>(workspace);
  uint8_t* own_w16 = a16 + GemmActivationBytes(tokens, blocks_per_row);
  const uint8_t* w16 = fragments != nullptr ? static_cast<const uint8_t*>(fragments) : own_w16;
  const uint32_t row_tiles = (rows + kTileRows - 1) / kTileRows;
  hipError_t status = LaunchPrepare(type, fragments != nullptr ? nullptr : w, rows,
                                    blocks_per_row, a_bf16, octets, a16, own_w16, stream);
  if (status != hipSuccess) return status;

  constexpr size_t lds_bytes = static_cast<size_t>(kStages) * kStageBytes;
  static bool allowed = false;
  if (!allowed) {
    status = hipFuncSetAttribute(reinterpret_cast<const void*>(KquantGemmKernel),
                                 hipFuncAttributeMaxDynamicSharedMemorySize,
                                 static_cast<int>(lds_bytes));
    if (status != hipSuccess) return status;
    allowed = true;
  }
  GemmShape shape;
  shape.rows = rows;
  shape.c_stride = c_stride;
  shape.nb = blocks_per_row;
  shape.tokens = static_cast<uint32_t>(tokens);
  shape.row_tiles = row_tiles;
  shape.token_tiles = static_cast<uint32_t>((tokens + kTileTokens - 1) / kTileTokens);
  shape.band = (shape.row_tiles + kXcds - 1) / kXcds;
  shape.total = shape.row_tiles * shape.token_tiles;
  shape.per_xcd = (shape.total + kXcds - 1) / kXcds;
  // One workgroup per CU, the same number on every XCD, no more than there are tiles.
  uint32_t per_xcd_groups = static_cast<uint32_t>(DeviceComputeUnits()) / kXcds;
  if (per_xcd_groups == 0) per_xcd_groups = 1;
  if (per_xcd_groups > shape.per_xcd) per_xcd_groups = shape.per_xcd;
  hipLaunchKernelGGL(KquantGemmKernel, dim3(per_xcd_groups * kXcds), dim3(kGemmThreads),
                     lds_bytes, stream, w16, a16, c, shape);
  return hipGetLastError();
}

}  // namespace gufo
