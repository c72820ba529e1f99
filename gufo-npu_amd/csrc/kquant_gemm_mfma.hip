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
// Decomposition: one persistent workgroup of 8 waves per CU walks its share of the
// 128-token x 256-row tiles.  Each wave owns 32 weight rows: it reads their packed
// blocks into registers one super-block ahead, builds the operand fragments on the
// fly and multiplies them with the four 32-token tiles.  The activations of half a
// super-block (128 tokens x 128 fp16 = 32 KB, a "stage") go from global memory
// straight into LDS (global_load_lds_dwordx4) into a ring of four stages, three
// halves ahead of the matrix cores - across tile boundaries too, so the copies of a
// tile's first halves and the stores of the previous tile's results overlap.
//
// The matrix instruction does not care which k a lane's 8 values belong to as long as
// both operands agree, so k is dealt to lanes the way the packed block likes it: of
// each 64 values (32 bytes of codes: low nibbles one sub-block, high nibbles the
// next), lane half u owns bytes 16 u .. 16 u + 15 - one 16-byte load - and its four
// steps take (low, first 8), (low, second 8), (high, first 8), (high, second 8).
//
// Tiles are ordered (band of row tiles, token tile, row tile within the band) and the
// order is cut in 8 pieces, one per XCD (workgroups go to XCDs round-robin): an XCD's
// slice of the packed matrix stays in its L2 while it walks the token tiles, and the
// workgroups running together share activation tiles.
#include <type_traits>

#include "kernels.hpp"
#include "kquant_common.hpp"

namespace gufo {
namespace {

typedef _Float16 Half8 __attribute__((ext_vector_type(8)));
typedef _Float16 Half2 __attribute__((ext_vector_type(2)));
typedef float Float16v __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(3))) void* LdsPointer;

constexpr int kGemmThreads = 512;
constexpr int kGemmWaves = kGemmThreads / 64;
constexpr int kTileTokens = 128;
constexpr int kTileRows = 32 * kGemmWaves;
constexpr int kRowBytes = 256;                            // one token's half super-block as fp16
constexpr int kStageBytes = kTileTokens * kRowBytes;      // 32 KB
constexpr int kStages = 4;
constexpr int kAhead = kStages - 1;                       // halves the copies run ahead
constexpr int kCopiesPerWave = kStageBytes / 1024 / kGemmWaves;  // 1 KB per wave instruction
constexpr int kRowLoads = 5;                              // vector loads of one PackedRow
constexpr int kTileStores = 16;                           // 16-byte stores of a whole tile, per wave
// Operations a wave has issued after the copies of half h when it reaches the top of
// half h: the copies of two more halves and the row loads of one (h even) or two blocks.
constexpr int kEvenYounger = 2 * kCopiesPerWave + kRowLoads;
constexpr int kOddYounger = 2 * kCopiesPerWave + 2 * kRowLoads;
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
//
// The loads are issued from inline assembly and waited for by WaitForRow below, not by
// the compiler: its own bookkeeping falls back to draining every vector-memory
// operation - the copies into LDS that are meant to stay in flight included - once the
// stores of a finished tile are pending in the same loop.
struct PackedRow {
  U32x4 header;     // d, dmin, 12 scale bytes
  U32x4 codes[4];   // codes[p] = qs[32 p + 16 u .. +16)

  // Starts the kRowLoads loads; the fields hold nothing until WaitForRow has returned.
  __device__ __forceinline__ void StartLoad(const uint8_t* blk, uint32_t u) {
    const uint8_t* half = blk + 16 * u;
    asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(header) : "v"(blk) : "memory");
    asm volatile("global_load_dwordx4 %0, %1, off offset:16" : "=v"(codes[0]) : "v"(half) : "memory");
    asm volatile("global_load_dwordx4 %0, %1, off offset:48" : "=v"(codes[1]) : "v"(half) : "memory");
    asm volatile("global_load_dwordx4 %0, %1, off offset:80" : "=v"(codes[2]) : "v"(half) : "memory");
    asm volatile("global_load_dwordx4 %0, %1, off offset:112" : "=v"(codes[3]) : "v"(half) : "memory");
  }
};

// Waits until at most kYounger vector-memory operations issued after row's loads are
// outstanding, which is when the loads have landed; ties the fields to the wait so that
// no use of them moves above it.
template <int kYounger>
__device__ __forceinline__ void WaitForRow(PackedRow& row) {
  static_assert(kYounger == 0 || kYounger == kCopiesPerWave,
                "the counts the copy schedule produces");
  static_assert(kCopiesPerWave == 4, "update the literal below");
  if constexpr (kYounger == 0) {
    asm volatile("s_waitcnt vmcnt(0)"
                 : "+v"(row.header), "+v"(row.codes[0]), "+v"(row.codes[1]), "+v"(row.codes[2]),
                   "+v"(row.codes[3])
                 :
                 : "memory");
  } else {
    asm volatile("s_waitcnt vmcnt(4)"
                 : "+v"(row.header), "+v"(row.codes[0]), "+v"(row.codes[1]), "+v"(row.codes[2]),
                   "+v"(row.codes[3])
                 :
                 : "memory");
  }
}

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

// Step s = 4 p + 2 high + half of a super-block: this lane's 8 dequantized values,
// k = 64 p + 32 high + 16 u + 8 half .. +8 of sub-block j = 2 p + high = s / 2, whose
// scale and offset the caller passes.
__device__ __forceinline__ Half8 WeightFragment(const PackedRow& row, int s, float scale,
                                                float offset) {
  const int p = s >> 2;
  const uint32_t b0 = (s & 1) ? row.codes[p].z : row.codes[p].x;
  const uint32_t b1 = (s & 1) ? row.codes[p].w : row.codes[p].y;
  const uint32_t shift = (s & 2) ? 4 : 0;
  const uint32_t n0 = (b0 >> shift) & 0x0F0F0F0Fu;
  const uint32_t n1 = (b1 >> shift) & 0x0F0F0F0Fu;
  // perm selectors: result bytes [3..0] = [0x64, q_hi, 0x64, q_lo]; source 1 (nibbles)
  // holds bytes 0-3, source 0 (the constant) bytes 4-7.
  U32x4 out;
  out.x = DequantPair(n0, 0x04010400u, scale, offset);  // codes 0, 1
  out.y = DequantPair(n0, 0x04030402u, scale, offset);  // codes 2, 3
  out.z = DequantPair(n1, 0x04010400u, scale, offset);  // codes 4, 5
  out.w = DequantPair(n1, 0x04030402u, scale, offset);  // codes 6, 7
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
  uint32_t band;         // weight-row tiles per band; the last band may hold fewer
  uint32_t per_xcd;      // consecutive tiles of the order each XCD takes
  uint32_t total;        // row_tiles * token_tiles
  uint32_t vector_stores;  // c and its rows are 16-byte aligned
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

// Waits until at most kPending of this wave's vector-memory operations are outstanding
// (they retire in order, loads, copies into LDS and stores alike).
template <int kPending>
__device__ __forceinline__ void WaitVectorMemory() {
  if constexpr (kPending == 0) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  } else if constexpr (kPending == 13) {
    asm volatile("s_waitcnt vmcnt(13)" ::: "memory");
  } else if constexpr (kPending == 18) {
    asm volatile("s_waitcnt vmcnt(18)" ::: "memory");
  } else if constexpr (kPending == 29) {
    asm volatile("s_waitcnt vmcnt(29)" ::: "memory");
  } else {
    static_assert(kPending == 34, "a count the copy schedule does not produce");
    asm volatile("s_waitcnt vmcnt(34)" ::: "memory");
  }
}

// The workgroup barrier alone.  __syncthreads() adds a release fence that drains every
// vector-memory operation of the wave, the prefetches included; here the waits that
// matter are explicit: each wave waits for its own copies into LDS before the barrier,
// and has consumed its LDS reads of the stage about to be refilled by then.
__device__ __forceinline__ void TileBarrier() {
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// One workgroup per CU (the stage ring takes 128 KB of LDS): 2 waves per SIMD.
//
// The stream: this workgroup's tiles one after the other, each 2 nb halves.  Per wave,
// vector-memory operations are issued in a fixed order - at the top of stream half h
// the copies of half h + 3 (kCopiesPerWave instructions), then, if h is even, the
// packed rows of the block after the current one (kRowLoads loads) - so that "the
// copies of half h have landed" is a fixed count of younger operations allowed in
// flight: 13 for even h, 18 for odd h.  Stores of finished tiles only add younger
// operations, which makes a wait stricter, never too weak.  The last two blocks of
// the stream, where copies run out, drain completely instead.
__global__ __launch_bounds__(kGemmThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void
KquantGemmKernel(const uint8_t* __restrict__ w, const uint8_t* __restrict__ a16,
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
  const uint32_t total_blocks = n_tiles * nb;
  const uint32_t total_halves = 2 * total_blocks;

  // ---- copies global -> LDS ----
  // Wave instruction i of this wave fills the 1 KB holding token rows 4 c .. 4 c + 3 of
  // a stage (c = wave * kCopiesPerWave + i); lane l supplies LDS slot l % 16 of row
  // 4 c + l / 16, that is piece slot ^ Swizzle(row) of the token's half block.  Rows
  // past the last token repeat it; their products are not stored.
  uint32_t copy_offset[kCopiesPerWave];  // bytes from a16 + 256 * (half within the tile)
  auto aim_copies = [&](uint32_t token_tile) {
#pragma unroll
    for (int i = 0; i < kCopiesPerWave; ++i) {
      const uint32_t t = 4 * (wave * kCopiesPerWave + i) + (lane >> 4);
      const uint32_t token = min(token_tile * kTileTokens + t, shape.tokens - 1);
      copy_offset[i] = token * (nb * 512) + (((lane & 15u) ^ Swizzle(t & 15u)) << 4);
    }
  };
  uint32_t copy_half = 0;    // stream half the next copy brings in
  uint32_t copy_within = 0;  // the same, within its tile
  uint32_t copy_tile = 0;    // index into this workgroup's tiles
  auto copy_next_half = [&]() {
    const uint8_t* base = a16 + static_cast<size_t>(copy_within) * kRowBytes;
    uint8_t* stage = stages + (copy_half % kStages) * kStageBytes;
#pragma unroll
    for (int i = 0; i < kCopiesPerWave; ++i) {
      uint8_t* dst = stage + (wave * kCopiesPerWave + i) * 1024;
      __builtin_amdgcn_global_load_lds(base + copy_offset[i], (LdsPointer)dst, 16, 0, 0);
    }
    ++copy_half;
    if (++copy_within == 2 * nb) {
      copy_within = 0;
      if (++copy_tile < n_tiles) {
        aim_copies(DecodeTile(shape, first + copy_tile * stride).token_tile);
      }
    }
  };

  // ---- packed weight rows, one block ahead ----
  const uint8_t* load_ptr = nullptr;  // this lane's row, next block to load
  uint32_t load_within = 0;
  uint32_t load_tile = 0;
  auto aim_loads = [&](uint32_t row_tile) {
    const uint32_t r = min(row_tile * kTileRows + wave * 32 + n, shape.rows - 1);
    load_ptr = w + static_cast<size_t>(r) * nb * kQ4Block;
  };
  auto load_next_block = [&](PackedRow& into) {
    into.StartLoad(load_ptr, u);
    load_ptr += kQ4Block;
    if (++load_within == nb) {
      load_within = 0;
      if (++load_tile < n_tiles) aim_loads(DecodeTile(shape, first + load_tile * stride).row_tile);
    }
  };

  Float16v acc[4];
  auto clear_acc = [&]() {
#pragma unroll
    for (int m = 0; m < 4; ++m) {
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[m][i] = 0.0f;
    }
  };
  clear_acc();

  // This lane's activation fragment of step s, token tile m: piece StepPiece(s) | 2 u of
  // row 32 m + n, at slot StepPiece(s) ^ flip.
  const uint32_t flip = Swizzle(n & 15u) ^ (u << 1);
  const uint32_t read_base = n * kRowBytes;

  // The weight operand runs one step ahead of the matrix cores across halves, blocks
  // and tiles: `bf` enters a half holding its first step's fragment and leaves holding
  // the next half's; `scale`/`offset` belong to the sub-block last dequantized.
  Half8 bf;
  float scale, offset;

  // One half super-block: 8 steps on the stage of stream half `half`.  While step s
  // multiplies, the activation fragments of step s + 1 are on their way from LDS and
  // the weight fragment of the step after it (of `follow`, the next block, after the
  // last step of a block) is being dequantized between the matrix instructions.
  // follow's loads are waited for just before that, with kYounger operations issued since.
  auto multiply_half = [&](uint32_t half, const PackedRow& cur, PackedRow& follow, auto half_tag,
                           auto younger_tag) {
    constexpr int kHalf = decltype(half_tag)::value;
    constexpr int kYounger = decltype(younger_tag)::value;
    const uint8_t* tile = stages + (half % kStages) * kStageBytes + read_base;
    Half8 af[4];
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      af[m] = *reinterpret_cast<const Half8*>(tile + ((StepPiece(0) ^ flip) << 4) +
                                              m * 32 * kRowBytes);
    }
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      Half8 af_next[4];
      if (s + 1 < 8) {
        const uint8_t* at = tile + ((StepPiece(s + 1) ^ flip) << 4);
#pragma unroll
        for (int m = 0; m < 4; ++m) {
          af_next[m] = *reinterpret_cast<const Half8*>(at + m * 32 * kRowBytes);
        }
      }
      // Nothing moves across: the reads of step s + 1 are issued before step s multiplies.
      __builtin_amdgcn_sched_barrier(0);
      const int upcoming = 8 * kHalf + s + 1;  // the step being dequantized
      if (upcoming == 16) WaitForRow<kYounger>(follow);
      const PackedRow& source = upcoming < 16 ? cur : follow;
      if (upcoming % 2 == 0) {
        SubBlockAffine(source.header, (upcoming % 16) / 2, &scale, &offset);
      }
      const Half8 bf_next = WeightFragment(source, upcoming % 16, scale, offset);
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf, af[m], acc[m], 0, 0, 0);
      }
      // Within the step: each matrix instruction followed by a quarter of that work.
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 7, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      if (s + 1 < 8) {
#pragma unroll
        for (int m = 0; m < 4; ++m) af[m] = af_next[m];
      }
      bf = bf_next;
    }
  };

  // ---- the tile being multiplied ----
  uint32_t tile_index = 0;
  uint32_t block_within = 0;
  TileCoord tile = DecodeTile(shape, first);
  // With the weights as the first operand, accumulator register i of token tile m holds
  // weight row 8 (i/4) + 4 u + i%4 of this wave's 32 and token 32 m + n: four registers
  // are four consecutive floats of a row of c.  A tile that lies wholly inside c stores
  // them as kTileStores 16-byte stores per wave; a ragged one stores float by float.
  // Returns whether the fixed number of stores was issued.
  auto finish_tile = [&]() -> bool {
    const uint32_t row0 = tile.row_tile * kTileRows + wave * 32;
    const uint32_t token_first = tile.token_tile * kTileTokens;
    const bool whole = shape.vector_stores != 0 && row0 + 32 <= shape.rows &&
                       token_first + kTileTokens <= shape.tokens;
    if (whole) {
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        float* at = c + static_cast<size_t>(token_first + m * 32 + n) * shape.rows + row0 + 4 * u;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          typedef float Float4 __attribute__((ext_vector_type(4)));
          const Float4 v = {acc[m][4 * q], acc[m][4 * q + 1], acc[m][4 * q + 2], acc[m][4 * q + 3]};
          *reinterpret_cast<Float4*>(at + 8 * q) = v;
        }
      }
    } else {
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        const uint32_t t = token_first + m * 32 + n;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const uint32_t row = row0 + 8 * (i >> 2) + 4 * u + (i & 3);
          if (t < shape.tokens && row < shape.rows) {
            c[static_cast<size_t>(t) * shape.rows + row] = acc[m][i];
          }
        }
      }
    }
    clear_acc();
    if (++tile_index < n_tiles) tile = DecodeTile(shape, first + tile_index * stride);
    return whole;
  };

  // ---- prologue: the operations the steady state would have issued before half 0 ----
  aim_copies(tile.token_tile);
  aim_loads(tile.row_tile);
  PackedRow cur, next;
  copy_next_half();                                   // half 0
  if (total_halves > 1) copy_next_half();             // half 1
  load_next_block(cur);                               // block 0
  if (total_halves > 2) copy_next_half();             // half 2
  WaitForRow<0>(cur);
  next = cur;  // defined contents for the dequantization past the last block
  SubBlockAffine(cur.header, 0, &scale, &offset);
  bf = WeightFragment(cur, 0, scale, offset);

  constexpr std::integral_constant<int, 0> kDrain{};  // unused by first halves
  uint32_t block = 0;
  // Steady state: every copy and load below exists, so the counts hold.
  // Halves left whose copies were issued before the stores of a finished tile: for
  // those the stores are kTileStores more younger operations.
  uint32_t behind_stores = 0;
  for (; block + 2 < total_blocks; ++block) {
    if (behind_stores > 0) {
      WaitVectorMemory<kEvenYounger + kTileStores>();
      --behind_stores;
    } else {
      WaitVectorMemory<kEvenYounger>();
    }
    TileBarrier();
    copy_next_half();
    __builtin_amdgcn_sched_barrier(0);  // the waits count on this issue order
    load_next_block(next);
    multiply_half(2 * block, cur, next, std::integral_constant<int, 0>{}, kDrain);
    if (behind_stores > 0) {
      WaitVectorMemory<kOddYounger + kTileStores>();
      --behind_stores;
    } else {
      WaitVectorMemory<kOddYounger>();
    }
    TileBarrier();
    copy_next_half();
    // Since the row loads at the top of the block: this half's copies.
    multiply_half(2 * block + 1, cur, next, std::integral_constant<int, 1>{},
                  std::integral_constant<int, kCopiesPerWave>{});
    if (++block_within == nb) {
      block_within = 0;
      behind_stores = finish_tile() ? kAhead : 0;
    }
    cur = next;
  }
  // The last two blocks: whatever copies and loads remain, complete drains.
  for (; block < total_blocks; ++block) {
    WaitVectorMemory<0>();
    TileBarrier();
    if (copy_half < total_halves) copy_next_half();
    if (block + 1 < total_blocks) load_next_block(next);
    multiply_half(2 * block, cur, next, std::integral_constant<int, 0>{}, kDrain);
    WaitVectorMemory<0>();
    TileBarrier();
    if (copy_half < total_halves) copy_next_half();
    multiply_half(2 * block + 1, cur, next, std::integral_constant<int, 1>{}, kDrain);
    if (++block_within == nb) {
      block_within = 0;
      finish_tile();
    }
    cur = next;
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
  // Activation bytes are addressed with 32 bits.
  if (blocks_per_row == 0 || tokens > 0xFFFFFFFFull / (512ull * blocks_per_row)) {
    return hipErrorInvalidValue;
  }
  const size_t octets = tokens * blocks_per_row * 32;
  hipLaunchKernelGGL(PrepareActivations, dim3(static_cast<uint32_t>((octets + 255) / 256)),
                     dim3(256), 0, stream, reinterpret_cast<const U32x4*>(a_bf16), octets,
                     static_cast<U32x4*>(workspace));
  hipError_t status = hipGetLastError();
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
  shape.nb = blocks_per_row;
  shape.tokens = static_cast<uint32_t>(tokens);
  shape.row_tiles = (rows + kTileRows - 1) / kTileRows;
  shape.token_tiles = static_cast<uint32_t>((tokens + kTileTokens - 1) / kTileTokens);
  shape.band = (shape.row_tiles + kXcds - 1) / kXcds;
  shape.total = shape.row_tiles * shape.token_tiles;
  shape.per_xcd = (shape.total + kXcds - 1) / kXcds;
  shape.vector_stores = (rows % 4 == 0 && reinterpret_cast<uintptr_t>(c) % 16 == 0) ? 1 : 0;
  // One workgroup per CU, the same number on every XCD, no more than there are tiles.
  uint32_t per_xcd_groups = static_cast<uint32_t>(DeviceComputeUnits()) / kXcds;
  if (per_xcd_groups == 0) per_xcd_groups = 1;
  if (per_xcd_groups > shape.per_xcd) per_xcd_groups = shape.per_xcd;
  hipLaunchKernelGGL(KquantGemmKernel, dim3(per_xcd_groups * kXcds), dim3(kGemmThreads),
                     lds_bytes, stream, w, static_cast<const uint8_t*>(workspace), c, shape);
  return hipGetLastError();
}

}  // namespace gufo
