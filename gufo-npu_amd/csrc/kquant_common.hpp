// Device-side helpers shared by the K-quant kernels: block geometry, fp16
// conversion, unaligned vector loads and the 6-bit scale unpack.
//
// Block layouts (src/core/quant.cpp:32,61,97 of the reference):
//   Q4_K 144 B: d, dmin (fp16) | 12 packed scale bytes | qs[128]
//   Q5_K 176 B: d, dmin (fp16) | 12 packed scale bytes | qh[32] | qs[128]
//   Q6_K 210 B: ql[128] | qh[64] | int8 scales[16] | d (fp16)
//   Q8_0  34 B: d (fp16) | 32 int8          (src/core/quant.cpp:22-31), 32 values
//   F32    4 B: the value
// The kernels walk every row in steps of 256 values - one K-quant super-block, eight
// Q8_0 blocks or 256 floats - so every row length is a multiple of 256.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace gufo {

constexpr int kTypeF32 = 0;
constexpr int kTypeQ80 = 8;
constexpr int kTypeQ4K = 12;
constexpr int kTypeQ5K = 13;
constexpr int kTypeQ6K = 14;
constexpr int kSuperBlock = 256;

// Bytes of 256 consecutive values of a row; 0 for a type the kernels do not take.
__host__ __device__ constexpr int BlockBytes(int type) {
  return type == kTypeQ4K   ? 144
         : type == kTypeQ5K ? 176
         : type == kTypeQ6K ? 210
         : type == kTypeQ80 ? 8 * 34
         : type == kTypeF32 ? 256 * 4
                            : 0;
}

// Bytes and values of one block as the GGUF format defines it
// (src/core/quant.cpp:186-219 of the reference).
__host__ __device__ constexpr int FormatBlockBytes(int type) {
  return type == kTypeQ80 ? 34 : type == kTypeF32 ? 4 : BlockBytes(type);
}
__host__ __device__ constexpr int FormatBlockValues(int type) {
  return type == kTypeQ80 ? 32 : type == kTypeF32 ? 1 : BlockBytes(type) != 0 ? 256 : 0;
}

// fp16 bits -> fp32, exact for every input (subnormals included): the hardware
// conversion v_cvt_f32_f16.
__device__ __forceinline__ float HalfBitsToFloat(uint32_t bits) {
  return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(bits)));
}

// Vector loads from addresses that are only 2-byte aligned (Q6_K blocks are
// 210 bytes).  gfx950 global loads take any byte alignment.
typedef uint32_t U32x2A2 __attribute__((ext_vector_type(2), aligned(2)));
typedef uint32_t U32x4A2 __attribute__((ext_vector_type(4), aligned(2)));
typedef uint32_t U32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t U32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ U32x2 Load8Align2(const uint8_t* p) {
  const U32x2A2 v = *reinterpret_cast<const U32x2A2*>(p);
  return U32x2{v.x, v.y};
}
__device__ __forceinline__ U32x4 Load16Align2(const uint8_t* p) {
  const U32x4A2 v = *reinterpret_cast<const U32x4A2*>(p);
  return U32x4{v.x, v.y, v.z, v.w};
}
__device__ __forceinline__ U32x4 Load16(const uint8_t* p) {
  return *reinterpret_cast<const U32x4*>(p);
}
__device__ __forceinline__ uint32_t Load2(const uint8_t* p) {
  return *reinterpret_cast<const uint16_t*>(p);
}

// 6-bit scale and min of sub-block j (0..7) from the 12 packed bytes held in
// three dwords s0 (bytes 0-3), s1 (bytes 4-7), s2 (bytes 8-11): the bit layout of
// quant::ScaleMinK4 (src/core/quant.cpp:158-167 of the reference).
__device__ __forceinline__ void ScaleMinK4(uint32_t s0, uint32_t s1, uint32_t s2,
                                           int j, uint32_t* scale, uint32_t* min) {
  const int sh = 8 * (j & 3);
  const uint32_t a = s0 >> sh;  // byte j&3 of bytes 0-3
  const uint32_t b = s1 >> sh;  // byte j&3 of bytes 4-7
  const uint32_t c = s2 >> sh;  // byte j&3 of bytes 8-11
  const uint32_t lo_scale = a & 63u;
  const uint32_t lo_min = b & 63u;
  const uint32_t hi_scale = (c & 15u) | ((a >> 2) & 0x30u);
  const uint32_t hi_min = ((c >> 4) & 15u) | ((b >> 2) & 0x30u);
  *scale = j < 4 ? lo_scale : hi_scale;
  *min = j < 4 ? lo_min : hi_min;
}

// The four bytes of `w` as floats (v_cvt_f32_ubyte0..3).
__device__ __forceinline__ float Byte0(uint32_t w) { return static_cast<float>(w & 0xFFu); }
__device__ __forceinline__ float Byte1(uint32_t w) { return static_cast<float>((w >> 8) & 0xFFu); }
__device__ __forceinline__ float Byte2(uint32_t w) { return static_cast<float>((w >> 16) & 0xFFu); }
__device__ __forceinline__ float Byte3(uint32_t w) { return static_cast<float>(w >> 24); }

// Sum over the lanes of a power-of-two group of `width` consecutive lanes; every
// lane of the group ends with the total.  The order of additions depends only on
// `width`, so results repeat bit for bit.
__device__ __forceinline__ float GroupSum(float v, int width) {
  for (int off = 1; off < width; off <<= 1) {
    v += __shfl_xor(v, off, 64);
  }
  return v;
}

// A candidate of the greedy pick: a value and where it stands.
struct Best {
  float value;
  uint32_t index;
};
constexpr uint32_t kNoIndex = 0xFFFFFFFFu;

// The better of two candidates under std::max_element's rule (first maximum
// wins): the larger value, the lower index on equal values
// (src/core/sampling.cpp:327-329 of the reference).  A total order on (value, index)
// pairs without NaN, so the result does not depend on the order of reduction; a NaN
// never replaces anything.
__device__ __forceinline__ Best Better(Best a, Best b) {
  const bool take_b = b.value > a.value || (b.value == a.value && b.index < a.index);
  return take_b ? b : a;
}

__device__ __forceinline__ Best WaveBest(Best v) {
  for (int off = 32; off > 0; off >>= 1) {
    Best o;
    o.value = __shfl_xor(v.value, off, 64);
    o.index = __shfl_xor(v.index, off, 64);
    v = Better(v, o);
  }
  return v;
}

}  // namespace gufo
