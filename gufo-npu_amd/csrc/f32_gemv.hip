// Matrix-vector products over rows stored as fp32: gguf_dot::DotF32
// (src/models/qwen35/gguf_dot.hpp:71-75 of the reference) behind the same launch
// description as the K-quant kernels.  Real model files keep a few small tensors in
// fp32 (the MoE router and its shared-expert gate, the linear-attention alpha and beta
// projections), so this kernel is about latency, not bandwidth: one wave per row, the
// lanes stride over the row in float4 pieces, fp32 fma into one partial sum per lane,
// then a fixed-order butterfly over the wave.  A token column's arithmetic does not
// depend on how many columns the launch carries, so column t of an N-column call
// equals the one-column call bit for bit, as with the K-quant kernels.
#include "kernels.hpp"
#include "kquant_common.hpp"

namespace gufo {
namespace {

constexpr int kF32Threads = 256;
constexpr int kF32Waves = kF32Threads / 64;

typedef float Float4 __attribute__((ext_vector_type(4)));

struct F32Params {
  GemvLaunch launch;
  uint32_t start[kMaxGemvParts];  // first flat row of each part
  uint32_t cols;
};

template <int NTOK>
__global__ __launch_bounds__(kF32Threads) void F32GemvKernel(const F32Params prm,
                                                             const float* __restrict__ x,
                                                             float* __restrict__ y) {
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = blockIdx.x * kF32Waves + (threadIdx.x >> 6);
  const uint32_t waves = gridDim.x * kF32Waves;
  const uint32_t cols = prm.cols;
  for (uint32_t flat = wave; flat < prm.launch.total_rows; flat += waves) {
    // The part this row belongs to.
    const uint8_t* base = prm.launch.part[0].rows;
    uint32_t start = 0;
    uint32_t y_offset = prm.launch.part[0].y_offset;
#pragma unroll
    for (int p = 1; p < kMaxGemvParts; ++p) {
      if (p < static_cast<int>(prm.launch.n_parts) && flat >= prm.start[p]) {
        base = prm.launch.part[p].rows;
        start = prm.start[p];
        y_offset = prm.launch.part[p].y_offset;
      }
    }
    const float* row =
        reinterpret_cast<const float*>(base) + static_cast<size_t>(flat - start) * cols;
    float sum[NTOK];
#pragma unroll
    for (int t = 0; t < NTOK; ++t) sum[t] = 0.0f;
    // cols is a multiple of 256: every lane takes cols / 256 pieces.  Eight pieces of the
    // row are requested before the first is used; the sums run in piece order.
    constexpr int kAhead = 8;
    const uint32_t pieces = cols / 256;
    for (uint32_t first = 0; first < pieces; first += kAhead) {
      Float4 w[kAhead];
#pragma unroll
      for (int i = 0; i < kAhead; ++i) {
        const uint32_t piece = min(first + i, pieces - 1);
        w[i] = *reinterpret_cast<const Float4*>(row + 256 * piece + 4 * lane);
      }
#pragma unroll
      for (int i = 0; i < kAhead; ++i) {
        if (first + i >= pieces) break;
        const uint32_t k = 256 * (first + i) + 4 * lane;
#pragma unroll
        for (int t = 0; t < NTOK; ++t) {
          const Float4 v =
              *reinterpret_cast<const Float4*>(x + static_cast<size_t>(t) * cols + k);
          sum[t] = __builtin_fmaf(w[i].x, v.x, sum[t]);
          sum[t] = __builtin_fmaf(w[i].y, v.y, sum[t]);
          sum[t] = __builtin_fmaf(w[i].z, v.z, sum[t]);
          sum[t] = __builtin_fmaf(w[i].w, v.w, sum[t]);
        }
      }
    }
#pragma unroll
    for (int t = 0; t < NTOK; ++t) {
      float total = sum[t];
      for (int off = 32; off > 0; off >>= 1) total += __shfl_xor(total, off, 64);
      if (lane == 0) {
        y[static_cast<size_t>(t) * prm.launch.y_stride + y_offset + (flat - start)] = total;
      }
    }
  }
}

template <int NTOK>
hipError_t LaunchF32(const F32Params& prm, const float* x, float* y, dim3 grid,
                     hipStream_t stream) {
  hipLaunchKernelGGL((F32GemvKernel<NTOK>), grid, dim3(kF32Threads), 0, stream, prm, x, y);
  return hipGetLastError();
}

}  // namespace

hipError_t LaunchGemvF32(const GemvLaunch& launch, const float* x, int tokens, float* y,
                         hipStream_t stream) {
  if (launch.n_parts < 1 || launch.n_parts > static_cast<uint32_t>(kMaxGemvParts) ||
      launch.blocks_per_row == 0 || tokens < 1 || tokens > kMaxGemvTokens) {
    return hipErrorInvalidValue;
  }
  if (launch.total_rows == 0) return hipSuccess;
  F32Params prm;
  prm.launch = launch;
  prm.cols = launch.blocks_per_row * kSuperBlock;
  uint32_t start = 0;
  for (uint32_t p = 0; p < static_cast<uint32_t>(kMaxGemvParts); ++p) {
    prm.start[p] = start;
    if (p < launch.n_parts) start += launch.part[p].n_rows;
  }
  uint32_t blocks = (launch.total_rows + kF32Waves - 1) / kF32Waves;
  const uint32_t resident = static_cast<uint32_t>(DeviceComputeUnits()) * 8;
  if (blocks > resident) blocks = resident;
  const dim3 grid(blocks);
  switch (tokens) {
    case 1: return LaunchF32<1>(prm, x, y, grid, stream);
    case 2: return LaunchF32<2>(prm, x, y, grid, stream);
    case 3: return LaunchF32<3>(prm, x, y, grid, stream);
    default: return LaunchF32<4>(prm, x, y, grid, stream);
  }
}

}  // namespace gufo
