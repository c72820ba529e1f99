// Small kernels beside the matrix products: the greedy pick over logits and a
// streaming-read probe that measures the read bandwidth a kernel can reach.
#include "kernels.hpp"
#include "kquant_common.hpp"

namespace gufo {
namespace {

__device__ __forceinline__ Best BlockBest(Best v) {
  __shared__ Best per_wave[4];
  v = WaveBest(v);
  if ((threadIdx.x & 63) == 0) per_wave[threadIdx.x >> 6] = v;
  __syncthreads();
  Best r = per_wave[0];
  for (int w = 1; w < 4; ++w) r = Better(r, per_wave[w]);
  return r;
}

__global__ __launch_bounds__(256) void ArgmaxPartial(const float* __restrict__ v,
                                                     uint32_t n, Best* partial) {
  Best best;
  best.value = -INFINITY;
  best.index = 0xFFFFFFFFu;
  for (uint32_t i = blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256) {
    Best c;
    c.value = v[i];
    c.index = i;
    best = Better(best, c);
  }
  best = BlockBest(best);
  if (threadIdx.x == 0) partial[blockIdx.x] = best;
}

__global__ __launch_bounds__(256) void ArgmaxFinal(const Best* partial, uint32_t count,
                                                   int64_t* out) {
  Best best;
  best.value = -INFINITY;
  best.index = 0xFFFFFFFFu;
  for (uint32_t i = threadIdx.x; i < count; i += 256) best = Better(best, partial[i]);
  best = BlockBest(best);
  if (threadIdx.x == 0) {
    // All -inf (or NaN) input: max_element returns the first element.
    *out = best.index == 0xFFFFFFFFu ? 0 : static_cast<int64_t>(best.index);
  }
}

__global__ __launch_bounds__(256) void ReadProbe(const U32x4* __restrict__ src,
                                                 size_t n_vec, uint32_t* sink) {
  uint32_t acc = 0;
  const size_t stride = static_cast<size_t>(gridDim.x) * 256;
  size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  // Eight independent 16-byte loads in flight per lane; consecutive workgroups read
  // consecutive 4 KB, so the requests in flight at any moment cover one contiguous region.
  constexpr int kInFlight = 8;
  for (; i + (kInFlight - 1) * stride < n_vec; i += kInFlight * stride) {
    U32x4 v[kInFlight];
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) v[u] = __builtin_nontemporal_load(src + i + u * stride);
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  for (; i < n_vec; i += stride) {
    const U32x4 a = src[i];
    acc ^= a.x ^ a.y ^ a.z ^ a.w;
  }
  // The loads must stay alive, the store must (almost) never happen: an atomic per
  // wave on one address would time the atomics, not the reads.
  if (acc == 0x9E3779B9u) *sink = acc;
}

__global__ __launch_bounds__(256) void WriteProbe(U32x4* __restrict__ dst, size_t n_vec) {
  const size_t stride = static_cast<size_t>(gridDim.x) * 256;
  const U32x4 value = {0x3F800000u, 0x3F800000u, 0x3F800000u, 0x3F800000u};
  for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < n_vec; i += stride) {
    dst[i] = value;
  }
}

}  // namespace

hipError_t LaunchWriteProbe(void* dst, size_t bytes, hipStream_t stream) {
  const size_t n_vec = bytes / 16;
  if (n_vec == 0) return hipSuccess;
  size_t blocks = (n_vec + 256 * 4 - 1) / (256 * 4);
  if (blocks > 256 * 16) blocks = 256 * 16;
  hipLaunchKernelGGL(WriteProbe, dim3(static_cast<uint32_t>(blocks)), dim3(256), 0, stream,
                     static_cast<U32x4*>(dst), n_vec);
  return hipGetLastError();
}

hipError_t LaunchArgmax(const float* v, size_t n, void* scratch, int64_t* out,
                        hipStream_t stream) {
  if (n == 0 || n > 0xFFFFFFF0ull) return hipErrorInvalidValue;
  Best* partial = static_cast<Best*>(scratch);
  uint32_t blocks = static_cast<uint32_t>((n + 1023) / 1024);
  if (blocks > static_cast<uint32_t>(kArgmaxBlocks)) blocks = kArgmaxBlocks;
  hipLaunchKernelGGL(ArgmaxPartial, dim3(blocks), dim3(256), 0, stream, v,
                     static_cast<uint32_t>(n), partial);
  hipLaunchKernelGGL(ArgmaxFinal, dim3(1), dim3(256), 0, stream, partial, blocks, out);
  return hipGetLastError();
}

hipError_t LaunchReadProbe(const void* src, size_t bytes, uint32_t* sink,
                           hipStream_t stream) {
  const size_t n_vec = bytes / 16;
  if (n_vec == 0) return hipSuccess;
  // At most three workgroups per compute unit: measured, a larger grid loses 20% (the
  // requests in flight then spread over too many DRAM pages at once).
  size_t blocks = (n_vec + 256 * 8 - 1) / (256 * 8);
  const size_t resident = static_cast<size_t>(DeviceComputeUnits()) * 3;
  if (blocks > resident) blocks = resident;
  hipLaunchKernelGGL(ReadProbe, dim3(static_cast<uint32_t>(blocks)), dim3(256), 0,
                     stream, static_cast<const U32x4*>(src), n_vec, sink);
  return hipGetLastError();
}

}  // namespace gufo
