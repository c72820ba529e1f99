// Mixture-of-experts control kernels: top-k routing, grouping of the (token, slot)
// pairs by expert, and the weighted combine.  The expert products themselves are
// KquantMoeGemvKernel in kquant_gemv.hip.
#include "kernels.hpp"
#include "kquant_common.hpp"

namespace gufo {
namespace {

// ---- routing -----------------------------------------------------------------
// qwen35::Route (src/models/qwen35/moe.cpp:16-42 of the reference): probabilities
// exp(logit - max) in double, the k largest in order (the lower index on equal
// probabilities), weights p/total/top with top = sum of the chosen p/total,
// floored at the smallest normal fp16.
//
// One workgroup per token, one thread per expert.  Instead of k rounds of a
// wave-wide arg-max, every thread counts the experts that precede its own in the
// reference's order (higher probability, or equal probability and lower index):
// that count is the expert's slot, and the experts whose count is below k are the
// chosen ones.  The order is total, so the result does not depend on scheduling.

constexpr int kRouteThreads = 256;
constexpr int kRoutePerThread = kMaxRouteExperts / kRouteThreads;

__global__ __launch_bounds__(kRouteThreads) void RouteKernel(
    const float* __restrict__ logits, int experts, int k, int* ids, float* weights) {
  __shared__ double lds_prob[kMaxRouteExperts];
  __shared__ double lds_chosen[kMaxRouteK];
  __shared__ double lds_wave[kRouteThreads / 64];
  __shared__ float lds_wave_max[kRouteThreads / 64];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const float* row = logits + static_cast<size_t>(blockIdx.x) * experts;

  float max_logit = -INFINITY;
  for (int e = tid; e < experts; e += kRouteThreads) max_logit = fmaxf(max_logit, row[e]);
  for (int off = 32; off > 0; off >>= 1) {
    max_logit = fmaxf(max_logit, __shfl_xor(max_logit, off, 64));
  }
  if (lane == 0) lds_wave_max[wave] = max_logit;
  __syncthreads();
  max_logit = fmaxf(fmaxf(lds_wave_max[0], lds_wave_max[1]),
                    fmaxf(lds_wave_max[2], lds_wave_max[3]));

  double prob[kRoutePerThread];
  double total = 0.0;
#pragma unroll
  for (int j = 0; j < kRoutePerThread; ++j) {
    const int e = tid + kRouteThreads * j;
    prob[j] = 0.0;
    if (e < experts) {
      prob[j] = exp(static_cast<double>(row[e]) - static_cast<double>(max_logit));
      lds_prob[e] = prob[j];
      total += prob[j];
    }
  }
  for (int off = 32; off > 0; off >>= 1) total += __shfl_xor(total, off, 64);
  if (lane == 0) lds_wave[wave] = total;
  __syncthreads();
  total = (lds_wave[0] + lds_wave[1]) + (lds_wave[2] + lds_wave[3]);

#pragma unroll
  for (int j = 0; j < kRoutePerThread; ++j) {
    const int e = tid + kRouteThreads * j;
    if (e >= experts) continue;
    const double mine = prob[j];
    int before = 0;
    for (int o = 0; o < experts; ++o) {
      const double other = lds_prob[o];
      before += (other > mine || (other == mine && o < e)) ? 1 : 0;
    }
    if (before < k) {
      ids[static_cast<size_t>(blockIdx.x) * k + before] = e;
      lds_chosen[before] = mine;
    }
  }
  __syncthreads();
  if (tid < k) {
    // top = sum over slots, in slot order, of p/total.
    double top = 0.0;
    for (int slot = 0; slot < k; ++slot) top += lds_chosen[slot] / total;
    top = fmax(top, 6.103515625e-5);
    weights[static_cast<size_t>(blockIdx.x) * k + tid] =
        static_cast<float>(lds_chosen[tid] / total / top);
  }
}

// ---- grouping ----------------------------------------------------------------
// Reference::Ffn's assigned[e] lists (src/models/qwen35/reference.cpp:562-565 of
// the reference) as a counting sort in one workgroup: histogram, exclusive scan,
// then one thread per expert walks the pairs in order, which keeps every list
// ascending without atomics on positions.

constexpr int kGroupThreads = 256;
constexpr int kGroupPerThread = kMaxGroupExperts / kGroupThreads;

// Exclusive prefix sums over the workgroup of one value per thread; *total gets the
// sum.  `scratch` holds one int per wave.
__device__ __forceinline__ int BlockExclusiveScan(int value, int* scratch, int* total) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  int inclusive = value;
  for (int off = 1; off < 64; off <<= 1) {
    const int up = __shfl_up(inclusive, off, 64);
    if (lane >= off) inclusive += up;
  }
  __syncthreads();  // scratch may still be read by an earlier scan
  if (lane == 63) scratch[wave] = inclusive;
  __syncthreads();
  int before = 0;
  int sum = 0;
  for (int w = 0; w < kGroupThreads / 64; ++w) {
    if (w < wave) before += scratch[w];
    sum += scratch[w];
  }
  *total = sum;
  return before + inclusive - value;
}

__global__ __launch_bounds__(kGroupThreads) void MoeGroupKernel(
    const int* __restrict__ ids, int n_pairs, int experts, int capacity, int* counts,
    int* offsets, int* pairs, uint8_t* pair_valid, MoeSegment* segments,
    MoeTables* tables) {
  __shared__ int lds_ids[kMaxGroupPairs];
  __shared__ int lds_count[kMaxGroupExperts];
  __shared__ int lds_scan[kGroupThreads / 64];
  __shared__ int lds_invalid;
  const int tid = threadIdx.x;

  if (tid == 0) lds_invalid = 0;
  for (int e = tid; e < kMaxGroupExperts; e += kGroupThreads) lds_count[e] = 0;
  __syncthreads();
  for (int i = tid; i < n_pairs; i += kGroupThreads) {
    const int e = ids[i];
    const bool ok = e >= 0 && e < experts;
    lds_ids[i] = ok ? e : -1;
    pair_valid[i] = ok ? 1 : 0;
    if (ok) {
      atomicAdd(&lds_count[e], 1);
    } else {
      atomicAdd(&lds_invalid, 1);
    }
  }
  __syncthreads();

  // Thread t owns experts t*kGroupPerThread .. +kGroupPerThread: their pair counts,
  // segment counts and "chosen at all" flags, scanned across the workgroup.
  int count[kGroupPerThread];
  int my_pairs = 0;
  int my_segments = 0;
  int my_distinct = 0;
#pragma unroll
  for (int j = 0; j < kGroupPerThread; ++j) {
    count[j] = lds_count[tid * kGroupPerThread + j];
    my_pairs += count[j];
    my_segments += (count[j] + capacity - 1) / capacity;
    my_distinct += count[j] != 0 ? 1 : 0;
  }
  int total_pairs, total_segments, total_distinct;
  int pair_offset = BlockExclusiveScan(my_pairs, lds_scan, &total_pairs);
  int segment_offset = BlockExclusiveScan(my_segments, lds_scan, &total_segments);
  BlockExclusiveScan(my_distinct, lds_scan, &total_distinct);
  if (tid == 0) {
    tables->n_segments = total_segments;
    tables->n_distinct = total_distinct;
    tables->n_invalid = lds_invalid;
    tables->pad = 0;
    offsets[experts] = total_pairs;
    // Invalid pairs go last so that `pairs` stays a permutation of the pair ids.
    int pos = total_pairs;
    for (int i = 0; i < n_pairs && pos < n_pairs; ++i) {
      if (lds_ids[i] < 0) pairs[pos++] = i;
    }
  }
#pragma unroll
  for (int j = 0; j < kGroupPerThread; ++j) {
    const int e = tid * kGroupPerThread + j;
    if (e >= experts) break;
    const int c = count[j];
    counts[e] = c;
    offsets[e] = pair_offset;
    int pos = pair_offset;
    int seg = segment_offset;
    pair_offset += c;
    segment_offset += (c + capacity - 1) / capacity;
    if (c == 0) continue;
    int in_seg = 0;
    for (int i = 0; i < n_pairs; ++i) {
      if (lds_ids[i] != e) continue;
      pairs[pos++] = i;
      segments[seg].pair[in_seg++] = i;
      if (in_seg == capacity) {
        segments[seg].expert = e;
        segments[seg].n_pairs = in_seg;
        for (int f = in_seg; f < kMaxGemvTokens; ++f) segments[seg].pair[f] = i;
        ++seg;
        in_seg = 0;
      }
    }
    if (in_seg != 0) {
      segments[seg].expert = e;
      segments[seg].n_pairs = in_seg;
      for (int f = in_seg; f < kMaxGemvTokens; ++f) {
        segments[seg].pair[f] = segments[seg].pair[0];
      }
    }
  }
}

// ---- combine -----------------------------------------------------------------
// out[t][i] = sum over slots in slot order of weight * routed row, in double
// (src/models/qwen35/reference.cpp:595-606 of the reference).  One fixed order,
// no atomics: repeated runs give identical bits.
__global__ __launch_bounds__(256) void MoeCombineKernel(
    const float* __restrict__ rows, const float* __restrict__ weights,
    const uint8_t* __restrict__ pair_valid, int k, int hidden, float* __restrict__ y) {
  const int t = blockIdx.y;
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= hidden) return;
  double acc = 0.0;
  for (int slot = 0; slot < k; ++slot) {
    const size_t s = static_cast<size_t>(t) * k + slot;
    if (pair_valid[s] == 0) continue;
    acc += static_cast<double>(weights[s]) * static_cast<double>(rows[s * hidden + i]);
  }
  y[static_cast<size_t>(t) * hidden + i] = static_cast<float>(acc);
}

}  // namespace

hipError_t LaunchRoute(const float* logits, int tokens, int experts, int k, int* ids,
                       float* weights, hipStream_t stream) {
  if (tokens < 0 || experts < 1 || experts > kMaxRouteExperts || k < 1 ||
      k > kMaxRouteK || k > experts) {
    return hipErrorInvalidValue;
  }
  if (tokens == 0) return hipSuccess;
  hipLaunchKernelGGL(RouteKernel, dim3(tokens), dim3(kRouteThreads), 0, stream, logits,
                     experts, k, ids, weights);
  return hipGetLastError();
}

hipError_t LaunchMoeGroup(const int* ids, int n_pairs, int experts, int capacity,
                          int* counts, int* offsets, int* pairs, uint8_t* pair_valid,
                          MoeSegment* segments, MoeTables* tables, hipStream_t stream) {
  if (n_pairs < 0 || n_pairs > kMaxGroupPairs || experts < 1 ||
      experts > kMaxGroupExperts || capacity < 1 || capacity > kMaxGemvTokens) {
    return hipErrorInvalidValue;
  }
  hipLaunchKernelGGL(MoeGroupKernel, dim3(1), dim3(kGroupThreads), 0, stream, ids,
                     n_pairs, experts, capacity, counts, offsets, pairs, pair_valid,
                     segments, tables);
  return hipGetLastError();
}

hipError_t LaunchMoeCombine(const float* rows, const float* weights,
                            const uint8_t* pair_valid, int tokens, int k, int hidden,
                            float* y, hipStream_t stream) {
  if (tokens <= 0 || hidden <= 0) return hipSuccess;
  hipLaunchKernelGGL(MoeCombineKernel, dim3((hidden + 255) / 256, tokens), dim3(256), 0,
                     stream, rows, weights, pair_valid, k, hidden, y);
  return hipGetLastError();
}

}  // namespace gufo
