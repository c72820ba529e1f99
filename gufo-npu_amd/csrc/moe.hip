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
// floored at the smallest normal fp16.  One wave per token; lane l holds experts
// l, l+64, ...

struct Candidate {
  double prob;
  int index;
};

__device__ __forceinline__ Candidate BetterCandidate(Candidate a, Candidate b) {
  const bool take_b = b.prob > a.prob || (b.prob == a.prob && b.index < a.index);
  return take_b ? b : a;
}

constexpr int kRoutePerLane = kMaxRouteExperts / 64;

__global__ __launch_bounds__(64) void RouteKernel(const float* __restrict__ logits,
                                                  int experts, int k, int* ids,
                                                  float* weights) {
  const int lane = threadIdx.x;
  const float* row = logits + static_cast<size_t>(blockIdx.x) * experts;

  float max_logit = -INFINITY;
  for (int e = lane; e < experts; e += 64) max_logit = fmaxf(max_logit, row[e]);
  for (int off = 32; off > 0; off >>= 1) {
    max_logit = fmaxf(max_logit, __shfl_xor(max_logit, off, 64));
  }

  // prob < 0 marks "no expert here" or "already chosen".
  double prob[kRoutePerLane];
  double total = 0.0;
#pragma unroll
  for (int j = 0; j < kRoutePerLane; ++j) {
    const int e = lane + 64 * j;
    prob[j] = -1.0;
    if (e < experts) {
      prob[j] = exp(static_cast<double>(row[e]) - static_cast<double>(max_logit));
      total += prob[j];
    }
  }
  for (int off = 32; off > 0; off >>= 1) total += __shfl_xor(total, off, 64);

  double my_prob = 0.0;  // lane `slot` keeps the slot's probability
  int my_index = 0;
  for (int slot = 0; slot < k; ++slot) {
    Candidate best;
    best.prob = -1.0;
    best.index = 0x7FFFFFFF;
#pragma unroll
    for (int j = 0; j < kRoutePerLane; ++j) {
      Candidate c;
      c.prob = prob[j];
      c.index = lane + 64 * j;
      if (prob[j] >= 0.0) best = BetterCandidate(best, c);
    }
    for (int off = 32; off > 0; off >>= 1) {
      Candidate o;
      o.prob = __shfl_xor(best.prob, off, 64);
      o.index = __shfl_xor(best.index, off, 64);
      best = BetterCandidate(best, o);
    }
    // The owner retires the winner.
#pragma unroll
    for (int j = 0; j < kRoutePerLane; ++j) {
      if (lane + 64 * j == best.index) prob[j] = -1.0;
    }
    if (lane == slot) {
      my_prob = best.prob;
      my_index = best.index;
    }
  }

  // top = sum over slots, in slot order, of p/total.
  double top = 0.0;
  for (int slot = 0; slot < k; ++slot) {
    const double p = __shfl(my_prob, slot, 64);
    top += p / total;
  }
  top = fmax(top, 6.103515625e-5);
  if (lane < k) {
    ids[static_cast<size_t>(blockIdx.x) * k + lane] = my_index;
    weights[static_cast<size_t>(blockIdx.x) * k + lane] =
        static_cast<float>(my_prob / total / top);
  }
}

// ---- grouping ----------------------------------------------------------------
// Reference::Ffn's assigned[e] lists (src/models/qwen35/reference.cpp:562-565 of
// the reference) as a counting sort in one workgroup: histogram, exclusive scan,
// then one thread per expert walks the pairs in order, which keeps every list
// ascending without atomics on positions.

constexpr int kGroupThreads = 256;

__global__ __launch_bounds__(kGroupThreads) void MoeGroupKernel(
    const int* __restrict__ ids, int n_pairs, int experts, int capacity, int* counts,
    int* offsets, int* pairs, uint8_t* pair_valid, MoeSegment* segments,
    MoeTables* tables) {
  __shared__ int lds_ids[kMaxGroupPairs];
  __shared__ int lds_count[kMaxGroupExperts];
  __shared__ int lds_offset[kMaxGroupExperts + 1];
  __shared__ int lds_segment0[kMaxGroupExperts + 1];
  __shared__ int lds_invalid;
  const int tid = threadIdx.x;

  if (tid == 0) lds_invalid = 0;
  for (int e = tid; e < experts; e += kGroupThreads) lds_count[e] = 0;
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
  if (tid == 0) {
    int offset = 0;
    int segment = 0;
    int distinct = 0;
    for (int e = 0; e < experts; ++e) {
      const int c = lds_count[e];
      lds_offset[e] = offset;
      lds_segment0[e] = segment;
      offset += c;
      segment += (c + capacity - 1) / capacity;
      distinct += c != 0 ? 1 : 0;
    }
    lds_offset[experts] = offset;
    lds_segment0[experts] = segment;
    tables->n_segments = segment;
    tables->n_distinct = distinct;
    tables->n_invalid = lds_invalid;
    tables->pad = 0;
  }
  __syncthreads();
  for (int e = tid; e <= experts; e += kGroupThreads) {
    offsets[e] = lds_offset[e];
    if (e < experts) counts[e] = lds_count[e];
  }
  // Invalid pairs go last so that `pairs` stays a permutation of the pair ids.
  if (tid == 0) {
    int pos = lds_offset[experts];
    for (int i = 0; i < n_pairs; ++i) {
      if (lds_ids[i] < 0) pairs[pos++] = i;
    }
  }
  for (int e = tid; e < experts; e += kGroupThreads) {
    const int c = lds_count[e];
    if (c == 0) continue;
    int pos = lds_offset[e];
    int seg = lds_segment0[e];
    int in_seg = 0;
    for (int i = 0; i < n_pairs; ++i) {
      if (lds_ids[i] != e) continue;
      pairs[pos++] = i;
      segments[seg].pair[in_seg++] = i;
      if (in_seg == capacity) {
        segments[seg].expert = e;
        segments[seg].n_pairs = in_seg;
        ++seg;
        in_seg = 0;
      }
    }
    if (in_seg != 0) {
      segments[seg].expert = e;
      segments[seg].n_pairs = in_seg;
      for (int j = in_seg; j < kMaxGemvTokens; ++j) {
        segments[seg].pair[j] = segments[seg].pair[0];
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
  hipLaunchKernelGGL(RouteKernel, dim3(tokens), dim3(64), 0, stream, logits, experts, k,
                     ids, weights);
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
                     n_pairs, experts, capacity, counts, offsets, pairs, pair_valid, segments,
                     tables);
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
