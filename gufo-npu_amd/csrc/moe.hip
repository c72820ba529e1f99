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
// One workgroup per token, one thread per expert (four at 1024 experts).  Instead of k
// rounds of a workgroup-wide arg-max, a thread counts the experts that precede its own
// in the reference's order (higher probability, or equal probability and lower
// index): that count is the expert's slot, and the experts whose count is below k are
// the chosen ones.  The order is total, so the result does not depend on scheduling.
//
// Counting against every expert would be experts^2 comparisons, so it runs in two
// levels.  First inside chunks of 64 experts: an expert preceded by k others of its own
// chunk cannot be chosen.  The survivors (at most k per chunk) are listed, and each
// counts its predecessors among the survivors only - which is its true count whenever
// that is below k, because everything that precedes a chosen expert is itself chosen
// and so survived its own chunk.

constexpr int kRouteThreads = 256;
constexpr int kRoutePerThread = kMaxRouteExperts / kRouteThreads;
constexpr int kRouteChunk = 64;

typedef double Double2 __attribute__((ext_vector_type(2)));

// Whether expert `other_index` with probability `other` precedes (mine, my_index).
__device__ __forceinline__ int Precedes(double other, int other_index, double mine, int my_index) {
  return (other > mine || (other == mine && other_index < my_index)) ? 1 : 0;
}

__global__ __launch_bounds__(kRouteThreads) void RouteKernel(
    const float* __restrict__ logits, size_t logit_stride, int experts, int k, int* ids,
    float* weights) {
  __shared__ __align__(16) double lds_prob[kMaxRouteExperts];
  __shared__ __align__(16) double lds_survivor[kMaxRouteExperts];
  __shared__ int lds_survivor_index[kMaxRouteExperts];
  __shared__ double lds_chosen[kMaxRouteK];
  __shared__ double lds_wave[kRouteThreads / 64];
  __shared__ float lds_wave_max[kRouteThreads / 64];
  __shared__ int lds_survivors;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const float* row = logits + static_cast<size_t>(blockIdx.x) * logit_stride;
  const int padded = (experts + kRouteChunk - 1) / kRouteChunk * kRouteChunk;

  float logit[kRoutePerThread];
  float max_logit = -INFINITY;
#pragma unroll
  for (int j = 0; j < kRoutePerThread; ++j) {
    const int e = tid + kRouteThreads * j;
    logit[j] = e < experts ? row[e] : -INFINITY;
    max_logit = fmaxf(max_logit, logit[j]);
  }
  for (int off = 32; off > 0; off >>= 1) {
    max_logit = fmaxf(max_logit, __shfl_xor(max_logit, off, 64));
  }
  if (lane == 0) lds_wave_max[wave] = max_logit;
  if (tid == 0) lds_survivors = 0;
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
      prob[j] = exp(static_cast<double>(logit[j]) - static_cast<double>(max_logit));
      lds_prob[e] = prob[j];
      total += prob[j];
    } else if (e < padded) {
      lds_prob[e] = -1.0;  // precedes nothing
    }
  }
  for (int off = 32; off > 0; off >>= 1) total += __shfl_xor(total, off, 64);
  if (lane == 0) lds_wave[wave] = total;
  __syncthreads();
  total = (lds_wave[0] + lds_wave[1]) + (lds_wave[2] + lds_wave[3]);

  // Level one: predecessors inside the expert's own chunk of 64.
  int mine_slot[kRoutePerThread];
#pragma unroll
  for (int j = 0; j < kRoutePerThread; ++j) {
    const int e = tid + kRouteThreads * j;
    mine_slot[j] = -1;
    if (e >= experts) continue;
    const int base = e & ~(kRouteChunk - 1);
    const Double2* chunk = reinterpret_cast<const Double2*>(lds_prob + base);
    int before = 0;
#pragma unroll
    for (int i = 0; i < kRouteChunk / 2; ++i) {
      const Double2 others = chunk[i];
      before += Precedes(others.x, base + 2 * i, prob[j], e);
      before += Precedes(others.y, base + 2 * i + 1, prob[j], e);
    }
    if (before < k) {
      mine_slot[j] = atomicAdd(&lds_survivors, 1);
      lds_survivor[mine_slot[j]] = prob[j];
      lds_survivor_index[mine_slot[j]] = e;
    }
  }
  __syncthreads();

  // Level two: predecessors among the survivors.
  const int survivors = lds_survivors;
#pragma unroll
  for (int j = 0; j < kRoutePerThread; ++j) {
    if (mine_slot[j] < 0) continue;
    const int e = tid + kRouteThreads * j;
    int before = 0;
    int s = 0;
    for (; s + 4 <= survivors; s += 4) {
      const Double2 a = *reinterpret_cast<const Double2*>(lds_survivor + s);
      const Double2 b = *reinterpret_cast<const Double2*>(lds_survivor + s + 2);
      before += Precedes(a.x, lds_survivor_index[s], prob[j], e);
      before += Precedes(a.y, lds_survivor_index[s + 1], prob[j], e);
      before += Precedes(b.x, lds_survivor_index[s + 2], prob[j], e);
      before += Precedes(b.y, lds_survivor_index[s + 3], prob[j], e);
    }
    for (; s < survivors; ++s) {
      before += Precedes(lds_survivor[s], lds_survivor_index[s], prob[j], e);
    }
    if (before < k) {
      ids[static_cast<size_t>(blockIdx.x) * k + before] = e;
      lds_chosen[before] = prob[j];
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

// The segment list alone, for a call of at most 64 pairs (a decode step: a few tokens
// times k), in one wave with no LDS: lane i owns pair i and learns, from the other
// lanes' expert ids read lane by lane into scalar registers, how many earlier pairs
// chose the same expert (its place in the expert's list), how many pairs did
// altogether, and how many segments the lower-numbered experts take.  Segments come
// out in ascending expert order with ascending pairs, as MoeGroupKernel writes them.
__global__ __launch_bounds__(64) void MoeGroupSmallKernel(
    const int* __restrict__ ids, int n_pairs, int experts, int capacity,
    uint8_t* pair_valid, MoeSegment* segments, MoeTables* tables) {
  const int lane = threadIdx.x;
  const bool present = lane < n_pairs;
  int expert = present ? ids[lane] : -1;
  const bool valid = present && expert >= 0 && expert < experts;
  if (!valid) expert = -1;
  if (present) pair_valid[lane] = valid ? 1 : 0;

  int place = 0;  // earlier pairs of the same expert
  int count = 0;  // all pairs of the same expert
  for (int j = 0; j < n_pairs; ++j) {
    const int other = __builtin_amdgcn_readlane(expert, j);
    const bool same = valid && other == expert;
    place += (same && j < lane) ? 1 : 0;
    count += same ? 1 : 0;
  }
  const bool leads = valid && place == 0;
  const int own_segments = leads ? (count + capacity - 1) / capacity : 0;
  int first_segment = 0;   // segments of lower-numbered experts
  int total_segments = 0;
  int distinct = 0;
  for (int j = 0; j < n_pairs; ++j) {
    const int other_segments = __builtin_amdgcn_readlane(own_segments, j);
    if (other_segments == 0) continue;  // uniform
    const int other = __builtin_amdgcn_readlane(expert, j);
    first_segment += (valid && other < expert) ? other_segments : 0;
    total_segments += other_segments;
    ++distinct;
  }
  if (valid) {
    const int segment = first_segment + place / capacity;
    const int slot = place - (place / capacity) * capacity;
    segments[segment].pair[slot] = lane;
    if (slot == 0) {
      const int here = min(capacity, count - place);
      segments[segment].expert = expert;
      segments[segment].n_pairs = here;
      // Unused entries repeat a pair of the segment, so that reading them is harmless.
      for (int f = here; f < kMaxGemvTokens; ++f) segments[segment].pair[f] = lane;
    }
  }
  const int invalid = __builtin_popcountll(__ballot(present && !valid));
  if (lane == 0) {
    tables->n_segments = total_segments;
    tables->n_distinct = distinct;
    tables->n_invalid = invalid;
    tables->pad = 0;
  }
}

// ---- combine -----------------------------------------------------------------
// out[t][i] = sum over slots in slot order of weight * routed row, in double
// (src/models/qwen35/reference.cpp:595-606 of the reference).  One fixed order,
// no atomics: repeated runs give identical bits.
//
// With a shared expert the sum starts from its output times SharedExpertScale of the
// token's gate logit, sigmoid in double rounded to fp32, the product in fp32
// (src/models/qwen35/moe.cpp:44-47, decoder.cpp:539-542).
__device__ __forceinline__ double SharedTerm(const MoeShared& shared, int t, int hidden, int i) {
  if (shared.rows == nullptr) return 0.0;
  const double logit = static_cast<double>(shared.gate_logit[static_cast<size_t>(t) * shared.gate_stride]);
  const float scale = static_cast<float>(1.0 / (1.0 + exp(-logit)));
  return static_cast<double>(shared.rows[static_cast<size_t>(t) * hidden + i] * scale);
}

__global__ __launch_bounds__(256) void MoeCombineKernel(
    const float* __restrict__ rows, const float* __restrict__ weights,
    const uint8_t* __restrict__ pair_valid, int k, int hidden, const MoeShared shared,
    float* y) {  // may be shared.rows: every thread reads its element before writing it
  const int t = blockIdx.y;
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= hidden) return;
  double acc = SharedTerm(shared, t, hidden, i);
  for (int slot = 0; slot < k; ++slot) {
    const size_t s = static_cast<size_t>(t) * k + slot;
    if (pair_valid[s] == 0) continue;
    acc += static_cast<double>(weights[s]) * static_cast<double>(rows[s * hidden + i]);
  }
  y[static_cast<size_t>(t) * hidden + i] = static_cast<float>(acc);
}

// One token, pairs not grouped: validity comes from the ids themselves, and thread 0 of
// the launch writes the header the grouping kernel would have written.
__global__ __launch_bounds__(256) void MoeCombineDirectKernel(
    const float* __restrict__ rows, const float* __restrict__ weights,
    const int32_t* __restrict__ ids, int experts, int k, int hidden, const MoeShared shared,
    float* y, MoeTables* tables) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i == 0) {
    int invalid = 0;
    int distinct = 0;
    for (int s = 0; s < k; ++s) {
      const int e = ids[s];
      if (e < 0 || e >= experts) {
        ++invalid;
        continue;
      }
      bool seen = false;
      for (int r = 0; r < s; ++r) seen = seen || ids[r] == e;
      distinct += seen ? 0 : 1;
    }
    tables->n_segments = k - invalid;
    tables->n_distinct = distinct;
    tables->n_invalid = invalid;
    tables->pad = 0;
  }
  if (i >= hidden) return;
  double acc = SharedTerm(shared, 0, hidden, i);
  for (int slot = 0; slot < k; ++slot) {
    const int e = ids[slot];
    if (e < 0 || e >= experts) continue;
    acc += static_cast<double>(weights[slot]) *
           static_cast<double>(rows[static_cast<size_t>(slot) * hidden + i]);
  }
  y[i] = static_cast<float>(acc);
}

}  // namespace

hipError_t LaunchMoeCombineDirect(const float* rows, const float* weights, const int32_t* ids,
                                  int experts, int k, int hidden, const MoeShared& shared,
                                  float* y, MoeTables* tables, hipStream_t stream) {
  if (hidden <= 0 || k <= 0) return hipErrorInvalidValue;
  hipLaunchKernelGGL(MoeCombineDirectKernel, dim3((hidden + 255) / 256), dim3(256), 0, stream,
                     rows, weights, ids, experts, k, hidden, shared, y, tables);
  return hipGetLastError();
}

hipError_t LaunchRoute(const float* logits, size_t logit_stride, int tokens, int experts, int k,
                       int* ids, float* weights, hipStream_t stream) {
  if (tokens < 0 || experts < 1 || experts > kMaxRouteExperts || k < 1 ||
      k > kMaxRouteK || k > experts || logit_stride < static_cast<size_t>(experts)) {
    return hipErrorInvalidValue;
  }
  if (tokens == 0) return hipSuccess;
  hipLaunchKernelGGL(RouteKernel, dim3(tokens), dim3(kRouteThreads), 0, stream, logits,
                     logit_stride, experts, k, ids, weights);
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

hipError_t LaunchMoeGroupSmall(const int* ids, int n_pairs, int experts, int capacity,
                               uint8_t* pair_valid, MoeSegment* segments, MoeTables* tables,
                               hipStream_t stream) {
  if (n_pairs < 0 || n_pairs > kMaxSmallGroupPairs || experts < 1 || capacity < 1 ||
      capacity > kMaxGemvTokens) {
    return hipErrorInvalidValue;
  }
  hipLaunchKernelGGL(MoeGroupSmallKernel, dim3(1), dim3(64), 0, stream, ids, n_pairs, experts,
                     capacity, pair_valid, segments, tables);
  return hipGetLastError();
}

hipError_t LaunchMoeCombine(const float* rows, const float* weights,
                            const uint8_t* pair_valid, int tokens, int k, int hidden,
                            const MoeShared& shared, float* y, hipStream_t stream) {
  if (tokens <= 0 || hidden <= 0) return hipSuccess;
  hipLaunchKernelGGL(MoeCombineKernel, dim3((hidden + 255) / 256, tokens), dim3(256), 0,
                     stream, rows, weights, pair_valid, k, hidden, shared, y);
  return hipGetLastError();
}

}  // namespace gufo
