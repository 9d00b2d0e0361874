// Routing glue around the grouped matmul of an expert MLP: a stable counting sort of the flattened
// top-k expert ids (which yields the expert-sorted row order and the cumulative int64 group_list the
// grouped matmul consumes), the row gather into that order, and the weighted combine back to token
// order.  The reference leaves these steps to its caller and only shows the construction of
// group_list on the host (benchmark/test_grouped_matmul.py:46-50: sort the expert ids, count,
// cumulative sum); here they run on the device so that the MoE layer needs no host round trip.
//
// Sort: ids are cut into slices of kSlice consecutive entries, one wave per slice.
//   moe_hist_kernel    per-slice histogram over experts (ids outside [0, E) count as bucket E)
//   moe_scan_kernel    one workgroup: per expert the exclusive prefix over slices, then the exclusive
//                      prefix over experts; writes group_list
//   moe_scatter_kernel every wave walks its slice in order, 64 ids at a time; lanes with equal ids
//                      find each other with one ballot per id bit and are ranked by lane number, so
//                      the sort is stable and its result does not depend on scheduling
#include "aops_common.h"

namespace aops {

constexpr int kSlice = 512;
constexpr int kMoeWaves = 4;         // waves (= slices) per workgroup of the histogram/scatter kernels
constexpr int kMoeMaxExperts = 4095; // (E + 1) ints per wave must fit the LDS: 4 x 4096 x 4 B

__device__ __forceinline__ int moe_bucket(int id, int num_experts) {
  return (id < 0 || id >= num_experts) ? num_experts : id;
}

__global__ __launch_bounds__(kMoeWaves* kWave) void moe_hist_kernel(
    const int32_t* __restrict__ ids, int64_t n, int num_experts, int num_slices,
    int32_t* __restrict__ counts /* [num_slices][E+1] */) {
  extern __shared__ int32_t hist_lds[];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int slice = blockIdx.x * kMoeWaves + wave;
  const int buckets = num_experts + 1;
  int32_t* h = hist_lds + wave * buckets;
  if (slice >= num_slices) return;  // wave uniform; no workgroup barrier below
  for (int e = lane; e < buckets; e += kWave) h[e] = 0;
  const int64_t begin = (int64_t)slice * kSlice;
  int idv[kSlice / kWave];  // all loads first: one memory latency per slice instead of eight
#pragma unroll
  for (int b = 0; b < kSlice / kWave; ++b) {
    const int64_t i = begin + b * kWave + lane;
    idv[b] = i < n ? ids[i] : -1;
  }
#pragma unroll
  for (int b = 0; b < kSlice / kWave; ++b) {
    const int64_t i = begin + b * kWave + lane;
    if (i < n) atomicAdd(&h[moe_bucket(idv[b], num_experts)], 1);
  }
  int32_t* out = counts + (int64_t)slice * buckets;
  for (int e = lane; e < buckets; e += kWave) out[e] = h[e];
}

// counts[slice][e] -> exclusive prefix over slices (in place); base[e] = exclusive prefix of the
// per-expert totals; group_list[e] = base[e] + total[e] for e < E.  One workgroup of 16 waves:
// a wave scans one expert's column across the slices (slices along the lanes), then the
// workgroup scans the per-expert totals.
__global__ __launch_bounds__(1024) void moe_scan_kernel(int32_t* __restrict__ counts, int num_slices,
                                                         int num_experts, int32_t* __restrict__ base,
                                                         int64_t* __restrict__ group_list) {
  __shared__ int32_t totals[kMoeMaxExperts + 1];
  __shared__ int32_t wave_sums[16];
  __shared__ int32_t carry;
  const int buckets = num_experts + 1;
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  constexpr int kCols = 8;  // expert columns a wave scans together (their loads overlap)
  for (int e0 = wave * kCols; e0 < buckets; e0 += 16 * kCols) {
    int running[kCols];
#pragma unroll
    for (int j = 0; j < kCols; ++j) running[j] = 0;
    for (int s0 = 0; s0 < num_slices; s0 += kWave) {
      const int s = s0 + lane;
      int c[kCols];
#pragma unroll
      for (int j = 0; j < kCols; ++j)
        c[j] = (s < num_slices && e0 + j < buckets) ? counts[(int64_t)s * buckets + e0 + j] : 0;
#pragma unroll
      for (int j = 0; j < kCols; ++j) {
        int incl = c[j];
#pragma unroll
        for (int d = 1; d < kWave; d <<= 1) {
          const int up = __shfl_up(incl, d);
          if (lane >= d) incl += up;
        }
        if (s < num_slices && e0 + j < buckets)
          counts[(int64_t)s * buckets + e0 + j] = running[j] + incl - c[j];
        running[j] += __shfl(incl, kWave - 1);
      }
    }
#pragma unroll
    for (int j = 0; j < kCols; ++j)
      if (lane == 0 && e0 + j < buckets) totals[e0 + j] = running[j];
  }
  if (tid == 0) carry = 0;
  __syncthreads();
  for (int e0 = 0; e0 < buckets; e0 += 1024) {
    const int e = e0 + tid;
    const int total = e < buckets ? totals[e] : 0;
    int incl = total;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
      const int up = __shfl_up(incl, d);
      if (lane >= d) incl += up;
    }
    if (lane == kWave - 1) wave_sums[wave] = incl;
    __syncthreads();
    int before = carry;
    for (int w = 0; w < wave; ++w) before += wave_sums[w];
    const int excl = before + incl - total;
    if (e < buckets) {
      base[e] = excl;
      if (e < num_experts) group_list[e] = (int64_t)excl + total;
    }
    __syncthreads();
    if (tid == 1023) carry = excl + total;
    __syncthreads();
  }
}

// SCAN = false: counts holds the exclusive prefixes over the slices and base the exclusive prefix
// over the buckets (moe_scan_kernel ran).  SCAN = true (few slices, at most kFoldBuckets buckets):
// counts holds the raw histograms and every wave derives its own starting positions from them -
// the per-bucket sum over the earlier slices and the exclusive scan of the bucket totals - which
// saves the scan kernel's launch; the wave of slice 0 writes group_list.
constexpr int kFoldSlices = 128;
constexpr int kFoldBuckets = 256;

template <bool SCAN>
__global__ __launch_bounds__(kMoeWaves* kWave) void moe_scatter_kernel(
    const int32_t* __restrict__ ids, int64_t n, int num_experts, int num_slices,
    const int32_t* __restrict__ counts, const int32_t* __restrict__ base,
    int32_t* __restrict__ sorted_idx, int32_t* __restrict__ inverse_idx, int id_bits,
    int64_t* __restrict__ group_list) {
  extern __shared__ int32_t run_lds[];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int slice = blockIdx.x * kMoeWaves + wave;
  const int buckets = num_experts + 1;
  int32_t* running = run_lds + wave * buckets;
  if (slice >= num_slices) return;  // wave uniform; no workgroup barrier below
  if constexpr (SCAN) {
    constexpr int kPer = kFoldBuckets / kWave;  // bucket e = lane + 64*j
    int before[kPer], total[kPer];
#pragma unroll
    for (int j = 0; j < kPer; ++j) before[j] = total[j] = 0;
    // 32 rows of loads in flight: the histograms of a prefill batch (64 slices) arrive in two round trips
    constexpr int kRows = 32;
    for (int s0 = 0; s0 < num_slices; s0 += kRows) {
      int c[kRows][kPer];
#pragma unroll
      for (int u = 0; u < kRows; ++u)
#pragma unroll
        for (int j = 0; j < kPer; ++j) {
          const int e = lane + kWave * j;
          c[u][j] = (s0 + u < num_slices && e < buckets) ? counts[(int64_t)(s0 + u) * buckets + e] : 0;
        }
#pragma unroll
      for (int u = 0; u < kRows; ++u)
#pragma unroll
        for (int j = 0; j < kPer; ++j) {
          total[j] += c[u][j];
          if (s0 + u < slice) before[j] += c[u][j];
        }
    }
    int carry = 0;
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
      int incl = total[j];
#pragma unroll
      for (int d = 1; d < kWave; d <<= 1) {
        const int up = __shfl_up(incl, d);
        if (lane >= d) incl += up;
      }
      const int excl = carry + incl - total[j];
      carry += __shfl(incl, kWave - 1);
      const int e = lane + kWave * j;
      if (e < buckets) running[e] = excl + before[j];
      if (slice == 0 && e < num_experts) group_list[e] = (int64_t)excl + total[j];
    }
  } else {
    const int32_t* mine = counts + (int64_t)slice * buckets;
    for (int e = lane; e < buckets; e += kWave) running[e] = base[e] + mine[e];
  }
  const int64_t begin = (int64_t)slice * kSlice;
  const uint64_t lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
  int idv[kSlice / kWave];  // all loads first: one memory latency per slice instead of eight
#pragma unroll
  for (int b = 0; b < kSlice / kWave; ++b) {
    const int64_t i = begin + b * kWave + lane;
    idv[b] = i < n ? ids[i] : -1;
  }
#pragma unroll
  for (int b = 0; b < kSlice / kWave; ++b) {
    const int64_t i = begin + b * kWave + lane;
    const bool live = i < n;
    const int e = live ? moe_bucket(idv[b], num_experts) : 0;
    // lanes of this batch that hold the same bucket, one ballot per bit of the bucket number
    uint64_t same = __ballot(live);
    for (int bit = 0; bit < id_bits; ++bit) {
      const bool set = (e >> bit) & 1;
      const uint64_t m = __ballot(set);
      same &= set ? m : ~m;
    }
    // the lowest lane of every group advances the group's running position; LDS operations of a
    // wave execute in order, so the next batch sees the update
    const int leader = live ? __builtin_ctzll(same) : lane;
    int first = 0;
    if (live && lane == leader) {
      first = running[e];
      running[e] = first + __builtin_popcountll(same);
    }
    first = __shfl(first, leader);
    if (live) {
      const int pos = first + __builtin_popcountll(same & lt_mask);
      sorted_idx[pos] = (int32_t)i;
      if (inverse_idx) inverse_idx[i] = pos;
    }
  }
}

// out[j, :] = x[sorted_idx[j] / topk, :] for the rows that belong to a group (j < group_list[E-1]).
__global__ __launch_bounds__(256) void moe_gather_kernel(const f16* __restrict__ x,
                                                          const int32_t* __restrict__ sorted_idx,
                                                          const int64_t* __restrict__ group_list,
                                                          f16* __restrict__ out, int64_t n, int topk,
                                                          int num_experts, uint32_t vec_per_row) {
  const int64_t total = group_list[num_experts - 1];
  const int64_t rows = total < n ? total : n;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t j = i / vec_per_row;
  if (j >= rows) return;
  const uint32_t c = (uint32_t)(i - j * vec_per_row);
  // an index outside the routing table reads the last token instead of faulting
  const int64_t src = min(max((int64_t)sorted_idx[j], (int64_t)0), n - 1) / topk;
  st128_stream(out + (j * vec_per_row + c) * 8, ld128(x + (src * vec_per_row + c) * 8));
}

// out[t, :] = f16( sum_k weights[t, k] * y[inverse_idx[t*topk + k], :] ) over the k whose expert id is
// valid, accumulated in fp32 in the order of k.
__global__ __launch_bounds__(256) void moe_combine_kernel(
    const f16* __restrict__ y, const int32_t* __restrict__ inverse_idx,
    const float* __restrict__ weights, const int32_t* __restrict__ ids, f16* __restrict__ out,
    int64_t tokens, int topk, int num_experts, uint32_t vec_per_row) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t t = i / vec_per_row;
  if (t >= tokens) return;
  const uint32_t c = (uint32_t)(i - t * vec_per_row);
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  constexpr int kRows = 8;
  // eight routed rows at a time, loads first (independent), then the fp32 accumulation in the order of k
  for (int k0 = 0; k0 < topk; k0 += kRows) {
    f16x8 v[kRows];
    float wgt[kRows];
#pragma unroll
    for (int j = 0; j < kRows; ++j) {
      const int k = k0 + j;
      const int64_t f = t * topk + (k < topk ? k : topk - 1);
      const int id = ids[f];
      const bool ok = k < topk && id >= 0 && id < num_experts;
      wgt[j] = ok ? weights[f] : 0.f;
      // rows of ids that are not routed are never written: read row 0 instead and drop the value
      const int64_t row = ok ? min(max((int64_t)inverse_idx[f], (int64_t)0), tokens * topk - 1) : 0;
      v[j] = ld128_stream(y + (row * vec_per_row + c) * 8);
      if (!ok) v[j] = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
    }
#pragma unroll
    for (int j = 0; j < kRows; ++j)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = __builtin_fmaf(wgt[j], (float)v[j][e], acc[e]);
  }
  f16x8 o;
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = (f16)acc[e];
  st128_stream(out + (t * vec_per_row + c) * 8, o);
}

// Routing tables of a decode step (at most kSmallSort ids): one workgroup, one launch.  Histogram
// with LDS atomics, exclusive scan of the buckets by all four waves (group_list falls out of it),
// then wave 0 walks the ids in order, 64 at a time, exactly as moe_scatter_kernel walks a slice.
constexpr int kSmallSort = 1024;
constexpr int kSmallThreads = 4 * kWave;
constexpr int kSmallPerThread = (kMoeMaxExperts + 1) / kSmallThreads;  // consecutive buckets per thread in the scan

__global__ __launch_bounds__(kSmallThreads) void moe_sort_small_kernel(
    const int32_t* __restrict__ ids, int n, int num_experts, int32_t* __restrict__ sorted_idx,
    int32_t* __restrict__ inverse_idx, int id_bits, int64_t* __restrict__ group_list) {
  __shared__ int32_t bucket[kSmallSort];
  __shared__ int32_t running[kMoeMaxExperts + 1];
  __shared__ int32_t wave_total[4];
  const int t = threadIdx.x;
  const int lane = t & (kWave - 1);
  const int wave = t / kWave;
  const int buckets = num_experts + 1;
  for (int e = t; e < kMoeMaxExperts + 1; e += kSmallThreads) running[e] = 0;
  int mine[kSmallSort / kSmallThreads];
#pragma unroll
  for (int u = 0; u < kSmallSort / kSmallThreads; ++u) {
    const int i = t + u * kSmallThreads;
    mine[u] = i < n ? moe_bucket(ids[i], num_experts) : buckets;
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < kSmallSort / kSmallThreads; ++u) {
    const int i = t + u * kSmallThreads;
    bucket[i] = mine[u];
    if (i < n) atomicAdd(&running[mine[u]], 1);
  }
  __syncthreads();
  // exclusive scan: thread t owns buckets [t*kSmallPerThread, (t+1)*kSmallPerThread)
  int cnt[kSmallPerThread];
  int sum = 0;
#pragma unroll
  for (int u = 0; u < kSmallPerThread; ++u) {
    cnt[u] = running[t * kSmallPerThread + u];
    sum += cnt[u];
  }
  int incl = sum;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int up = __shfl_up(incl, d);
    if (lane >= d) incl += up;
  }
  if (lane == kWave - 1) wave_total[wave] = incl;
  __syncthreads();
  int excl = incl - sum;
  for (int v = 0; v < wave; ++v) excl += wave_total[v];
#pragma unroll
  for (int u = 0; u < kSmallPerThread; ++u) {
    const int e = t * kSmallPerThread + u;
    running[e] = excl;
    excl += cnt[u];
    if (e < num_experts) group_list[e] = excl;
  }
  __syncthreads();
  if (wave != 0) return;
  const uint64_t lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
  for (int i0 = 0; i0 < n; i0 += kWave) {
    const int i = i0 + lane;
    const bool live = i < n;
    const int e = live ? bucket[i] : 0;
    uint64_t same = __ballot(live);
    for (int bit = 0; bit < id_bits; ++bit) {
      const bool set = (e >> bit) & 1;
      const uint64_t m = __ballot(set);
      same &= set ? m : ~m;
    }
    const int leader = live ? __builtin_ctzll(same) : lane;
    int first = 0;
    if (live && lane == leader) {
      first = running[e];
      running[e] = first + __builtin_popcountll(same);
    }
    first = __shfl(first, leader);
    if (live) {
      const int pos = first + __builtin_popcountll(same & lt_mask);
      sorted_idx[pos] = i;
      if (inverse_idx) inverse_idx[i] = pos;
    }
  }
}

static int64_t moe_slices(int64_t n) { return (n + kSlice - 1) / kSlice; }

}  // namespace aops

extern "C" size_t aops_moe_sort_workspace(int64_t n, int64_t num_experts) {
  using namespace aops;
  if (n < 0 || num_experts <= 0 || num_experts > kMoeMaxExperts || n > 0x7fffffff) return 0;
  return (size_t)((moe_slices(n) + 1) * (num_experts + 1)) * sizeof(int32_t) + 16;
}

extern "C" int aops_moe_sort_i32(const int32_t* expert_ids, int64_t n, int64_t num_experts,
                                 int32_t* sorted_idx, int32_t* inverse_idx, int64_t* group_list,
                                 void* workspace, size_t workspace_bytes, void* stream) {
  using namespace aops;
  if (n < 0 || num_experts <= 0 || num_experts > kMoeMaxExperts || n > 0x7fffffff)
    return AOPS_ERR_INVALID_ARGUMENT;
  if (!group_list) return AOPS_ERR_INVALID_ARGUMENT;
  if (n > 0 && (!expert_ids || !sorted_idx)) return AOPS_ERR_INVALID_ARGUMENT;
  const size_t need = aops_moe_sort_workspace(n, num_experts);
  if (!workspace || workspace_bytes < need) return AOPS_ERR_WORKSPACE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  int id_bits = 1;  // bits needed for bucket numbers 0..num_experts
  while ((1 << id_bits) <= (int)num_experts) ++id_bits;
  // one launch instead of two up to 512 ids, instead of three (more than 256 buckets) up to 1024
  if (n > 0 && (n <= kSmallSort / 2 || (n <= kSmallSort && num_experts + 1 > kFoldBuckets))) {
    moe_sort_small_kernel<<<1, kSmallThreads, 0, s>>>(expert_ids, (int)n, (int)num_experts, sorted_idx,
                                                     inverse_idx, id_bits, group_list);
    return record_launch_status(hipGetLastError());
  }
  const int slices = (int)moe_slices(n);
  const int buckets = (int)num_experts + 1;
  int32_t* counts = static_cast<int32_t*>(workspace);           // [slices][E+1]
  int32_t* base = counts + (int64_t)slices * buckets;           // [E+1]
  const size_t lds = (size_t)kMoeWaves * buckets * sizeof(int32_t);
  const unsigned grid = (unsigned)((slices + kMoeWaves - 1) / kMoeWaves);
  if (slices > 0) {
    moe_hist_kernel<<<grid, kMoeWaves * kWave, lds, s>>>(expert_ids, n, (int)num_experts, slices, counts);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return record_launch_status(e);
  }
  if (slices > 0 && slices <= kFoldSlices && buckets <= kFoldBuckets) {  // two launches
    moe_scatter_kernel<true><<<grid, kMoeWaves * kWave, lds, s>>>(expert_ids, n, (int)num_experts, slices,
                                                                 counts, base, sorted_idx, inverse_idx,
                                                                 id_bits, group_list);
    return record_launch_status(hipGetLastError());
  }
  moe_scan_kernel<<<1, 1024, 0, s>>>(counts, slices, (int)num_experts, base, group_list);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return record_launch_status(e);
  if (slices > 0) {
    moe_scatter_kernel<false><<<grid, kMoeWaves * kWave, lds, s>>>(expert_ids, n, (int)num_experts, slices,
                                                                  counts, base, sorted_idx, inverse_idx,
                                                                  id_bits, group_list);
    e = hipGetLastError();
  }
  return record_launch_status(e);
}

extern "C" int aops_moe_gather_f16(const void* x, const int32_t* sorted_idx, const int64_t* group_list,
                                   void* out, int64_t n, int64_t topk, int64_t hidden,
                                   int64_t num_experts, void* stream) {
  using namespace aops;
  if (n < 0 || topk <= 0 || topk > 0x7fffffff || hidden <= 0 || hidden % 8 != 0 || num_experts <= 0 ||
      n > 0x7fffffff || hidden > 0x7fffffff)
    return AOPS_ERR_INVALID_ARGUMENT;
  if (n == 0) return AOPS_OK;
  if (!x || !sorted_idx || !group_list || !out) return AOPS_ERR_INVALID_ARGUMENT;
  const int64_t total = n * (hidden / 8);
  if (total / 256 + 1 > 0x7fffffff) return AOPS_ERR_INVALID_ARGUMENT;
  moe_gather_kernel<<<(unsigned)((total + 255) / 256), 256, 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<const f16*>(x), sorted_idx, group_list, static_cast<f16*>(out), n, (int)topk,
      (int)num_experts, (uint32_t)(hidden / 8));
  return record_launch_status(hipGetLastError());
}

extern "C" int aops_moe_combine_f16(const void* y, const int32_t* inverse_idx, const float* weights,
                                    const int32_t* expert_ids, void* out, int64_t tokens, int64_t topk,
                                    int64_t hidden, int64_t num_experts, void* stream) {
  using namespace aops;
  if (tokens < 0 || topk <= 0 || topk > 0x7fffffff || hidden <= 0 || hidden % 8 != 0 ||
      num_experts <= 0 || hidden > 0x7fffffff || tokens * topk > 0x7fffffff)
    return AOPS_ERR_INVALID_ARGUMENT;
  if (tokens == 0) return AOPS_OK;
  if (!y || !inverse_idx || !weights || !expert_ids || !out) return AOPS_ERR_INVALID_ARGUMENT;
  const int64_t total = tokens * (hidden / 8);
  if (total / 256 + 1 > 0x7fffffff) return AOPS_ERR_INVALID_ARGUMENT;
  moe_combine_kernel<<<(unsigned)((total + 255) / 256), 256, 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<const f16*>(y), inverse_idx, weights, expert_ids, static_cast<f16*>(out), tokens,
      (int)topk, (int)num_experts, (uint32_t)(hidden / 8));
  return record_launch_status(hipGetLastError());
}
