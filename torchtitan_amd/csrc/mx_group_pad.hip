// Token-group padding for MoE grouped GEMMs: sizes, offsets and the permutation that moves
// routed tokens into expert-grouped, alignment-padded order.  Integer work, one launch.
//
// Every workgroup redoes the two small prefix sums in LDS (n = ranks * experts <= 4096
// counters) and then fills its own slice of the output; no workspace, no host round trip.
#include "mx_common.h"

namespace mx {

constexpr int kPadMaxCounters = 4096;
constexpr int kPadThreads = 256;

// Exclusive prefix sum of v[0..n) in place, n <= kPadMaxCounters, all 256 threads call it.
__device__ inline void block_exclusive_scan(int32_t* v, int n, int32_t* partial /*[256]*/) {
  const int tid = threadIdx.x;
  const int per = (n + kPadThreads - 1) / kPadThreads;
  const int lo = min(tid * per, n), hi = min(lo + per, n);
  int32_t sum = 0;
  for (int i = lo; i < hi; ++i) sum += v[i];
  partial[tid] = sum;
  __syncthreads();
  for (int off = 1; off < kPadThreads; off <<= 1) {
    const int32_t add = tid >= off ? partial[tid - off] : 0;
    __syncthreads();
    partial[tid] += add;
    __syncthreads();
  }
  int32_t run = partial[tid] - sum;  // exclusive prefix of this thread's chunk
  for (int i = lo; i < hi; ++i) {
    const int32_t c = v[i];
    v[i] = run;
    run += c;
  }
  __syncthreads();
}

__global__ __launch_bounds__(kPadThreads) void group_offsets_pad_kernel(
    const int32_t* __restrict__ counts, int experts, int ranks, int64_t max_len, int alignment,
    int64_t* __restrict__ perm, int32_t* __restrict__ m_sizes, int32_t* __restrict__ m_offsets) {
  __shared__ int32_t cnt[kPadMaxCounters];    // counts[r * experts + e]
  __shared__ int32_t start[kPadMaxCounters];  // exclusive prefix of counts in that order
  __shared__ int32_t woff[kPadMaxCounters];   // per expert: write offset (exclusive prefix of m_sizes)
  __shared__ int32_t msz[kPadMaxCounters];
  __shared__ int32_t partial[kPadThreads];
  const int tid = threadIdx.x;
  const int n = experts * ranks;
  for (int i = tid; i < n; i += kPadThreads) {
    const int32_t c = counts[i];
    cnt[i] = c;
    start[i] = c;
  }
  __syncthreads();
  block_exclusive_scan(start, n, partial);
  for (int e = tid; e < experts; e += kPadThreads) {
    int32_t tot = 0;
    for (int r = 0; r < ranks; ++r) tot += cnt[r * experts + e];
    tot = tot < alignment ? alignment : tot;
    const int32_t sz = (tot + alignment - 1) / alignment * alignment;
    msz[e] = sz;
    woff[e] = sz;
  }
  __syncthreads();
  block_exclusive_scan(woff, experts, partial);
  if (blockIdx.x == 0)
    for (int e = tid; e < experts; e += kPadThreads) {
      m_sizes[e] = msz[e];
      m_offsets[e] = woff[e] + msz[e];
    }

  // this workgroup's slice of the permutation
  const int64_t per_block = (max_len + gridDim.x - 1) / gridDim.x;
  const int64_t p_lo = (int64_t)blockIdx.x * per_block;
  const int64_t p_hi = p_lo + per_block < max_len ? p_lo + per_block : max_len;
  for (int64_t p = p_lo + tid; p < p_hi; p += kPadThreads) {
    // last expert whose write offset is <= p
    int lo = 0, hi = experts - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if ((int64_t)woff[mid] <= p) lo = mid; else hi = mid - 1;
    }
    const int e = lo;
    int64_t j = p - woff[e];
    int64_t value = -1;
    if (j < msz[e] || e == experts - 1) {
      for (int r = 0; r < ranks; ++r) {
        const int32_t c = cnt[r * experts + e];
        if (j < c) {
          value = (int64_t)start[r * experts + e] + j;
          break;
        }
        j -= c;
      }
    }
    perm[p] = value;
  }
}

// Routing plan of an MoE layer in one launch: from the tokens-per-expert counts and the
// expert-sorted order of the (token, choice) pairs, the aligned group layout and every map the
// fused layer needs: for each padded row its token (or -1) and routing score, for each pair its
// padded row, and the padded inclusive group ends.
__global__ __launch_bounds__(kPadThreads) void moe_route_plan_kernel(
    const int32_t* __restrict__ counts, int experts, const int64_t* __restrict__ order,
    const float* __restrict__ scores, int64_t pairs, int top_k, int64_t max_len, int alignment,
    int32_t* __restrict__ m_offsets, int64_t* __restrict__ src_row, float* __restrict__ row_score,
    int64_t* __restrict__ pos) {
  __shared__ int32_t cnt[kPadMaxCounters];
  __shared__ int32_t start[kPadMaxCounters];  // exclusive prefix of counts
  __shared__ int32_t woff[kPadMaxCounters];   // exclusive prefix of the padded sizes
  __shared__ int32_t partial[kPadThreads];
  const int tid = threadIdx.x;
  for (int i = tid; i < experts; i += kPadThreads) {
    const int32_t c = counts[i];
    cnt[i] = c;
    start[i] = c;
    const int32_t tot = c < alignment ? alignment : c;
    woff[i] = (tot + alignment - 1) / alignment * alignment;
  }
  __syncthreads();
  block_exclusive_scan(start, experts, partial);
  if (blockIdx.x == 0)
    for (int e = tid; e < experts; e += kPadThreads) m_offsets[e] = woff[e];  // sizes, for now
  __syncthreads();
  block_exclusive_scan(woff, experts, partial);
  if (blockIdx.x == 0)
    for (int e = tid; e < experts; e += kPadThreads) m_offsets[e] += woff[e];  // inclusive ends
  const int64_t per_block = (max_len + gridDim.x - 1) / gridDim.x;
  const int64_t p_lo = (int64_t)blockIdx.x * per_block;
  const int64_t p_hi = p_lo + per_block < max_len ? p_lo + per_block : max_len;
  for (int64_t p = p_lo + tid; p < p_hi; p += kPadThreads) {
    int lo = 0, hi = experts - 1;  // last expert whose write offset is <= p
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if ((int64_t)woff[mid] <= p) lo = mid; else hi = mid - 1;
    }
    const int64_t j = p - woff[lo];
    int64_t token = -1;
    float score = 0.f;
    if (j < cnt[lo]) {
      const int64_t i = (int64_t)start[lo] + j;  // position in the expert-sorted order
      if (i < pairs) {
        const int64_t pair = order[i];
        if (pair >= 0 && pair < pairs) {
          token = pair / top_k;
          if (scores) score = scores[pair];
          pos[pair] = p;
        }
      }
    }
    src_row[p] = token;
    row_score[p] = score;
  }
}

}  // namespace mx

using namespace mx;

extern "C" int mx_moe_route_plan(const int32_t* counts, int64_t experts, const int64_t* order,
                                 const float* scores, int64_t pairs, int64_t top_k, int64_t max_len,
                                 int64_t alignment, int32_t* m_offsets, int64_t* src_row,
                                 float* row_score, int64_t* pos, void* stream) {
  if (experts <= 0 || pairs < 0 || top_k <= 0 || max_len < 0 || alignment <= 0) return MX_ERR_INVALID_ARG;
  if (!counts || !m_offsets || (pairs > 0 && (!order || !pos)) || (max_len > 0 && (!src_row || !row_score)))
    return MX_ERR_INVALID_ARG;
  if (experts > kPadMaxCounters || alignment > (1 << 20) || top_k > (1 << 20)) return MX_ERR_UNSUPPORTED;
  int64_t blocks = (max_len + 4095) / 4096;
  blocks = blocks < 1 ? 1 : (blocks > 1024 ? 1024 : blocks);
  hipLaunchKernelGGL(moe_route_plan_kernel, dim3((unsigned)blocks), dim3(kPadThreads), 0,
                     (hipStream_t)stream, counts, (int)experts, order, scores, pairs, (int)top_k,
                     max_len, (int)alignment, m_offsets, src_row, row_score, pos);
  return hipGetLastError() == hipSuccess ? MX_OK : MX_ERR_LAUNCH;
}

extern "C" int mx_group_offsets_pad(const int32_t* counts, int64_t experts_per_rank,
                                    int64_t num_ranks, int64_t max_len, int64_t alignment,
                                    int64_t* perm, int32_t* m_sizes, int32_t* m_offsets,
                                    void* stream) {
  if (experts_per_rank <= 0 || num_ranks <= 0 || max_len < 0 || alignment <= 0)
    return MX_ERR_INVALID_ARG;
  if (!counts || !m_sizes || !m_offsets || (max_len > 0 && !perm)) return MX_ERR_INVALID_ARG;
  if (experts_per_rank * num_ranks > kPadMaxCounters || alignment > (1 << 20))
    return MX_ERR_UNSUPPORTED;
  int64_t blocks = (max_len + 4095) / 4096;
  blocks = blocks < 1 ? 1 : (blocks > 1024 ? 1024 : blocks);
  hipLaunchKernelGGL(group_offsets_pad_kernel, dim3((unsigned)blocks), dim3(kPadThreads), 0,
                     (hipStream_t)stream, counts, (int)experts_per_rank, (int)num_ranks, max_len,
                     (int)alignment, perm, m_sizes, m_offsets);
  return hipGetLastError() == hipSuccess ? MX_OK : MX_ERR_LAUNCH;
}
