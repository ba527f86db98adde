// Stable counting sort of item indices by integer key (sender-sorted edge view, nodes grouped by
// element).  Buckets are filled with integer atomics in arbitrary order and then every item is
// moved to its rank within the bucket, the rank being the number of bucket members with a smaller
// item index.  The result is the unique stable order, so it is reproducible bit for bit although
// atomics are used on the way.
#include <algorithm>

#include "common.hpp"

namespace cm {
namespace {

constexpr int kScanThreads = 1024;

__global__ void fill_i32_kernel(int32_t *p, int64_t n, int32_t value) {
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x)
    p[i] = value;
}

__global__ void histogram_kernel(const int32_t *__restrict__ keys, int64_t n, int nkeys,
                                 int32_t *__restrict__ counts) {
  const int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  if (i >= n) return;
  const int k = keys[i];
  if (static_cast<unsigned>(k) < static_cast<unsigned>(nkeys)) atomicAdd(&counts[k], 1);
}

// One workgroup: offsets = exclusive scan of counts (nkeys + 1 entries), cursor = copy of the first
// nkeys.  Every thread owns a contiguous run of keys.
__global__ __launch_bounds__(kScanThreads) void scan_kernel(const int32_t *__restrict__ counts, int nkeys,
                                                            int32_t *__restrict__ offsets,
                                                            int32_t *__restrict__ cursor) {
  __shared__ int part[kScanThreads];
  const int t = threadIdx.x;
  const int per = (nkeys + kScanThreads - 1) / kScanThreads;
  const int lo = min(t * per, nkeys);
  const int hi = min(lo + per, nkeys);
  int sum = 0;
  for (int k = lo; k < hi; ++k) sum += counts[k];
  part[t] = sum;
  __syncthreads();
  for (int d = 1; d < kScanThreads; d <<= 1) {
    const int v = t >= d ? part[t - d] : 0;
    __syncthreads();
    part[t] += v;
    __syncthreads();
  }
  int run = part[t] - sum;  // exclusive prefix of this thread's run
  for (int k = lo; k < hi; ++k) {
    offsets[k] = run;
    cursor[k] = run;
    run += counts[k];
  }
  if (t == kScanThreads - 1) offsets[nkeys] = part[t];
}

__global__ void bucket_fill_kernel(const int32_t *__restrict__ keys, int64_t n, int nkeys,
                                   int32_t *__restrict__ cursor, int32_t *__restrict__ bucketed) {
  const int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  if (i >= n) return;
  const int k = keys[i];
  if (static_cast<unsigned>(k) < static_cast<unsigned>(nkeys)) {
    const int pos = atomicAdd(&cursor[k], 1);
    bucketed[pos] = static_cast<int32_t>(i);
  }
}

__global__ void bucket_rank_kernel(const int32_t *__restrict__ keys, const int32_t *__restrict__ bucketed,
                                   const int32_t *__restrict__ offsets, int nkeys, int32_t *__restrict__ perm) {
  const int64_t p = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  if (p >= offsets[nkeys]) return;
  const int item = bucketed[p];
  const int k = keys[item];
  const int lo = offsets[k];
  const int hi = offsets[k + 1];
  int rank = 0;
  for (int q = lo; q < hi; ++q) rank += bucketed[q] < item ? 1 : 0;
  perm[lo + rank] = item;
}

}  // namespace
}  // namespace cm

extern "C" size_t cm_stable_key_sort_workspace(int64_t n, int64_t nkeys) {
  if (n < 0 || nkeys < 0) return 0;
  // counts[nkeys] + cursor[nkeys] + bucketed[n], each int32, rounded up to 256 bytes
  const size_t bytes = static_cast<size_t>(2 * nkeys + n) * sizeof(int32_t);
  return (bytes + 255) & ~static_cast<size_t>(255);
}

extern "C" int cm_stable_key_sort(const int32_t *keys, int64_t n, int64_t nkeys, int32_t *perm,
                                  int32_t *offsets, void *workspace, size_t workspace_bytes,
                                  cm_stream_t stream) {
  CM_REQUIRE(n >= 0 && nkeys >= 0, "cm_stable_key_sort: negative size");
  CM_REQUIRE(n < INT32_MAX && nkeys < INT32_MAX, "cm_stable_key_sort: sizes exceed int32 indexing");
  CM_REQUIRE(offsets != nullptr, "cm_stable_key_sort: offsets is NULL");
  CM_REQUIRE(n == 0 || (keys && perm), "cm_stable_key_sort: NULL pointer");
  if (workspace_bytes < cm_stable_key_sort_workspace(n, nkeys) || (workspace == nullptr && (n > 0 || nkeys > 0))) {
    cm::set_error("cm_stable_key_sort: workspace of %zu bytes, need %zu", workspace_bytes,
                  cm_stable_key_sort_workspace(n, nkeys));
    return CM_ENOSPC;
  }
  hipStream_t st = cm::as_stream(stream);
  int32_t *counts = static_cast<int32_t *>(workspace);
  int32_t *cursor = counts + nkeys;
  int32_t *bucketed = cursor + nkeys;
  const int block = 256;
  if (nkeys > 0) {
    const unsigned g = static_cast<unsigned>(std::min<int64_t>(cm::ceil_div(nkeys, block), 4096));
    hipLaunchKernelGGL(cm::fill_i32_kernel, dim3(g), dim3(block), 0, st, counts, nkeys, 0);
  }
  const unsigned gn = static_cast<unsigned>(cm::ceil_div(n > 0 ? n : 1, block));
  if (n > 0)
    hipLaunchKernelGGL(cm::histogram_kernel, dim3(gn), dim3(block), 0, st, keys, n, static_cast<int>(nkeys), counts);
  hipLaunchKernelGGL(cm::scan_kernel, dim3(1), dim3(cm::kScanThreads), 0, st, counts, static_cast<int>(nkeys), offsets, cursor);
  if (n > 0) {
    hipLaunchKernelGGL(cm::bucket_fill_kernel, dim3(gn), dim3(block), 0, st, keys, n, static_cast<int>(nkeys), cursor, bucketed);
    hipLaunchKernelGGL(cm::bucket_rank_kernel, dim3(gn), dim3(block), 0, st, keys, bucketed, offsets,
                       static_cast<int>(nkeys), perm);
  }
  return cm::check_launch("cm_stable_key_sort");
}
