// Stable counting sort of item indices by integer key (sender-sorted edge view, nodes grouped by
// element).  Two routes to the same unique stable order, reproducible bit for bit:
//  - many keys, small buckets (edges by sender): buckets are filled with integer atomics in arbitrary order and then
//    every item is moved to its rank within the bucket, the rank being the number of bucket members with a smaller
//    item index (a scan of the bucket: quadratic in the bucket size, which is tens of items here);
//  - few keys, large buckets (atoms by element): per-workgroup histograms, one scan over (key, workgroup), and a rank
//    inside the workgroup's 256 items, so the cost per item does not grow with the bucket.
#include <algorithm>
#include <mutex>

#include "common.hpp"

namespace cm {
namespace {

constexpr int kScanThreads = 1024;
constexpr int kScanStage = 32 * 1024;  // values staged in LDS at a time (128 KB)

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
// nkeys (skipped when NULL).  Every thread owns a contiguous run of keys.
__global__ __launch_bounds__(kScanThreads) void scan_kernel(const int32_t *__restrict__ counts, int nkeys,
                                                            int32_t *__restrict__ offsets,
                                                            int32_t *__restrict__ cursor) {
  __shared__ int part[kScanThreads];
  __shared__ int stage[kScanStage];
  const int total = workgroup_exclusive_scan<kScanThreads, kScanStage, int>(
      nkeys, stage, part, [&](int k) { return counts[k]; },
      [&](int k, int before, int) {
        offsets[k] = before;
        if (cursor) cursor[k] = before;
      });
  if (threadIdx.x == 0) offsets[nkeys] = total;
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

// ---- few keys, large buckets ----------------------------------------------------------------------------------
constexpr int kFewKeys = 64;       // route bound: keys per LDS histogram
constexpr int kFewBlock = 256;     // items per workgroup
constexpr int64_t kFewMinItems = 4096;

inline bool few_keys_route(int64_t n, int64_t nkeys) { return nkeys >= 1 && nkeys <= kFewKeys && n >= kFewMinItems; }

// block_counts[k * nblocks + b] = items of workgroup b with key k
__global__ __launch_bounds__(kFewBlock) void block_histogram_kernel(const int32_t *__restrict__ keys, int64_t n, int nkeys,
                                                                     int nblocks, int32_t *__restrict__ block_counts) {
  __shared__ int hist[kFewKeys];
  const int t = threadIdx.x;
  if (t < kFewKeys) hist[t] = 0;
  __syncthreads();
  const int64_t i = blockIdx.x * static_cast<int64_t>(kFewBlock) + t;
  if (i < n) {
    const int k = keys[i];
    if (static_cast<unsigned>(k) < static_cast<unsigned>(nkeys)) atomicAdd(&hist[k], 1);
  }
  __syncthreads();
  if (t < nkeys) block_counts[static_cast<int64_t>(t) * nblocks + blockIdx.x] = hist[t];
}

// base = exclusive scan of block_counts in (key, workgroup) order: item i of workgroup b with key k goes to
// base[k * nblocks + b] + (number of earlier items of b with key k).
__global__ __launch_bounds__(kFewBlock) void block_place_kernel(const int32_t *__restrict__ keys, int64_t n, int nkeys,
                                                                 int nblocks, const int32_t *__restrict__ base,
                                                                 int32_t *__restrict__ perm, int32_t *__restrict__ offsets) {
  __shared__ int skey[kFewBlock];
  const int t = threadIdx.x;
  const int64_t i = blockIdx.x * static_cast<int64_t>(kFewBlock) + t;
  int k = -1;
  if (i < n) {
    k = keys[i];
    if (static_cast<unsigned>(k) >= static_cast<unsigned>(nkeys)) k = -1;
  }
  skey[t] = k;
  __syncthreads();
  if (k >= 0) {
    int rank = 0;
    for (int j = 0; j < t; ++j) rank += skey[j] == k ? 1 : 0;
    perm[base[static_cast<int64_t>(k) * nblocks + blockIdx.x] + rank] = static_cast<int32_t>(i);
  }
  if (blockIdx.x == 0 && t <= nkeys) offsets[t] = base[static_cast<int64_t>(t) * nblocks];
}

}  // namespace
}  // namespace cm

extern "C" size_t cm_stable_key_sort_workspace(int64_t n, int64_t nkeys) {
  if (n < 0 || nkeys < 0) return 0;
  // counts[nkeys] + cursor[nkeys] + bucketed[n], each int32; the few-keys route instead keeps two tables over
  // (key, workgroup) plus the closing total; rounded up to 256 bytes
  size_t ints = static_cast<size_t>(2 * nkeys + n);
  if (cm::few_keys_route(n, nkeys)) {
    const size_t table = static_cast<size_t>(nkeys) * static_cast<size_t>(cm::ceil_div(n, cm::kFewBlock));
    ints = std::max(ints, 2 * table + 2);
  }
  const size_t bytes = ints * sizeof(int32_t);
  return (bytes + 255) & ~static_cast<size_t>(255);
}

namespace cm {
namespace {

// Enqueues the five kernels of the sort; `workspace` holds cm_stable_key_sort_workspace(n, nkeys) bytes.
int sort_enqueue(const int32_t *keys, int64_t n, int64_t nkeys, int32_t *perm, int32_t *offsets, void *workspace,
                 hipStream_t st, const char *what) {
  if (few_keys_route(n, nkeys)) {
    const int nblocks = static_cast<int>(ceil_div(n, kFewBlock));
    const int entries = static_cast<int>(nkeys) * nblocks;
    int32_t *block_counts = static_cast<int32_t *>(workspace);
    int32_t *base = block_counts + entries;  // entries + 1 values
    hipLaunchKernelGGL(block_histogram_kernel, dim3(nblocks), dim3(kFewBlock), 0, st, keys, n, static_cast<int>(nkeys), nblocks,
                       block_counts);
    hipLaunchKernelGGL(scan_kernel, dim3(1), dim3(kScanThreads), 0, st, block_counts, entries, base,
                       static_cast<int32_t *>(nullptr));
    hipLaunchKernelGGL(block_place_kernel, dim3(nblocks), dim3(kFewBlock), 0, st, keys, n, static_cast<int>(nkeys), nblocks, base,
                       perm, offsets);
    return check_launch(what);
  }
  int32_t *counts = static_cast<int32_t *>(workspace);
  int32_t *cursor = counts + nkeys;
  int32_t *bucketed = cursor + nkeys;
  const int block = 256;
  if (nkeys > 0) {
    const unsigned g = static_cast<unsigned>(std::min<int64_t>(ceil_div(nkeys, block), 4096));
    hipLaunchKernelGGL(fill_i32_kernel, dim3(g), dim3(block), 0, st, counts, nkeys, 0);
  }
  const unsigned gn = static_cast<unsigned>(ceil_div(n > 0 ? n : 1, block));
  if (n > 0)
    hipLaunchKernelGGL(histogram_kernel, dim3(gn), dim3(block), 0, st, keys, n, static_cast<int>(nkeys), counts);
  hipLaunchKernelGGL(scan_kernel, dim3(1), dim3(kScanThreads), 0, st, counts, static_cast<int>(nkeys), offsets, cursor);
  if (n > 0) {
    hipLaunchKernelGGL(bucket_fill_kernel, dim3(gn), dim3(block), 0, st, keys, n, static_cast<int>(nkeys), cursor, bucketed);
    hipLaunchKernelGGL(bucket_rank_kernel, dim3(gn), dim3(block), 0, st, keys, bucketed, offsets,
                       static_cast<int>(nkeys), perm);
  }
  return check_launch(what);
}

}  // namespace
}  // namespace cm

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
  return cm::sort_enqueue(keys, n, nkeys, perm, offsets, workspace, cm::as_stream(stream), "cm_stable_key_sort");
}

// ---- the same sort without a caller's workspace ---------------------------------------------------------------
// The counters, cursors and the bucketed item list live in a device array that is part of the library's code object:
// every GPU the library runs on holds its own copy at its own address for the life of the process.
#define CM_SORT_STATIC_BYTES (32u << 20)
static __device__ __align__(256) unsigned char scratch[CM_SORT_STATIC_BYTES];

namespace cm {
namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices] = {};  // device address of `scratch` on each GPU, looked up once per GPU

// Device address of this GPU's copy of `scratch` (nullptr after storing an error message).  In host code the
// array's name is only a handle for the runtime; kernels and copies must be given the address returned here.
void *static_scratch_of_current_device() {
  int dev = -1;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    set_error("cm_stable_key_sort_static: no usable current device (%s)", hipGetErrorString(err));
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void *ptr = nullptr;
    err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (err != hipSuccess || ptr == nullptr) {
      set_error("cm_stable_key_sort_static: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(err));
      return nullptr;
    }
    g_scratch_ptr[dev] = ptr;
  }
  return g_scratch_ptr[dev];
}

}  // namespace
}  // namespace cm

// Also the set-up call: looks the buffer's address up for the current device (when there is one), so that a later
// cm_stable_key_sort_static on this device makes no runtime query and can be recorded into a stream capture.
extern "C" size_t cm_stable_key_sort_static_capacity(void) {
  int count = 0;
  if (hipGetDeviceCount(&count) == hipSuccess && count > 0) (void)cm::static_scratch_of_current_device();
  return CM_SORT_STATIC_BYTES;
}

extern "C" int cm_stable_key_sort_static(const int32_t *keys, int64_t n, int64_t nkeys, int32_t *perm,
                                         int32_t *offsets, cm_stream_t stream) {
  CM_REQUIRE(n >= 0 && nkeys >= 0, "cm_stable_key_sort_static: negative size");
  CM_REQUIRE(n < INT32_MAX && nkeys < INT32_MAX, "cm_stable_key_sort_static: sizes exceed int32 indexing");
  CM_REQUIRE(offsets != nullptr, "cm_stable_key_sort_static: offsets is NULL");
  CM_REQUIRE(n == 0 || (keys && perm), "cm_stable_key_sort_static: NULL pointer");
  const size_t need = cm_stable_key_sort_workspace(n, nkeys);
  if (need > CM_SORT_STATIC_BYTES) {
    cm::set_error("cm_stable_key_sort_static: n = %lld items with nkeys = %lld need %zu bytes of scratch, the built-in "
                  "buffer holds %zu (4 * (n + 2 * nkeys) must not exceed it); use cm_stable_key_sort with a workspace",
                  static_cast<long long>(n), static_cast<long long>(nkeys), need,
                  static_cast<size_t>(CM_SORT_STATIC_BYTES));
    return CM_ENOSPC;
  }
  void *ws = cm::static_scratch_of_current_device();
  if (ws == nullptr) return CM_ELAUNCH;
  return cm::sort_enqueue(keys, n, nkeys, perm, offsets, ws, cm::as_stream(stream), "cm_stable_key_sort_static");
}
