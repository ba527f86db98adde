// Stable counting sort of item indices by integer key (sender-sorted edge view, nodes grouped by
// element).  Buckets are filled with integer atomics in arbitrary order and then every item is
// moved to its rank within the bucket, the rank being the number of bucket members with a smaller
// item index.  The result is the unique stable order, so it is reproducible bit for bit although
// atomics are used on the way.
#include <algorithm>
#include <mutex>

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

namespace cm {
namespace {

// Enqueues the five kernels of the sort; `workspace` holds cm_stable_key_sort_workspace(n, nkeys) bytes.
int sort_enqueue(const int32_t *keys, int64_t n, int64_t nkeys, int32_t *perm, int32_t *offsets, void *workspace,
                 hipStream_t st, const char *what) {
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

extern "C" size_t cm_stable_key_sort_static_capacity(void) { return CM_SORT_STATIC_BYTES; }

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
