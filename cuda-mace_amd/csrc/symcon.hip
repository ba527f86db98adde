// Symmetric contraction (correlation 3, scalar output) and its analytic gradient.
//
// The cubic form is evaluated over monomials x_i x_j x_k with i <= j <= k whose coefficients
// T3[e, t, c] (and T2, T1 for the quadratic and linear parts) are folded once per call from the
// sparse coupling tables and the per-element weights; that removes every permuted duplicate of the
// packed table from the inner loop.  Nodes are processed grouped by element so that a workgroup
// works with one coefficient set; a thread owns one channel, the node's 16 inputs and 16 gradient
// accumulators sit in LDS columns private to that thread (dynamic component indices, no bank
// conflicts, no synchronisation inside the monomial loop).
//
// Every kernel is a template over the scalar type: fp32 is the model's precision, fp64 is built because the reference
// dispatches the contraction on float and double (jit_wrappers/src/symmetric_contraction_wrapper.cpp:68).
#include <algorithm>

#include "common.hpp"
#include "symcon_lmax3.inc"

namespace cm {
namespace {

__device__ __forceinline__ float fmad(float a, float b, float c) { return fmaf(a, b, c); }
__device__ __forceinline__ double fmad(double a, double b, double c) { return fma(a, b, c); }

// T[e, t, c] = sum over the CSR row t of val * W[e, path, c]
template <typename S>
__global__ void fold_tables_kernel(const int32_t *__restrict__ off, const int32_t *__restrict__ path,
                                   const S *__restrict__ val, int nmono, const S *__restrict__ W, int ne, int P, int C,
                                   S *__restrict__ T) {
  const int64_t idx = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  if (idx >= static_cast<int64_t>(ne) * nmono * C) return;
  const int c = idx % C;
  const int t = (idx / C) % nmono;
  const int e = idx / (static_cast<int64_t>(C) * nmono);
  S acc = 0;
  for (int q = off[t]; q < off[t + 1]; ++q) {
    const int p = path[q];
    if (static_cast<unsigned>(p) < static_cast<unsigned>(P)) acc += val[q] * W[(static_cast<int64_t>(e) * P + p) * C + c];
  }
  T[idx] = acc;
}

template <typename S>
__global__ void copy_w1_kernel(const S *__restrict__ W1, int ne, int P1, int C, S *__restrict__ T1) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= ne * C) return;
  T1[idx] = W1[(static_cast<int64_t>(idx / C) * P1) * C + idx % C];
}

// Workgroup: blockDim.x = C threads (one per channel), NB nodes of one element at a time.
template <typename S, int NB, bool GRAD>
__global__ void symcon_forward_kernel(const S *__restrict__ X, const int32_t *__restrict__ node_perm,
                                      const int32_t *__restrict__ group_offsets, const int32_t *__restrict__ mono3,
                                      int n3, const int32_t *__restrict__ mono2, int n2, const S *__restrict__ T3,
                                      const S *__restrict__ T2, const S *__restrict__ T1, int nnodes, int ne,
                                      S *__restrict__ out, S *__restrict__ grad) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  S *smem = reinterpret_cast<S *>(smem_raw);
  const int C = blockDim.x;
  const int c = threadIdx.x;
  S *sx = smem;                 // [NB][16][C]
  S *sg = smem + NB * 16 * C;   // [NB][16][C] (GRAD only)

  int tile = blockIdx.x;
  int e = 0, pos0 = 0, gend = 0;
  bool found = false;
  for (e = 0; e < ne; ++e) {
    const int lo = group_offsets[e], hi = group_offsets[e + 1];
    const int tiles = (hi - lo + NB - 1) / NB;
    if (tile < tiles) {
      pos0 = lo + tile * NB;
      gend = hi;
      found = true;
      break;
    }
    tile -= tiles;
  }
  if (!found) return;
  const int nb = min(NB, gend - pos0);

  int node[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    node[b] = -1;
    if (b < nb) {
      const int n = node_perm[pos0 + b];
      if (static_cast<unsigned>(n) < static_cast<unsigned>(nnodes)) node[b] = n;
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      sx[(b * 16 + i) * C + c] = node[b] >= 0 ? X[(static_cast<int64_t>(node[b]) * 16 + i) * C + c] : S(0);
      if (GRAD) sg[(b * 16 + i) * C + c] = S(0);
    }
  }
  // every thread reads and writes only its own column c of sx / sg: no barrier needed

  S acc[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b) acc[b] = S(0);

  const S *t3 = T3 + static_cast<int64_t>(e) * n3 * C + c;
  for (int t = 0; t < n3; ++t) {
    const int ijk = mono3[t];
    const int i = ijk & 0xFF, j = (ijk >> 8) & 0xFF, k = (ijk >> 16) & 0xFF;
    const S w = t3[static_cast<int64_t>(t) * C];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const S xi = sx[(b * 16 + i) * C + c], xj = sx[(b * 16 + j) * C + c], xk = sx[(b * 16 + k) * C + c];
      const S wjk = w * xj * xk;
      acc[b] = fmad(wjk, xi, acc[b]);
      if (GRAD) {
        sg[(b * 16 + i) * C + c] += wjk;
        sg[(b * 16 + j) * C + c] += w * xi * xk;
        sg[(b * 16 + k) * C + c] += w * xi * xj;
      }
    }
  }
  const S *t2 = T2 + static_cast<int64_t>(e) * n2 * C + c;
  for (int t = 0; t < n2; ++t) {
    const int ij = mono2[t];
    const int i = ij & 0xFF, j = (ij >> 8) & 0xFF;
    const S w = t2[static_cast<int64_t>(t) * C];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const S xi = sx[(b * 16 + i) * C + c], xj = sx[(b * 16 + j) * C + c];
      acc[b] = fmad(w * xi, xj, acc[b]);
      if (GRAD) {
        sg[(b * 16 + i) * C + c] += w * xj;
        sg[(b * 16 + j) * C + c] += w * xi;
      }
    }
  }
  const S w1 = T1[static_cast<int64_t>(e) * C + c];
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    if (node[b] < 0) continue;
    out[static_cast<int64_t>(node[b]) * C + c] = fmad(w1, sx[(b * 16) * C + c], acc[b]);
    if (GRAD) {
#pragma unroll
      for (int i = 0; i < 16; ++i)
        grad[(static_cast<int64_t>(node[b]) * 16 + i) * C + c] = sg[(b * 16 + i) * C + c] + (i == 0 ? w1 : S(0));
    }
  }
}

// Specialised forward for the l_max = 3 structure known at build time: the monomial lists are unrolled, so a
// thread (= one channel) keeps its 77 + 16 + 1 coefficients, the node's 16 inputs and 16 gradient accumulators in
// registers and streams over `npb` nodes of one element.  No LDS; loads and stores are coalesced rows.  npb is 16 where
// that still gives every SIMD two waves (the coefficient loads are then a fifth of a wave's loads), fewer for fewer
// nodes, down to 2: at 5 000 nodes x 96 channels 16 nodes per wave leave the device at 0.6 waves per SIMD (29 us per
// launch, the time of one wave's 16 nodes).
constexpr int kMaxNodesPerBlock = 16;

template <typename S, bool GRAD>
__global__ __launch_bounds__(kWave) void symcon_lmax3_kernel(const S *__restrict__ X,
                                                            const int32_t *__restrict__ node_perm,
                                                            const int32_t *__restrict__ group_offsets,
                                                            const S *__restrict__ T3, const S *__restrict__ T2,
                                                            const S *__restrict__ T1, int nnodes, int ne, int C,
                                                            int npb, S *__restrict__ out, S *__restrict__ grad) {
  const int c = blockIdx.y * kWave + threadIdx.x;
  int tile = blockIdx.x;
  int e = 0, pos0 = 0, gend = 0;
  bool found = false;
  for (e = 0; e < ne; ++e) {
    const int lo = group_offsets[e], hi = group_offsets[e + 1];
    const int tiles = (hi - lo + npb - 1) / npb;
    if (tile < tiles) {
      pos0 = lo + tile * npb;
      gend = hi;
      found = true;
      break;
    }
    tile -= tiles;
  }
  if (!found || c >= C) return;
  const int nb = min(npb, gend - pos0);

  S t3[CM_SYMCON_N3], t2[CM_SYMCON_N2];
#pragma unroll
  for (int t = 0; t < CM_SYMCON_N3; ++t) t3[t] = T3[(static_cast<int64_t>(e) * CM_SYMCON_N3 + t) * C + c];
#pragma unroll
  for (int t = 0; t < CM_SYMCON_N2; ++t) t2[t] = T2[(static_cast<int64_t>(e) * CM_SYMCON_N2 + t) * C + c];
  const S t1 = T1[static_cast<int64_t>(e) * C + c];

  for (int b = 0; b < nb; ++b) {
    const int node = node_perm[pos0 + b];
    if (static_cast<unsigned>(node) >= static_cast<unsigned>(nnodes)) continue;
    const S *xp = X + static_cast<int64_t>(node) * 16 * C + c;
    S x[16], g[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      x[i] = xp[i * C];
      g[i] = S(0);
    }
    S acc = t1 * x[0];
    g[0] = t1;
#define CM_TERM3(t, i, j, k)                    \
  {                                             \
    const S w = t3[t];                      \
    const S wjk = w * (x[j] * x[k]);        \
    acc = fmad(wjk, x[i], acc);                 \
    if (GRAD) {                                 \
      g[i] += wjk;                              \
      g[j] = fmad(w * x[i], x[k], g[j]);        \
      g[k] = fmad(w * x[i], x[j], g[k]);        \
    }                                           \
  }
    CM_SYMCON_MONO3(CM_TERM3)
#undef CM_TERM3
#define CM_TERM2(t, i, j)                       \
  {                                             \
    const S w = t2[t];                      \
    acc = fmad(w * x[i], x[j], acc);            \
    if (GRAD) {                                 \
      g[i] = fmad(w, x[j], g[i]);               \
      g[j] = fmad(w, x[i], g[j]);               \
    }                                           \
  }
    CM_SYMCON_MONO2(CM_TERM2)
#undef CM_TERM2
    out[static_cast<int64_t>(node) * C + c] = acc;
    if (GRAD) {
      S *gp = grad + static_cast<int64_t>(node) * 16 * C + c;
#pragma unroll
      // streamed out: the gradient is read again only in the backward pass (measured 25 % faster at 128 channels)
      for (int i = 0; i < 16; ++i) __builtin_nontemporal_store(g[i], gp + i * C);
    }
  }
}

__global__ void symcon_backward_kernel(const float *__restrict__ grad, const float *__restrict__ gout, int64_t nnodes,
                                       int C, float *__restrict__ gX) {
  const int C4 = C / 4;
  const int64_t t = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  if (t >= nnodes * 16 * C4) return;
  const int c4 = t % C4;
  const int64_t n = t / (16 * C4);
  const f4 g = ld4(gout + n * C + 4 * c4);
  st4(gX + 4 * t, ld4_stream(grad + 4 * t) * g);
}

__global__ void symcon_backward_f64_kernel(const double *__restrict__ grad, const double *__restrict__ gout, int64_t total,
                                           int C, double *__restrict__ gX) {
  const int64_t t = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  if (t >= total) return;
  gX[t] = grad[t] * gout[(t / (16 * C)) * C + t % C];
}

template <typename S, int NB>
void launch_fwd(bool want_grad, unsigned grid, int C, hipStream_t st, const S *X, const int32_t *perm,
                const int32_t *offs, const int32_t *mono3, int n3, const int32_t *mono2, int n2, const S *T3,
                const S *T2, const S *T1, int nnodes, int ne, S *out, S *grad) {
  const size_t lds = static_cast<size_t>(NB) * 16 * C * sizeof(S) * (want_grad ? 2 : 1);
  if (want_grad)
    hipLaunchKernelGGL((symcon_forward_kernel<S, NB, true>), dim3(grid), dim3(C), lds, st, X, perm, offs, mono3, n3, mono2,
                       n2, T3, T2, T1, nnodes, ne, out, grad);
  else
    hipLaunchKernelGGL((symcon_forward_kernel<S, NB, false>), dim3(grid), dim3(C), lds, st, X, perm, offs, mono3, n3, mono2,
                       n2, T3, T2, T1, nnodes, ne, out, grad);
}

template <typename S>
int tables(const char *what, const int32_t *term3_off, const int32_t *term3_path, const S *term3_val, int n3,
           const int32_t *term2_off, const int32_t *term2_path, const S *term2_val, int n2, const S *W3, const S *W2,
           const S *W1, int nelements, int P3, int P2, int P1, int channels, S *T3, S *T2, S *T1, cm_stream_t stream) {
  CM_REQUIRE(n3 >= 0 && n2 >= 0 && nelements >= 1 && P3 >= 1 && P2 >= 1 && P1 >= 1 && channels >= 1, "%s: bad sizes", what);
  CM_REQUIRE(term3_off && term2_off && W3 && W2 && W1 && T1, "%s: NULL pointer", what);
  CM_REQUIRE((n3 == 0 || T3) && (n2 == 0 || T2), "%s: NULL output table", what);
  hipStream_t st = as_stream(stream);
  const int block = 256;
  if (n3 > 0) {
    const int64_t tot = static_cast<int64_t>(nelements) * n3 * channels;
    hipLaunchKernelGGL(fold_tables_kernel<S>, dim3(static_cast<unsigned>(ceil_div(tot, block))), dim3(block), 0, st,
                       term3_off, term3_path, term3_val, n3, W3, nelements, P3, channels, T3);
  }
  if (n2 > 0) {
    const int64_t tot = static_cast<int64_t>(nelements) * n2 * channels;
    hipLaunchKernelGGL(fold_tables_kernel<S>, dim3(static_cast<unsigned>(ceil_div(tot, block))), dim3(block), 0, st,
                       term2_off, term2_path, term2_val, n2, W2, nelements, P2, channels, T2);
  }
  hipLaunchKernelGGL(copy_w1_kernel<S>, dim3(static_cast<unsigned>(ceil_div(nelements * channels, block))), dim3(block), 0,
                     st, W1, nelements, P1, channels, T1);
  return check_launch(what);
}

template <typename S>
int forward(const char *what, const S *X, const int32_t *node_perm, const int32_t *group_offsets, const int32_t *mono3_ijk,
            int n3, const int32_t *mono2_ij, int n2, const S *T3, const S *T2, const S *T1, int64_t nnodes, int nelements,
            int channels, S *out, S *grad, cm_stream_t stream) {
  CM_REQUIRE(cm_channels_supported(channels), "%s: channels=%d must be a multiple of 32 in [32, 256]", what, channels);
  CM_REQUIRE(nnodes >= 0 && nnodes < INT32_MAX / 16, "%s: nnodes out of range", what);
  CM_REQUIRE(nelements >= 1 && n3 >= 0 && n2 >= 0, "%s: bad sizes", what);
  if (nnodes == 0) return CM_OK;
  CM_REQUIRE(X && node_perm && group_offsets && T1 && out, "%s: NULL pointer", what);
  const bool builtin = mono3_ijk == nullptr && mono2_ij == nullptr;
  CM_REQUIRE(builtin || ((n3 == 0 || (mono3_ijk && T3)) && (n2 == 0 || (mono2_ij && T2))), "%s: NULL table", what);
  hipStream_t st = as_stream(stream);
  if (builtin) {
    // built-in l_max = 3 structure: unrolled register kernel
    CM_REQUIRE(n3 == CM_SYMCON_N3 && n2 == CM_SYMCON_N2,
               "%s: built-in structure has %d cubic and %d quadratic monomials, got %d and %d", what, CM_SYMCON_N3,
               CM_SYMCON_N2, n3, n2);
    CM_REQUIRE(T3 && T2, "%s: NULL table", what);
    const int64_t column_blocks = ceil_div(channels, kWave);
    const int64_t two_waves_per_simd = static_cast<int64_t>(device_compute_units()) * 4 * 2;
    const int npb = static_cast<int>(std::max<int64_t>(2, std::min<int64_t>(kMaxNodesPerBlock, nnodes * column_blocks / two_waves_per_simd)));
    const dim3 grid(static_cast<unsigned>(ceil_div(nnodes, npb) + nelements), static_cast<unsigned>(column_blocks));
    if (grad)
      hipLaunchKernelGGL((symcon_lmax3_kernel<S, true>), grid, dim3(kWave), 0, st, X, node_perm, group_offsets, T3, T2, T1,
                         static_cast<int>(nnodes), nelements, channels, npb, out, grad);
    else
      hipLaunchKernelGGL((symcon_lmax3_kernel<S, false>), grid, dim3(kWave), 0, st, X, node_perm, group_offsets, T3, T2, T1,
                         static_cast<int>(nnodes), nelements, channels, npb, out, grad);
    return check_launch(what);
  }
  // LDS per workgroup is held to 32 KB in fp32, 64 KB in fp64 (two [NB][16][C] arrays) so that several fit a CU
  if (channels <= 128) {
    const unsigned grid = static_cast<unsigned>(ceil_div(nnodes, 2) + nelements);
    launch_fwd<S, 2>(grad != nullptr, grid, channels, st, X, node_perm, group_offsets, mono3_ijk, n3, mono2_ij, n2, T3, T2, T1,
                     static_cast<int>(nnodes), nelements, out, grad);
  } else {
    const unsigned grid = static_cast<unsigned>(nnodes + nelements);
    launch_fwd<S, 1>(grad != nullptr, grid, channels, st, X, node_perm, group_offsets, mono3_ijk, n3, mono2_ij, n2, T3, T2, T1,
                     static_cast<int>(nnodes), nelements, out, grad);
  }
  return check_launch(what);
}

}  // namespace
}  // namespace cm

extern "C" int cm_symcon_tables(const int32_t *term3_off, const int32_t *term3_path, const float *term3_val, int n3,
                                const int32_t *term2_off, const int32_t *term2_path, const float *term2_val, int n2,
                                const float *W3, const float *W2, const float *W1, int nelements, int P3, int P2,
                                int P1, int channels, float *T3, float *T2, float *T1, cm_stream_t stream) {
  return cm::tables("cm_symcon_tables", term3_off, term3_path, term3_val, n3, term2_off, term2_path, term2_val, n2, W3, W2, W1,
                    nelements, P3, P2, P1, channels, T3, T2, T1, stream);
}

extern "C" int cm_symcon_tables_f64(const int32_t *term3_off, const int32_t *term3_path, const double *term3_val, int n3,
                                    const int32_t *term2_off, const int32_t *term2_path, const double *term2_val, int n2,
                                    const double *W3, const double *W2, const double *W1, int nelements, int P3, int P2,
                                    int P1, int channels, double *T3, double *T2, double *T1, cm_stream_t stream) {
  return cm::tables("cm_symcon_tables_f64", term3_off, term3_path, term3_val, n3, term2_off, term2_path, term2_val, n2, W3, W2,
                    W1, nelements, P3, P2, P1, channels, T3, T2, T1, stream);
}

extern "C" int cm_symcon_forward(const float *X, const int32_t *node_perm, const int32_t *group_offsets,
                                 const int32_t *mono3_ijk, int n3, const int32_t *mono2_ij, int n2, const float *T3,
                                 const float *T2, const float *T1, int64_t nnodes, int nelements, int channels,
                                 float *out, float *grad, cm_stream_t stream) {
  return cm::forward("cm_symcon_forward", X, node_perm, group_offsets, mono3_ijk, n3, mono2_ij, n2, T3, T2, T1, nnodes,
                     nelements, channels, out, grad, stream);
}

extern "C" int cm_symcon_forward_f64(const double *X, const int32_t *node_perm, const int32_t *group_offsets,
                                     const int32_t *mono3_ijk, int n3, const int32_t *mono2_ij, int n2, const double *T3,
                                     const double *T2, const double *T1, int64_t nnodes, int nelements, int channels,
                                     double *out, double *grad, cm_stream_t stream) {
  return cm::forward("cm_symcon_forward_f64", X, node_perm, group_offsets, mono3_ijk, n3, mono2_ij, n2, T3, T2, T1, nnodes,
                     nelements, channels, out, grad, stream);
}

extern "C" int cm_symcon_builtin_structure(int32_t *mono3_ijk, int capacity3, int32_t *mono2_ij, int capacity2,
                                           int *n3, int *n2) {
  static const int32_t k3[] = {
#define CM_PACK3(t, i, j, k) ((i) | ((j) << 8) | ((k) << 16)),
      CM_SYMCON_MONO3(CM_PACK3)
#undef CM_PACK3
  };
  static const int32_t k2[] = {
#define CM_PACK2(t, i, j) ((i) | ((j) << 8)),
      CM_SYMCON_MONO2(CM_PACK2)
#undef CM_PACK2
  };
  if (n3) *n3 = CM_SYMCON_N3;
  if (n2) *n2 = CM_SYMCON_N2;
  if (mono3_ijk) {
    CM_REQUIRE(capacity3 >= CM_SYMCON_N3, "cm_symcon_builtin_structure: mono3 buffer too small");
    for (int t = 0; t < CM_SYMCON_N3; ++t) mono3_ijk[t] = k3[t];
  }
  if (mono2_ij) {
    CM_REQUIRE(capacity2 >= CM_SYMCON_N2, "cm_symcon_builtin_structure: mono2 buffer too small");
    for (int t = 0; t < CM_SYMCON_N2; ++t) mono2_ij[t] = k2[t];
  }
  return CM_OK;
}

extern "C" int cm_symcon_backward(const float *grad, const float *grad_out, int64_t nnodes, int channels, float *gX,
                                  cm_stream_t stream) {
  CM_REQUIRE(channels >= 4 && channels % 4 == 0, "cm_symcon_backward: channels must be a multiple of 4");
  CM_REQUIRE(nnodes >= 0, "cm_symcon_backward: negative size");
  if (nnodes == 0) return CM_OK;
  CM_REQUIRE(grad && grad_out && gX, "cm_symcon_backward: NULL pointer");
  const int block = 256;
  const int64_t threads = nnodes * 16 * (channels / 4);
  hipLaunchKernelGGL(cm::symcon_backward_kernel, dim3(static_cast<unsigned>(cm::ceil_div(threads, block))), dim3(block), 0,
                     cm::as_stream(stream), grad, grad_out, nnodes, channels, gX);
  return cm::check_launch("cm_symcon_backward");
}

extern "C" int cm_symcon_backward_f64(const double *grad, const double *grad_out, int64_t nnodes, int channels, double *gX,
                                      cm_stream_t stream) {
  CM_REQUIRE(channels >= 1, "cm_symcon_backward_f64: channels must be positive");
  CM_REQUIRE(nnodes >= 0, "cm_symcon_backward_f64: negative size");
  if (nnodes == 0) return CM_OK;
  CM_REQUIRE(grad && grad_out && gX, "cm_symcon_backward_f64: NULL pointer");
  const int block = 256;
  const int64_t total = nnodes * 16 * channels;
  hipLaunchKernelGGL(cm::symcon_backward_f64_kernel, dim3(static_cast<unsigned>(cm::ceil_div(total, block))), dim3(block), 0,
                     cm::as_stream(stream), grad, grad_out, total, channels, gX);
  return cm::check_launch("cm_symcon_backward_f64");
}
