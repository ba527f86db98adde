// Invariant message passing in fp64: forward and backward.
//
// The reference dispatches its message-passing kernels on float and double
// (jit_wrappers/src/invariant_message_passing_wrapper.cpp:102, :189); the model runs them in fp32, the double path
// serves accuracy studies and gradient checks.  Same operands and outputs as the fp32 entry points, in double.
//
// Work decomposition: one wavefront per receiver node; lane i owns channels i, i + 64, ... (KS = ceil(C / 64) of
// them), so every row access of X, R, grad_R and the per-edge scratch is a contiguous 512-byte segment per k.  The
// node's 16 x C accumulator (forward) or incoming gradient (backward) stays in registers while the wave walks the
// node's edges in order; Y[:, e] and sender[e] are wave-uniform loads.  Sums over edges run in edge order and sums
// over channels in a fixed butterfly, with no atomics: results are reproducible bit for bit.
#include "common.hpp"

namespace cm {
namespace {

// Butterfly over the wave that also transposes: on entry every lane holds 16 partial sums p[m]; on return the lane
// holds in p[0] the full sum of component m = 8 * bit5 + 4 * bit4 + 2 * bit3 + bit2 of its lane index.
__device__ __forceinline__ void wave_reduce16(double (&p)[16], int lane) {
#pragma unroll
  for (int level = 0; level < 4; ++level) {
    const int half = 8 >> level;  // values kept after this level
    const int off = 32 >> level;
    const bool up = (lane & off) != 0;
#pragma unroll
    for (int i = 0; i < half; ++i) {
      const double keep = up ? p[half + i] : p[i];
      const double give = up ? p[i] : p[half + i];
      p[i] = keep + __shfl_xor(give, off);
    }
  }
  p[0] += __shfl_xor(p[0], 2);
  p[0] += __shfl_xor(p[0], 1);
}

template <int KS>
__global__ __launch_bounds__(kWave) void mp_forward_f64_kernel(const double *__restrict__ X, const double *__restrict__ Y,
                                                              const double *__restrict__ R,
                                                              const int32_t *__restrict__ sender,
                                                              const int32_t *__restrict__ first_occ, int nnodes,
                                                              int64_t nedges, int C, double *__restrict__ out) {
  const int lane = threadIdx.x;
  const int node = blockIdx.x;
  int e0 = first_occ[node];
  int e1 = first_occ[nnodes + node];
  clamp_edge_range(e0, e1, nedges);
  double acc[16][KS];
#pragma unroll
  for (int m = 0; m < 16; ++m)
#pragma unroll
    for (int k = 0; k < KS; ++k) acc[m][k] = 0.0;

  for (int64_t e = e0; e < e1; ++e) {
    const int s = sender[e];
    const bool valid = static_cast<unsigned>(s) < static_cast<unsigned>(nnodes);
    double y[16];
#pragma unroll
    for (int m = 0; m < 16; ++m) y[m] = Y[m * nedges + e];
#pragma unroll
    for (int k = 0; k < KS; ++k) {
      const int c = lane + kWave * k;
      if (c < C) {
        const double x = valid ? X[static_cast<int64_t>(s) * C + c] : 0.0;
        const double *rp = R + e * (4 * C) + c;
        const double t[4] = {x * rp[0], x * rp[C], x * rp[2 * C], x * rp[3 * C]};
#pragma unroll
        for (int m = 0; m < 16; ++m) acc[m][k] = fma(y[m], t[l_of_m(m)], acc[m][k]);
      }
    }
  }
#pragma unroll
  for (int k = 0; k < KS; ++k) {
    const int c = lane + kWave * k;
    if (c < C) {
#pragma unroll
      for (int m = 0; m < 16; ++m) out[(static_cast<int64_t>(node) * 16 + m) * C + c] = acc[m][k];
    }
  }
}

template <int KS, bool WANT_GY, bool WANT_GR, bool WANT_GX>
__global__ __launch_bounds__(kWave) void mp_backward_edge_f64_kernel(
    const double *__restrict__ X, const double *__restrict__ Y, const double *__restrict__ R, const double *__restrict__ G,
    const int32_t *__restrict__ sender, const int32_t *__restrict__ first_occ, int nnodes, int64_t nedges, int C,
    double *__restrict__ gY, double *__restrict__ gR, double *__restrict__ gXe) {
  const int lane = threadIdx.x;
  const int node = blockIdx.x;
  int e0 = first_occ[node];
  int e1 = first_occ[nnodes + node];
  clamp_edge_range(e0, e1, nedges);
  if (e0 >= e1) return;

  double g[16][KS];
#pragma unroll
  for (int k = 0; k < KS; ++k) {
    const int c = lane + kWave * k;
#pragma unroll
    for (int m = 0; m < 16; ++m) g[m][k] = c < C ? G[(static_cast<int64_t>(node) * 16 + m) * C + c] : 0.0;
  }
  const int mine = ((lane >> 5) & 1) * 8 + ((lane >> 4) & 1) * 4 + ((lane >> 3) & 1) * 2 + ((lane >> 2) & 1);

  for (int64_t e = e0; e < e1; ++e) {
    const int s = sender[e];
    const bool valid = static_cast<unsigned>(s) < static_cast<unsigned>(nnodes);
    double y[16], p[16];
#pragma unroll
    for (int m = 0; m < 16; ++m) {
      y[m] = Y[m * nedges + e];
      p[m] = 0.0;
    }
#pragma unroll
    for (int k = 0; k < KS; ++k) {
      const int c = lane + kWave * k;
      if (c < C) {
        const double x = valid ? X[static_cast<int64_t>(s) * C + c] : 0.0;
        const double *rp = R + e * (4 * C) + c;
        const double r[4] = {rp[0], rp[C], rp[2 * C], rp[3 * C]};
        if constexpr (WANT_GR || WANT_GX) {
          double q[4] = {0.0, 0.0, 0.0, 0.0};
#pragma unroll
          for (int m = 0; m < 16; ++m) q[l_of_m(m)] = fma(y[m], g[m][k], q[l_of_m(m)]);
          if constexpr (WANT_GR) {
            double *gp = gR + e * (4 * C) + c;
#pragma unroll
            for (int l = 0; l < 4; ++l) gp[l * C] = x * q[l];
          }
          if constexpr (WANT_GX) gXe[e * C + c] = (r[0] * q[0] + r[1] * q[1]) + (r[2] * q[2] + r[3] * q[3]);
        }
        if constexpr (WANT_GY) {
#pragma unroll
          for (int m = 0; m < 16; ++m) p[m] = fma(g[m][k], x * r[l_of_m(m)], p[m]);
        }
      }
    }
    if constexpr (WANT_GY) {
      wave_reduce16(p, lane);
      if ((lane & 3) == 0) gY[mine * nedges + e] = p[0];
    }
  }
}

// gX[n, :] = sum, in the order of the sender-sorted view, of the per-edge rows gXe[e, :] of the edges sent by n
template <int KS>
__global__ __launch_bounds__(kWave) void mp_backward_sender_f64_kernel(const double *__restrict__ gXe,
                                                                      const int32_t *__restrict__ perm,
                                                                      const int32_t *__restrict__ offsets, int64_t nedges,
                                                                      int C, double *__restrict__ gX) {
  const int lane = threadIdx.x;
  const int node = blockIdx.x;
  double acc[KS];
#pragma unroll
  for (int k = 0; k < KS; ++k) acc[k] = 0.0;
  for (int q = offsets[node]; q < offsets[node + 1]; ++q) {
    const int e = perm[q];
    if (static_cast<unsigned>(e) >= static_cast<uint64_t>(nedges)) continue;
#pragma unroll
    for (int k = 0; k < KS; ++k) {
      const int c = lane + kWave * k;
      if (c < C) acc[k] += gXe[static_cast<int64_t>(e) * C + c];
    }
  }
#pragma unroll
  for (int k = 0; k < KS; ++k) {
    const int c = lane + kWave * k;
    if (c < C) gX[static_cast<int64_t>(node) * C + c] = acc[k];
  }
}

template <int KS, bool GY, bool GR, bool GX>
void launch_edge(const double *X, const double *Y, const double *R, const double *G, const int32_t *sender,
                 const int32_t *first_occ, int64_t nnodes, int64_t nedges, int C, double *gY, double *gR, double *gXe,
                 hipStream_t st) {
  hipLaunchKernelGGL((mp_backward_edge_f64_kernel<KS, GY, GR, GX>), dim3(static_cast<unsigned>(nnodes)), dim3(kWave), 0, st,
                     X, Y, R, G, sender, first_occ, static_cast<int>(nnodes), nedges, C, gY, gR, gXe);
}

template <int KS>
int launch_backward(const double *X, const double *Y, const double *R, const double *G, const int32_t *sender,
                    const int32_t *first_occ, const int32_t *perm, const int32_t *offsets, int64_t nnodes, int64_t nedges,
                    int C, double *gX, double *gY, double *gR, double *gXe, hipStream_t st) {
  const int key = (gY ? 4 : 0) | (gR ? 2 : 0) | (gX ? 1 : 0);
  switch (key) {
    case 7: launch_edge<KS, true, true, true>(X, Y, R, G, sender, first_occ, nnodes, nedges, C, gY, gR, gXe, st); break;
    case 6: launch_edge<KS, true, true, false>(X, Y, R, G, sender, first_occ, nnodes, nedges, C, gY, gR, gXe, st); break;
    case 5: launch_edge<KS, true, false, true>(X, Y, R, G, sender, first_occ, nnodes, nedges, C, gY, gR, gXe, st); break;
    case 4: launch_edge<KS, true, false, false>(X, Y, R, G, sender, first_occ, nnodes, nedges, C, gY, gR, gXe, st); break;
    case 3: launch_edge<KS, false, true, true>(X, Y, R, G, sender, first_occ, nnodes, nedges, C, gY, gR, gXe, st); break;
    case 2: launch_edge<KS, false, true, false>(X, Y, R, G, sender, first_occ, nnodes, nedges, C, gY, gR, gXe, st); break;
    case 1: launch_edge<KS, false, false, true>(X, Y, R, G, sender, first_occ, nnodes, nedges, C, gY, gR, gXe, st); break;
    default: return CM_OK;
  }
  int rc = check_launch("cm_mp_backward_f64 (edge pass)");
  if (rc != CM_OK || !gX) return rc;
  hipLaunchKernelGGL(mp_backward_sender_f64_kernel<KS>, dim3(static_cast<unsigned>(nnodes)), dim3(kWave), 0, st, gXe, perm,
                     offsets, nedges, C, gX);
  return check_launch("cm_mp_backward_f64 (sender pass)");
}

}  // namespace
}  // namespace cm

#define CM_DISPATCH_KS(channels, ...)          \
  switch (((channels) + cm::kWave - 1) / cm::kWave) { \
    case 1: { constexpr int KS_ = 1; __VA_ARGS__; break; } \
    case 2: { constexpr int KS_ = 2; __VA_ARGS__; break; } \
    case 3: { constexpr int KS_ = 3; __VA_ARGS__; break; } \
    default: { constexpr int KS_ = 4; __VA_ARGS__; break; } \
  }

extern "C" int cm_mp_forward_f64(const double *X, const double *Y, const double *R, const int32_t *sender,
                                 const int32_t *first_occ, int64_t nnodes, int64_t nedges, int channels, double *out,
                                 cm_stream_t stream) {
  CM_REQUIRE(cm_channels_supported(channels), "cm_mp_forward_f64: channels=%d must be a multiple of 32 in [32, 256]", channels);
  CM_REQUIRE(nedges >= 0 && nnodes >= 0, "cm_mp_forward_f64: negative size");
  CM_REQUIRE(nedges < INT32_MAX && nnodes < INT32_MAX / 2, "cm_mp_forward_f64: sizes exceed int32 indexing");
  if (nnodes == 0) return CM_OK;
  CM_REQUIRE(X && first_occ && out, "cm_mp_forward_f64: NULL pointer");
  CM_REQUIRE(nedges == 0 || (Y && R && sender), "cm_mp_forward_f64: NULL edge operand");
  CM_DISPATCH_KS(channels, hipLaunchKernelGGL(cm::mp_forward_f64_kernel<KS_>, dim3(static_cast<unsigned>(nnodes)),
                                              dim3(cm::kWave), 0, cm::as_stream(stream), X, Y, R, sender, first_occ,
                                              static_cast<int>(nnodes), nedges, channels, out));
  return cm::check_launch("cm_mp_forward_f64");
}

extern "C" int cm_mp_backward_f64(const double *X, const double *Y, const double *R, const double *grad_out,
                                  const int32_t *sender, const int32_t *first_occ, const int32_t *sender_perm,
                                  const int32_t *sender_offsets, int64_t nnodes, int64_t nedges, int channels, double *gX,
                                  double *gY, double *gR, double *edge_scratch, cm_stream_t stream) {
  CM_REQUIRE(cm_channels_supported(channels), "cm_mp_backward_f64: channels=%d must be a multiple of 32 in [32, 256]", channels);
  CM_REQUIRE(nedges >= 0 && nnodes >= 0, "cm_mp_backward_f64: negative size");
  CM_REQUIRE(nedges < INT32_MAX && nnodes < INT32_MAX / 2, "cm_mp_backward_f64: sizes exceed int32 indexing");
  if (nnodes == 0) return CM_OK;
  CM_REQUIRE(X && grad_out && first_occ, "cm_mp_backward_f64: NULL pointer");
  CM_REQUIRE(nedges == 0 || (Y && R && sender), "cm_mp_backward_f64: NULL edge operand");
  CM_REQUIRE(!gX || (sender_offsets && (nedges == 0 || (sender_perm && edge_scratch))),
             "cm_mp_backward_f64: gX wanted but sender_perm / sender_offsets / edge_scratch missing");
  int rc = CM_EINVAL;
  CM_DISPATCH_KS(channels, rc = cm::launch_backward<KS_>(X, Y, R, grad_out, sender, first_occ, sender_perm, sender_offsets, nnodes,
                                                         nedges, channels, gX, gY, gR, edge_scratch, cm::as_stream(stream)));
  return rc;
}
