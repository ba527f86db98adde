// Invariant message passing with one radial weight per spherical-harmonic COMPONENT instead of one per degree:
//
//   out[n, m, c] = sum_{e -> n} X[sender[e], c] * Y[m, e] * R[e, m, c],        R [nedges, 16, channels]
//
// The reference's op takes R [nedges, 4, channels] (cuda/src/invariant_message_passing_impl.cu:138: the weight of
// component m is radial[edge * 4 * C + floor(sqrt(m)) * C + c]); this is the same op for callers that hold a weight per
// component (four times the radial bytes).  Same decomposition as the kernels of mp.hip: one wave per receiver node,
// a lane owns a few channels, Y and the senders of up to 64 edges staged in LDS, R streamed once (non-temporal), no
// atomics; the per-edge contributions to grad_X are summed per sender by the sender pass of mp.hip.
#include "mp_common.hpp"

namespace cm {
namespace {
using namespace mp;

template <int C>
__global__ __launch_bounds__(kWave) void mp_per_m_forward_kernel(const float *__restrict__ X, const float *__restrict__ Y,
                                                                const float *__restrict__ R,
                                                                const int32_t *__restrict__ sender,
                                                                const int32_t *__restrict__ first_occ, int nnodes,
                                                                int64_t nedges, float *__restrict__ out) {
  using K = Cfg<C>;  // at most four channels per lane: 16 weight vectors and 16 accumulators stay in registers
  using vec = typename K::vec;
  __shared__ __attribute__((aligned(16))) float sY[kChunk * 16];
  __shared__ int sS[kChunk];
  const int lane = threadIdx.x;
  const int slot = lane / K::SW;
  const int cl = lane % K::SW;
  const bool active = cl < K::LPE;
  const int node = blockIdx.x;
  int e0 = first_occ[node];
  int e1 = first_occ[nnodes + node];
  clamp_edge_range(e0, e1, nedges);

  vec acc[16];
#pragma unroll
  for (int m = 0; m < 16; ++m) acc[m] = zerov<vec>();
  for (int base = e0; base < e1; base += kChunk) {
    const int cnt = min(kChunk, e1 - base);
    __syncthreads();
    stage_chunk(Y, sender, nedges, base, cnt, lane, sY, sS);
    __syncthreads();
    if (active) {
      auto one = [&](int j) {
        const int64_t e = base + j;
        const int s = sS[j];
        const float *rp = R + e * (16 * C) + K::off(cl);
        vec r[16];
#pragma unroll
        for (int m = 0; m < 16; ++m) r[m] = K::ld_stream(rp + m * C);
        vec x = zerov<vec>();
        if (static_cast<unsigned>(s) < static_cast<unsigned>(nnodes)) x = K::ld(X + static_cast<int64_t>(s) * C + K::off(cl));
        const float *yp = sY + j * 16;
#pragma unroll
        for (int m = 0; m < 16; ++m) acc[m] += (yp[m] * x) * r[m];
      };
      // two edges per slot at a time, their 2 x 16 rows requested together
      int j = slot;
      for (; j + K::EPW < cnt; j += 2 * K::EPW) {
        one(j);
        one(j + K::EPW);
      }
      if (j < cnt) one(j);
    }
  }
#pragma unroll
  for (int off = kWave / 2; off >= K::SW; off >>= 1) {
#pragma unroll
    for (int m = 0; m < 16; ++m) acc[m] += shfl_downv(acc[m], off);
  }
  if (slot == 0 && active) {
    float *op = out + static_cast<int64_t>(node) * (16 * C) + K::off(cl);
#pragma unroll
    for (int m = 0; m < 16; ++m) K::st_stream(op + m * C, acc[m]);
  }
}

// gR[e, m, c] = X[s, c] Y[m, e] g[n, m, c];  gY[m, e] = sum_c g[n, m, c] R[e, m, c] X[s, c];
// gXe[e, c] = sum_m g[n, m, c] R[e, m, c] Y[m, e]
template <int C, bool WANT_GY, bool WANT_GR, bool WANT_GX>
__global__ __launch_bounds__(kWave) void mp_per_m_backward_edge_kernel(
    const float *__restrict__ X, const float *__restrict__ Y, const float *__restrict__ R, const float *__restrict__ G,
    const int32_t *__restrict__ sender, const int32_t *__restrict__ first_occ, int nnodes, int64_t nedges,
    float *__restrict__ gY, float *__restrict__ gR, float *__restrict__ gXe) {
  using K = Cfg<C>;
  using vec = typename K::vec;
  __shared__ __attribute__((aligned(16))) float sY[kChunk * 16];
  __shared__ int sS[kChunk];
  __shared__ float sGY[16 * kChunk];  // [m][edge]
  const int node = blockIdx.x;
  const int lane = threadIdx.x;
  const int slot = lane / K::SW;
  const int cl = lane % K::SW;
  const bool active = cl < K::LPE;
  int e0 = first_occ[node];
  int e1 = first_occ[nnodes + node];
  clamp_edge_range(e0, e1, nedges);
  if (e0 >= e1) return;

  vec g[16];
  {
    const float *gp = G + static_cast<int64_t>(node) * (16 * C) + K::off(cl);
#pragma unroll
    for (int m = 0; m < 16; ++m) g[m] = active ? K::ld(gp + m * C) : zerov<vec>();
  }
  for (int base = e0; base < e1; base += kChunk) {
    const int cnt = min(kChunk, e1 - base);
    __syncthreads();
    stage_chunk(Y, sender, nedges, base, cnt, lane, sY, sS);
    __syncthreads();
    // every lane of a slot takes part in the reduction, so the loop bound is slot-uniform
    for (int j = slot; j < cnt; j += K::EPW) {
      const int64_t e = base + j;
      const int s = sS[j];
      vec x = zerov<vec>();
      if (active && static_cast<unsigned>(s) < static_cast<unsigned>(nnodes)) x = K::ld(X + static_cast<int64_t>(s) * C + K::off(cl));
      const float *yp = sY + j * 16;
      const float *rp = R + e * (16 * C) + K::off(cl);
      vec gx = zerov<vec>();
      float p[16];
#pragma unroll
      for (int m = 0; m < 16; ++m) {
        const vec yg = yp[m] * g[m];
        if constexpr (WANT_GR) {
          if (active) K::st_stream(gR + e * (16 * C) + m * C + K::off(cl), x * yg);
        }
        if constexpr (WANT_GY || WANT_GX) {
          const vec r = active ? K::ld_stream(rp + m * C) : zerov<vec>();
          if constexpr (WANT_GX) gx += r * yg;
          if constexpr (WANT_GY) p[m] = dotv(g[m], x * r);
        }
      }
      if constexpr (WANT_GX) {
        if (active) K::st_stream(gXe + e * C + K::off(cl), gx);
      }
      if constexpr (WANT_GY) {
        slot_reduce16<K::SW>(p, cl);
        store_reduced16<K::SW>(p, cl, j, sGY);
      }
    }
    if constexpr (WANT_GY) {
      __syncthreads();
      if (lane < cnt) {
        const int64_t e = base + lane;
#pragma unroll
        for (int m = 0; m < 16; ++m) gY[m * nedges + e] = sGY[m * kChunk + lane];
      }
    }
  }
}

template <int C, bool GY, bool GR, bool GX>
void launch_edge(const float *X, const float *Y, const float *R, const float *G, const int32_t *sender,
                 const int32_t *first_occ, int64_t nnodes, int64_t nedges, float *gY, float *gR, float *gXe, hipStream_t st) {
  hipLaunchKernelGGL((mp_per_m_backward_edge_kernel<C, GY, GR, GX>), dim3(static_cast<unsigned>(nnodes)), dim3(kWave), 0, st, X, Y,
                     R, G, sender, first_occ, static_cast<int>(nnodes), nedges, gY, gR, gXe);
}

template <int C>
int launch_backward(const float *X, const float *Y, const float *R, const float *G, const int32_t *sender,
                    const int32_t *first_occ, const int32_t *perm, const int32_t *offsets, int64_t nnodes, int64_t nedges,
                    float *gX, float *gY, float *gR, float *gXe, hipStream_t st) {
  const int key = (gY ? 4 : 0) | (gR ? 2 : 0) | (gX ? 1 : 0);
  switch (key) {
    case 7: launch_edge<C, true, true, true>(X, Y, R, G, sender, first_occ, nnodes, nedges, gY, gR, gXe, st); break;
    case 6: launch_edge<C, true, true, false>(X, Y, R, G, sender, first_occ, nnodes, nedges, gY, gR, gXe, st); break;
    case 5: launch_edge<C, true, false, true>(X, Y, R, G, sender, first_occ, nnodes, nedges, gY, gR, gXe, st); break;
    case 4: launch_edge<C, true, false, false>(X, Y, R, G, sender, first_occ, nnodes, nedges, gY, gR, gXe, st); break;
    case 3: launch_edge<C, false, true, true>(X, Y, R, G, sender, first_occ, nnodes, nedges, gY, gR, gXe, st); break;
    case 2: launch_edge<C, false, true, false>(X, Y, R, G, sender, first_occ, nnodes, nedges, gY, gR, gXe, st); break;
    case 1: launch_edge<C, false, false, true>(X, Y, R, G, sender, first_occ, nnodes, nedges, gY, gR, gXe, st); break;
    default: return CM_OK;
  }
  int rc = check_launch("cm_mp_backward_per_m (edge pass)");
  if (rc != CM_OK) return rc;
  if (gX) rc = mp::launch_sender_pass(C, gXe, perm, offsets, nnodes, nedges, gX, st);
  return rc;
}

}  // namespace
}  // namespace cm

extern "C" int cm_mp_forward_per_m(const float *X, const float *Y, const float *R, const int32_t *sender,
                                   const int32_t *first_occ, int64_t nnodes, int64_t nedges, int channels, float *out,
                                   cm_stream_t stream) {
  CM_REQUIRE(cm_channels_supported(channels), "cm_mp_forward_per_m: channels=%d must be a multiple of 32 in [32, 256]", channels);
  CM_REQUIRE(nedges >= 0 && nnodes >= 0, "cm_mp_forward_per_m: negative size");
  CM_REQUIRE(nedges < INT32_MAX && nnodes < INT32_MAX / 2, "cm_mp_forward_per_m: sizes exceed int32 indexing");
  if (nnodes == 0) return CM_OK;
  CM_REQUIRE(X && first_occ && out, "cm_mp_forward_per_m: NULL pointer");
  CM_REQUIRE(nedges == 0 || (Y && R && sender), "cm_mp_forward_per_m: NULL edge operand");
  int rc = CM_EINVAL;
  CM_DISPATCH_C(channels, {
    hipLaunchKernelGGL(cm::mp_per_m_forward_kernel<C_>, dim3(static_cast<unsigned>(nnodes)), dim3(cm::kWave), 0, cm::as_stream(stream),
                       X, Y, R, sender, first_occ, static_cast<int>(nnodes), nedges, out);
    rc = cm::check_launch("cm_mp_forward_per_m");
  });
  return rc;
}

extern "C" int cm_mp_backward_per_m(const float *X, const float *Y, const float *R, const float *grad_out,
                                    const int32_t *sender, const int32_t *first_occ, const int32_t *sender_perm,
                                    const int32_t *sender_offsets, int64_t nnodes, int64_t nedges, int channels, float *gX,
                                    float *gY, float *gR, float *edge_scratch, cm_stream_t stream) {
  CM_REQUIRE(cm_channels_supported(channels), "cm_mp_backward_per_m: channels=%d must be a multiple of 32 in [32, 256]", channels);
  CM_REQUIRE(nedges >= 0 && nnodes >= 0, "cm_mp_backward_per_m: negative size");
  CM_REQUIRE(nedges < INT32_MAX && nnodes < INT32_MAX / 2, "cm_mp_backward_per_m: sizes exceed int32 indexing");
  if (nnodes == 0 || (!gX && !gY && !gR)) return CM_OK;
  CM_REQUIRE(X && grad_out && first_occ, "cm_mp_backward_per_m: NULL pointer");
  CM_REQUIRE(nedges == 0 || (Y && R && sender), "cm_mp_backward_per_m: NULL edge operand");
  CM_REQUIRE(!gX || (sender_offsets && (nedges == 0 || (sender_perm && edge_scratch))),
             "cm_mp_backward_per_m: gX needs sender_perm, sender_offsets and edge_scratch");
  int rc = CM_EINVAL;
  CM_DISPATCH_C(channels, rc = cm::launch_backward<C_>(X, Y, R, grad_out, sender, first_occ, sender_perm, sender_offsets, nnodes,
                                                       nedges, gX, gY, gR, edge_scratch, cm::as_stream(stream)));
  return rc;
}
