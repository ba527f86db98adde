// Invariant message passing for gfx950: CSR offsets, forward, backward.
//
// Work decomposition (all three big kernels): one wavefront per receiver node.  A lane owns four
// consecutive channels (one 16-byte load per row), so an edge occupies LPE = C/4 lanes; a wave is
// split into EPW = 64 / pow2ceil(LPE) slots that walk the node's contiguous edge range
// interleaved.  The radial weights R[e, 0:4, :] -- the one large operand -- are streamed from
// HBM straight into registers exactly once; the node's 16 x C accumulator (forward) or incoming
// gradient (backward) lives in registers for the whole segment; Y[0:16, e] and sender[e] of up to
// 64 edges are staged through LDS with coalesced row reads.  No atomics anywhere: partial sums
// of the slots are combined with cross-lane moves in a fixed order, so results are reproducible
// bit for bit.
#include "mp_common.hpp"

namespace cm {
namespace {

using namespace mp;

// -----------------------------------------------------------------------------------------------
// CSR offsets.  Thread e looks at receiver[e-1] -> receiver[e]; a change of value closes every
// node in (prev, cur) and opens every node in (prev, cur].  The last thread closes the tail.
// -----------------------------------------------------------------------------------------------
__global__ void first_occurences_kernel(const int32_t *__restrict__ receiver, int nedges, int nnodes,
                                        int32_t *__restrict__ first_occ) {
  const int e = blockIdx.x * blockDim.x + threadIdx.x;
  int32_t *start = first_occ;
  int32_t *end = first_occ + nnodes;
  if (nedges == 0) {
    for (int n = e; n < nnodes; n += gridDim.x * blockDim.x) {
      start[n] = 0;
      end[n] = 0;
    }
    return;
  }
  if (e >= nedges) return;
  int cur = receiver[e];
  cur = cur < 0 ? 0 : (cur >= nnodes ? nnodes - 1 : cur);
  int prev = -1;
  if (e > 0) {
    prev = receiver[e - 1];
    prev = prev < 0 ? 0 : (prev >= nnodes ? nnodes - 1 : prev);
  }
  for (int n = prev + 1; n <= cur; ++n) start[n] = e;
  for (int n = prev < 0 ? 0 : prev; n < cur; ++n) end[n] = e;
  if (e == nedges - 1) {
    end[cur] = nedges;
    for (int n = cur + 1; n < nnodes; ++n) {
      start[n] = nedges;
      end[n] = nedges;
    }
  }
}

// -----------------------------------------------------------------------------------------------
// forward
// -----------------------------------------------------------------------------------------------
template <int C>
__global__ __launch_bounds__(kWave) void mp_forward_kernel(
    const float *__restrict__ X, const float *__restrict__ Y, const float *__restrict__ R,
    const int32_t *__restrict__ sender, const int32_t *__restrict__ first_occ, int nnodes,
    int64_t nedges, float *__restrict__ out) {
  using K = Cfg<C, true>;
  using vec = typename K::vec;
  __shared__ __attribute__((aligned(16))) float sY[kChunk * 16];
  __shared__ int sS[kChunk];

  const int lane = threadIdx.x;
  const int slot = lane / K::SW;
  const int cl = lane % K::SW;
  const bool active = cl < K::LPE;
  const int node = blockIdx.x;
  const int e0 = first_occ[node];
  const int e1 = first_occ[nnodes + node];

  vec acc[16];
#pragma unroll
  for (int m = 0; m < 16; ++m) acc[m] = zerov<vec>();

  for (int base = e0; base < e1; base += kChunk) {
    const int cnt = min(kChunk, e1 - base);
    __syncthreads();
    stage_chunk(Y, sender, nedges, base, cnt, lane, sY, sS);
    __syncthreads();
    if (active) {
#pragma unroll 2
      for (int j = slot; j < cnt; j += K::EPW) {
        const int64_t e = base + j;
        const int s = sS[j];
        const float *rp = R + e * (4 * C) + K::off(cl);
        vec r0 = K::ld_stream(rp);
        vec r1 = K::ld_stream(rp + C);
        vec r2 = K::ld_stream(rp + 2 * C);
        vec r3 = K::ld_stream(rp + 3 * C);
        vec x = zerov<vec>();
        if (static_cast<unsigned>(s) < static_cast<unsigned>(nnodes)) x = K::ld(X + static_cast<int64_t>(s) * C + K::off(cl));
        const f4 *yp = reinterpret_cast<const f4 *>(sY + j * 16);
        const f4 ya = yp[0], yb = yp[1], yc = yp[2], yd = yp[3];
        const vec t0 = x * r0, t1 = x * r1, t2 = x * r2, t3 = x * r3;
        acc[0] += ya.x * t0;
        acc[1] += ya.y * t1;
        acc[2] += ya.z * t1;
        acc[3] += ya.w * t1;
        acc[4] += yb.x * t2;
        acc[5] += yb.y * t2;
        acc[6] += yb.z * t2;
        acc[7] += yb.w * t2;
        acc[8] += yc.x * t2;
        acc[9] += yc.y * t3;
        acc[10] += yc.z * t3;
        acc[11] += yc.w * t3;
        acc[12] += yd.x * t3;
        acc[13] += yd.y * t3;
        acc[14] += yd.z * t3;
        acc[15] += yd.w * t3;
      }
    }
  }

  // combine the slots: after the tree, slot 0 holds the node's sums
#pragma unroll
  for (int off = kWave / 2; off >= K::SW; off >>= 1) {
#pragma unroll
    for (int m = 0; m < 16; ++m) acc[m] += shfl_downv(acc[m], off);
  }
  if (slot == 0 && active) {
    // streamed out (non-temporal): measured 5 % faster than regular stores, which compete with the R stream for L2
    float *op = out + static_cast<int64_t>(node) * (16 * C) + K::off(cl);
#pragma unroll
    for (int m = 0; m < 16; ++m) K::st_stream(op + m * C, acc[m]);
  }
}

// -----------------------------------------------------------------------------------------------
// backward, edge pass: gR, gY and the per-edge contribution to gX
// -----------------------------------------------------------------------------------------------
template <int C, bool WANT_GY, bool WANT_GR, bool WANT_GX>
__global__ __launch_bounds__(kWave) void mp_backward_edge_kernel(
    const float *__restrict__ X, const float *__restrict__ Y, const float *__restrict__ R,
    const float *__restrict__ G, const int32_t *__restrict__ sender,
    const int32_t *__restrict__ first_occ, int nnodes, int64_t nedges, float *__restrict__ gY,
    float *__restrict__ gR, float *__restrict__ gXe) {
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
  const int e0 = first_occ[node];
  const int e1 = first_occ[nnodes + node];
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
      vec r0 = zerov<vec>(), r1 = zerov<vec>(), r2 = zerov<vec>(), r3 = zerov<vec>(), x = zerov<vec>();
      if (active) {
        const float *rp = R + e * (4 * C) + K::off(cl);
        r0 = K::ld_stream(rp);
        r1 = K::ld_stream(rp + C);
        r2 = K::ld_stream(rp + 2 * C);
        r3 = K::ld_stream(rp + 3 * C);
        if (static_cast<unsigned>(s) < static_cast<unsigned>(nnodes)) x = K::ld(X + static_cast<int64_t>(s) * C + K::off(cl));
      }
      const f4 *yp = reinterpret_cast<const f4 *>(sY + j * 16);
      const f4 ya = yp[0], yb = yp[1], yc = yp[2], yd = yp[3];

      if constexpr (WANT_GR || WANT_GX) {
        // q_l = sum_{m in l} Y[m] g[m]
        const vec q0 = ya.x * g[0];
        const vec q1 = ya.y * g[1] + ya.z * g[2] + ya.w * g[3];
        const vec q2 = yb.x * g[4] + yb.y * g[5] + yb.z * g[6] + yb.w * g[7] + yc.x * g[8];
        const vec q3 = yc.y * g[9] + yc.z * g[10] + yc.w * g[11] + yd.x * g[12] + yd.y * g[13] +
                      yd.z * g[14] + yd.w * g[15];
        if (active) {
          if constexpr (WANT_GR) {
            float *gp = gR + e * (4 * C) + K::off(cl);
            K::st_stream(gp, x * q0);
            K::st_stream(gp + C, x * q1);
            K::st_stream(gp + 2 * C, x * q2);
            K::st_stream(gp + 3 * C, x * q3);
          }
          if constexpr (WANT_GX) {
            K::st_stream(gXe + e * C + K::off(cl), r0 * q0 + r1 * q1 + r2 * q2 + r3 * q3);
          }
        }
      }
      if constexpr (WANT_GY) {
        const vec t0 = x * r0, t1 = x * r1, t2 = x * r2, t3 = x * r3;
        float p[16];
        p[0] = dotv(g[0], t0);
        p[1] = dotv(g[1], t1);
        p[2] = dotv(g[2], t1);
        p[3] = dotv(g[3], t1);
        p[4] = dotv(g[4], t2);
        p[5] = dotv(g[5], t2);
        p[6] = dotv(g[6], t2);
        p[7] = dotv(g[7], t2);
        p[8] = dotv(g[8], t2);
        p[9] = dotv(g[9], t3);
        p[10] = dotv(g[10], t3);
        p[11] = dotv(g[11], t3);
        p[12] = dotv(g[12], t3);
        p[13] = dotv(g[13], t3);
        p[14] = dotv(g[14], t3);
        p[15] = dotv(g[15], t3);
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

// -----------------------------------------------------------------------------------------------
// backward, sender pass: gX[n, :] = sum over the edges sent by n of the per-edge contributions
// -----------------------------------------------------------------------------------------------
template <int C>
__global__ __launch_bounds__(kWave) void mp_backward_sender_kernel(
    const float *__restrict__ gXe, const int32_t *__restrict__ perm,
    const int32_t *__restrict__ offsets, int nnodes, int64_t nedges, float *__restrict__ gX) {
  using K = Cfg<C>;
  using vec = typename K::vec;
  const int node = blockIdx.x;
  const int lane = threadIdx.x;
  const int slot = lane / K::SW;
  const int cl = lane % K::SW;
  const bool active = cl < K::LPE;
  const int k0 = offsets[node];
  const int k1 = offsets[node + 1];
  vec acc = zerov<vec>();
  if (active) {
    // four independent row gathers in flight per slot; the summation order stays fixed.  Every row is read exactly
    // once: streamed loads
    int k = k0 + slot;
    for (; k + 3 * K::EPW < k1; k += 4 * K::EPW) {
      const int ea = perm[k], eb = perm[k + K::EPW], ec = perm[k + 2 * K::EPW], ed = perm[k + 3 * K::EPW];
      const vec va = static_cast<unsigned>(ea) < static_cast<uint64_t>(nedges) ? K::ld_stream(gXe + static_cast<int64_t>(ea) * C + K::off(cl)) : zerov<vec>();
      const vec vb = static_cast<unsigned>(eb) < static_cast<uint64_t>(nedges) ? K::ld_stream(gXe + static_cast<int64_t>(eb) * C + K::off(cl)) : zerov<vec>();
      const vec vc = static_cast<unsigned>(ec) < static_cast<uint64_t>(nedges) ? K::ld_stream(gXe + static_cast<int64_t>(ec) * C + K::off(cl)) : zerov<vec>();
      const vec vd = static_cast<unsigned>(ed) < static_cast<uint64_t>(nedges) ? K::ld_stream(gXe + static_cast<int64_t>(ed) * C + K::off(cl)) : zerov<vec>();
      acc += (va + vb) + (vc + vd);
    }
    for (; k < k1; k += K::EPW) {
      const int e = perm[k];
      if (static_cast<unsigned>(e) < static_cast<uint64_t>(nedges)) acc += K::ld_stream(gXe + static_cast<int64_t>(e) * C + K::off(cl));
    }
  }
#pragma unroll
  for (int off = kWave / 2; off >= K::SW; off >>= 1) acc += shfl_downv(acc, off);
  if (slot == 0 && active) K::st(gX + static_cast<int64_t>(node) * C + K::off(cl), acc);
}

template <int C>
int launch_forward(const float *X, const float *Y, const float *R, const int32_t *sender,
                   const int32_t *first_occ, int64_t nnodes, int64_t nedges, float *out,
                   hipStream_t st) {
  hipLaunchKernelGGL(mp_forward_kernel<C>, dim3(static_cast<unsigned>(nnodes)), dim3(kWave), 0, st, X, Y, R,
                     sender, first_occ, static_cast<int>(nnodes), nedges, out);
  return check_launch("cm_mp_forward");
}

template <int C, bool GY, bool GR, bool GX>
void launch_edge(const float *X, const float *Y, const float *R, const float *G, const int32_t *sender,
                 const int32_t *first_occ, int64_t nnodes, int64_t nedges, float *gY, float *gR,
                 float *gXe, hipStream_t st) {
  hipLaunchKernelGGL((mp_backward_edge_kernel<C, GY, GR, GX>), dim3(static_cast<unsigned>(nnodes)), dim3(kWave),
                     0, st, X, Y, R, G, sender, first_occ, static_cast<int>(nnodes), nedges, gY, gR, gXe);
}

template <int C>
int launch_backward(const float *X, const float *Y, const float *R, const float *G, const int32_t *sender,
                    const int32_t *first_occ, const int32_t *perm, const int32_t *offsets, int64_t nnodes,
                    int64_t nedges, float *gX, float *gY, float *gR, float *gXe, hipStream_t st) {
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
  int rc = check_launch("cm_mp_backward (edge pass)");
  if (rc != CM_OK) return rc;
  if (gX) rc = mp::launch_sender_pass(C, gXe, perm, offsets, nnodes, nedges, gX, st);
  return rc;
}

template <int C>
int launch_sender(const float *gXe, const int32_t *perm, const int32_t *offsets, int64_t nnodes, int64_t nedges,
                  float *gX, hipStream_t st) {
  hipLaunchKernelGGL(mp_backward_sender_kernel<C>, dim3(static_cast<unsigned>(nnodes)), dim3(kWave), 0, st, gXe, perm,
                     offsets, static_cast<int>(nnodes), nedges, gX);
  return check_launch("cm_mp_backward (sender pass)");
}

}  // namespace

int mp::launch_sender_pass(int channels, const float *gXe, const int32_t *perm, const int32_t *offsets, int64_t nnodes,
                           int64_t nedges, float *gX, hipStream_t st) {
  int rc = CM_EINVAL;
  CM_DISPATCH_C(channels, rc = launch_sender<C_>(gXe, perm, offsets, nnodes, nedges, gX, st));
  return rc;
}

}  // namespace cm

extern "C" int cm_channels_supported(int channels) {
  return channels >= 32 && channels <= 256 && channels % 32 == 0;
}

extern "C" int cm_first_occurences(const int32_t *receiver, int64_t nedges, int64_t nnodes,
                                   int32_t *first_occ, cm_stream_t stream) {
  CM_REQUIRE(nedges >= 0 && nnodes >= 0, "cm_first_occurences: negative size");
  CM_REQUIRE(nedges < INT32_MAX && nnodes < INT32_MAX / 2, "cm_first_occurences: sizes exceed int32 indexing");
  if (nnodes == 0) return CM_OK;
  CM_REQUIRE(first_occ != nullptr, "cm_first_occurences: first_occ is NULL");
  CM_REQUIRE(nedges == 0 || receiver != nullptr, "cm_first_occurences: receiver is NULL");
  const int block = 256;
  const int64_t work = nedges > 0 ? nedges : nnodes;
  const unsigned grid = static_cast<unsigned>(nedges > 0 ? cm::ceil_div(work, block) : std::min<int64_t>(cm::ceil_div(work, block), 1024));
  hipLaunchKernelGGL(cm::first_occurences_kernel, dim3(grid), dim3(block), 0, cm::as_stream(stream), receiver,
                     static_cast<int>(nedges), static_cast<int>(nnodes), first_occ);
  return cm::check_launch("cm_first_occurences");
}

extern "C" int cm_mp_forward(const float *X, const float *Y, const float *R, const int32_t *sender,
                             const int32_t *first_occ, int64_t nnodes, int64_t nedges, int channels,
                             float *out, cm_stream_t stream) {
  CM_REQUIRE(cm_channels_supported(channels), "cm_mp_forward: channels=%d must be a multiple of 32 in [32, 256]", channels);
  CM_REQUIRE(nedges >= 0 && nnodes >= 0, "cm_mp_forward: negative size");
  CM_REQUIRE(nedges < INT32_MAX && nnodes < INT32_MAX / 2, "cm_mp_forward: sizes exceed int32 indexing");
  if (nnodes == 0) return CM_OK;
  CM_REQUIRE(X && first_occ && out, "cm_mp_forward: NULL pointer");
  CM_REQUIRE(nedges == 0 || (Y && R && sender), "cm_mp_forward: NULL edge operand");
  int rc = CM_EINVAL;
  CM_DISPATCH_C(channels, rc = cm::launch_forward<C_>(X, Y, R, sender, first_occ, nnodes, nedges, out, cm::as_stream(stream)));
  return rc;
}

extern "C" int cm_mp_backward(const float *X, const float *Y, const float *R, const float *grad_out,
                              const int32_t *sender, const int32_t *first_occ, const int32_t *sender_perm,
                              const int32_t *sender_offsets, int64_t nnodes, int64_t nedges, int channels,
                              float *gX, float *gY, float *gR, float *edge_scratch, cm_stream_t stream) {
  CM_REQUIRE(cm_channels_supported(channels), "cm_mp_backward: channels=%d must be a multiple of 32 in [32, 256]", channels);
  CM_REQUIRE(nedges >= 0 && nnodes >= 0, "cm_mp_backward: negative size");
  CM_REQUIRE(nedges < INT32_MAX && nnodes < INT32_MAX / 2, "cm_mp_backward: sizes exceed int32 indexing");
  if (nnodes == 0) return CM_OK;
  CM_REQUIRE(X && grad_out && first_occ, "cm_mp_backward: NULL pointer");
  CM_REQUIRE(nedges == 0 || (Y && R && sender), "cm_mp_backward: NULL edge operand");
  CM_REQUIRE(!gX || (sender_offsets && (nedges == 0 || (sender_perm && edge_scratch))),
             "cm_mp_backward: gX wanted but sender_perm / sender_offsets / edge_scratch missing");
  int rc = CM_EINVAL;
  CM_DISPATCH_C(channels, rc = cm::launch_backward<C_>(X, Y, R, grad_out, sender, first_occ, sender_perm, sender_offsets, nnodes,
                                                       nedges, gX, gY, gR, edge_scratch, cm::as_stream(stream)));
  return rc;
}
