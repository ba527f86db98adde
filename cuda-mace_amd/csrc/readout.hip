// Readouts of the two-layer invariant model and their derivative, one pass.
//
// The reference keeps upstream's readout modules in fp64 and feeds them the fp32 node features cast to double
// (models/InvariantMACE.py:196, 330-337, 343): a linear readout of the first layer's features, a one-hidden-layer
// readout (normalised silu gate) of the second layer's, then scale and shift.  Per step that is a dozen small fp64
// GEMM and element-wise launches forward and as many backward.  Here one kernel does all of it per node in fp64:
//
//   e[n]   = scale * ( h1[n] . w1  +  sum_j w2b[j] * act(z_j) ) + shift,      z = h2[n] . W2a,   act(z) = cst * z * sigmoid(z)
//   d2[n,c] = scale * sum_j W2a[c, j] * w2b[j] * act'(z_j)                     (= d e[n] / d h2[n, c], stored in fp32)
//   d e[n] / d h1[n, c] = scale * w1[c]                                        (constant, not stored)
//
// and, on request, the [N, 2C] fp64 concatenation of the features that the model returns as "node_feats" (row n
// optionally written to row feats_rows[n], for callers that keep their nodes in another order internally) and the
// node's total energy e[n] + e0[n] (e0: a given constant per node, e.g. the atomic reference energy), written to the same
// row.  The backward is then a scaling of those derivatives by the incoming gradient of e[n].
//
// Work split: a workgroup of 256 threads keeps W2a and w1 in LDS and walks tiles of 16 nodes; a tile's rows of both
// feature arrays are staged in LDS with coalesced 16-byte loads; thread (node, j) accumulates z_j over the channels,
// 16-lane shuffles reduce over j.
#include <cmath>

#include "common.hpp"
#include "readout.hpp"

namespace cm {
namespace {

constexpr int kNodes = 16;    // nodes per workgroup
constexpr int kHidden = 16;   // threads per node = largest hidden width handled
constexpr int kMaxC = 256;
constexpr int kLdW = kMaxC + 2;   // row stride (doubles) of W2a transposed, [hidden][channel]: rows j and j + 1 start 4 banks apart,
                                  // so the 16 hidden units of a node read their 16-byte pieces without conflicts
constexpr int kMaxGroups = 512;   // workgroups of a forward launch
constexpr int kLdS = kMaxC + 4;   // row stride (floats) of a feature tile: 16-byte aligned rows, the four nodes of a wave 4 banks apart
typedef double d2v __attribute__((ext_vector_type(2)));

__global__ __launch_bounds__(kNodes *kHidden) void readout_forward_kernel(
    const float *__restrict__ h1, const float *__restrict__ h2, const double *__restrict__ w1, const double *__restrict__ W2a,
    const double *__restrict__ w2b, double act_cst, double scale, double shift, int nnodes, int C, int H,
    double *__restrict__ node_es, float *__restrict__ d2, double *__restrict__ feats64,
    const int32_t *__restrict__ feats_rows, const double *__restrict__ node_e0, double *__restrict__ node_total) {
  __shared__ __attribute__((aligned(16))) double sW[kHidden * kLdW];  // W2a transposed [16, C]; rows beyond H are zero
  __shared__ double sw1[kMaxC];
  __shared__ __attribute__((aligned(16))) float s1[kNodes * kLdS];
  __shared__ __attribute__((aligned(16))) float s2[kNodes * kLdS];
  __shared__ double sD[kNodes * kHidden];  // w2b[j] * act'(z_j) per node
  const int t = threadIdx.x;
  // a workgroup stages the weights once and then walks tiles of 16 nodes; the rows of its next tile are requested
  // before the current one is worked on (one element per trip, each waited for, would cost a memory latency per trip)
  const int ntiles = (nnodes + kNodes - 1) / kNodes;
  constexpr int kTrips = kNodes * kMaxC / 4 / (kNodes * kHidden);  // 16-byte pieces per thread at the widest C
  const bool wide = C % 4 == 0;
  f4 a[kTrips], b[kTrips];
  auto request = [&](int tile) {
    const int node0 = tile * kNodes;
    const int n4 = min(kNodes, nnodes - node0) * C / 4;
    const float *p1 = h1 + static_cast<int64_t>(node0) * C, *p2 = h2 + static_cast<int64_t>(node0) * C;
#pragma unroll
    for (int u = 0; u < kTrips; ++u) {
      const int q = t + u * (kNodes * kHidden);
      a[u] = q < n4 ? ld4(p1 + 4 * q) : zero4();
      b[u] = q < n4 ? ld4(p2 + 4 * q) : zero4();
    }
  };
  if (wide && static_cast<int>(blockIdx.x) < ntiles) request(blockIdx.x);
  {
    // the weights: every element this thread stages is requested before the first is stored (one trip after the other,
    // each waiting for its load, is a memory latency per trip -- most of the launch for a few hundred nodes)
    constexpr int kWTrips = kMaxC * kHidden / (kNodes * kHidden);
    double wv[kWTrips];
#pragma unroll
    for (int u = 0; u < kWTrips; ++u) {
      const int i = t + u * (kNodes * kHidden);
      const int c = i / kHidden, j = i % kHidden;
      wv[u] = (c < C && j < H) ? W2a[c * H + j] : 0.0;
    }
    const double w1v = t < C ? w1[t] : 0.0;
#pragma unroll
    for (int u = 0; u < kWTrips; ++u) {
      const int i = t + u * (kNodes * kHidden);
      if (i < C * kHidden) sW[(i % kHidden) * kLdW + i / kHidden] = wv[u];
    }
    if (t < C) sw1[t] = w1v;
  }
  for (int tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
    const int node0 = tile * kNodes;
    const int rows = min(kNodes, nnodes - node0);
    __syncthreads();  // the previous tile's rows and sD have been read (and, before the first tile, the weights are written)
    // the tile's rows of both feature arrays -> LDS (and, on request, -> the fp64 concatenation)
    if (wide) {
      const int n4 = rows * C / 4;
#pragma unroll
      for (int u = 0; u < kTrips; ++u) {
        const int q = t + u * (kNodes * kHidden);
        if (q < n4) {
          const int r = 4 * q / C, c = 4 * q % C;
          *reinterpret_cast<f4 *>(s1 + r * kLdS + c) = a[u];
          *reinterpret_cast<f4 *>(s2 + r * kLdS + c) = b[u];
          if (feats64) {
            const int row = feats_rows ? feats_rows[node0 + r] : node0 + r;
            if (static_cast<unsigned>(row) < static_cast<unsigned>(nnodes)) {
              double *f = feats64 + static_cast<int64_t>(row) * (2 * C) + c;
#pragma unroll
              for (int k = 0; k < 4; ++k) {
                f[k] = a[u][k];
                f[C + k] = b[u][k];
              }
            }
          }
        }
      }
      if (tile + static_cast<int>(gridDim.x) < ntiles) request(tile + gridDim.x);
    } else {
      for (int i = t; i < rows * C; i += blockDim.x) {
        const int r = i / C, c = i % C;
        const float av = h1[static_cast<int64_t>(node0 + r) * C + c];
        const float bv = h2[static_cast<int64_t>(node0 + r) * C + c];
        s1[r * kLdS + c] = av;
        s2[r * kLdS + c] = bv;
        if (feats64) {
          const int row = feats_rows ? feats_rows[node0 + r] : node0 + r;
          if (static_cast<unsigned>(row) < static_cast<unsigned>(nnodes)) {
            feats64[static_cast<int64_t>(row) * (2 * C) + c] = av;
            feats64[static_cast<int64_t>(row) * (2 * C) + C + c] = bv;
          }
        }
      }
    }
    __syncthreads();
    const int r = t / kHidden, j = t % kHidden;
    const bool live = r < rows;
    // first readout: each of the node's 16 threads takes every 16th channel
    double e1 = 0.0, z = 0.0;
    if (live) {
      const float *row1 = s1 + r * kLdS;
      for (int c = j; c < C; c += kHidden) e1 += static_cast<double>(row1[c]) * sw1[c];
      // four independent partial sums (channels c = 0, 1, 2, 3 modulo 4): the fp64 multiply-add chain is otherwise as long
      // as the channel count.  Four channels per trip: one 16-byte read of the node's row, two of the weight row.
      double z0 = 0.0, z1 = 0.0, z2 = 0.0, z3 = 0.0;
      const float *srow = s2 + r * kLdS;
      const double *wrow = sW + j * kLdW;
      int c = 0;
      if (wide) {
#pragma unroll 2
        for (; c + 3 < C; c += 4) {
          const f4 x = *reinterpret_cast<const f4 *>(srow + c);
          const d2v w01 = *reinterpret_cast<const d2v *>(wrow + c), w23 = *reinterpret_cast<const d2v *>(wrow + c + 2);
          z0 += static_cast<double>(x.x) * w01.x;
          z1 += static_cast<double>(x.y) * w01.y;
          z2 += static_cast<double>(x.z) * w23.x;
          z3 += static_cast<double>(x.w) * w23.y;
        }
      } else {
        for (; c + 3 < C; c += 4) {
          z0 += static_cast<double>(srow[c]) * wrow[c];
          z1 += static_cast<double>(srow[c + 1]) * wrow[c + 1];
          z2 += static_cast<double>(srow[c + 2]) * wrow[c + 2];
          z3 += static_cast<double>(srow[c + 3]) * wrow[c + 3];
        }
      }
      for (; c < C; ++c) z0 += static_cast<double>(srow[c]) * wrow[c];
      z = (z0 + z1) + (z2 + z3);
    }
    double e2 = 0.0, dj = 0.0;
    if (live && j < H) {
      const double sig = 1.0 / (1.0 + exp(-z));
      e2 = w2b[j] * act_cst * z * sig;
      dj = w2b[j] * act_cst * (sig + z * sig * (1.0 - sig));
    }
    sD[t] = dj;
    double e = e1 + e2;
#pragma unroll
    for (int off = kHidden / 2; off > 0; off >>= 1) e += __shfl_xor(e, off);
    if (live && j == 0) {
      const double en = scale * e + shift;
      node_es[node0 + r] = en;
      if (node_total) {
        const int row = feats_rows ? feats_rows[node0 + r] : node0 + r;
        if (static_cast<unsigned>(row) < static_cast<unsigned>(nnodes)) node_total[row] = en + (node_e0 ? node_e0[node0 + r] : 0.0);
      }
    }
    __syncthreads();
    // d e / d h2: a thread keeps the 16 weights of its channel in registers and serves a share of the tile's rows
    // (256 / C row groups; the rows' 16 factors are read by all lanes of a group at once)
    const int groups = kNodes * kHidden / C;  // at least 1: C <= 256 = threads of the workgroup
    const int per = (kNodes + groups - 1) / groups;
    const int c = t % C, grp = t / C;
    if (grp < groups) {
      double wq[kHidden];
#pragma unroll
      for (int q = 0; q < kHidden; ++q) wq[q] = sW[q * kLdW + c];
      const int r1 = min(rows, (grp + 1) * per);
      for (int rr = grp * per; rr < r1; ++rr) {
        double acc = 0.0;
#pragma unroll
        for (int q = 0; q < kHidden; ++q) acc += wq[q] * sD[rr * kHidden + q];
        d2[static_cast<int64_t>(node0 + rr) * C + c] = static_cast<float>(scale * acc);
      }
    }
  }
}

__global__ void readout_backward_kernel(const double *__restrict__ g, const double *__restrict__ w1, const float *__restrict__ d2,
                                        double scale, int64_t total, int C, float *__restrict__ g1, float *__restrict__ g2) {
  const int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  if (i >= total) return;
  const double gn = g[i / C];
  if (g1) g1[i] = static_cast<float>(gn * scale * w1[i % C]);
  if (g2) g2[i] = static_cast<float>(gn * static_cast<double>(d2[i]));
}

}  // namespace
}  // namespace cm

namespace cm {

int readout_forward_with_totals(const float *h1, const float *h2, const double *w1, const double *W2a, const double *w2b,
                                double act_cst, double scale, double shift, int64_t nnodes, int channels, int hidden,
                                double *node_energies, float *d_h2, double *node_feats64, const int32_t *rows,
                                const double *node_e0, double *node_total, hipStream_t st) {
  CM_REQUIRE(channels >= 1 && channels <= kMaxC, "cm_readout_forward: channels=%d must be in [1, %d]", channels, kMaxC);
  CM_REQUIRE(hidden >= 1 && hidden <= kHidden, "cm_readout_forward: hidden=%d must be in [1, %d]", hidden, kHidden);
  CM_REQUIRE(nnodes >= 0 && nnodes < INT32_MAX / 2, "cm_readout_forward: nnodes out of range");
  if (nnodes == 0) return CM_OK;
  CM_REQUIRE(h1 && h2 && w1 && W2a && w2b && node_energies && d_h2, "cm_readout_forward: NULL pointer");
  // at most kMaxGroups workgroups (two per compute unit of a 256-unit device fit by their LDS): each stages the
  // weights once and walks several tiles
  const int64_t tiles = ceil_div(nnodes, kNodes);
  hipLaunchKernelGGL(readout_forward_kernel, dim3(static_cast<unsigned>(tiles < kMaxGroups ? tiles : kMaxGroups)),
                     dim3(kNodes * kHidden), 0, st, h1, h2, w1, W2a, w2b, act_cst, scale, shift, static_cast<int>(nnodes), channels,
                     hidden, node_energies, d_h2, node_feats64, rows, node_e0, node_total);
  return check_launch("cm_readout_forward");
}

}  // namespace cm

extern "C" int cm_readout_forward(const float *h1, const float *h2, const double *w1, const double *W2a, const double *w2b,
                                  double act_cst, double scale, double shift, int64_t nnodes, int channels, int hidden,
                                  double *node_energies, float *d_h2, double *node_feats64, const int32_t *feats_rows,
                                  cm_stream_t stream) {
  return cm::readout_forward_with_totals(h1, h2, w1, W2a, w2b, act_cst, scale, shift, nnodes, channels, hidden, node_energies, d_h2,
                                         node_feats64, feats_rows, nullptr, nullptr, cm::as_stream(stream));
}

extern "C" int cm_readout_backward(const double *grad_node_energies, const double *w1, const float *d_h2, double scale,
                                   int64_t nnodes, int channels, float *grad_h1, float *grad_h2, cm_stream_t stream) {
  CM_REQUIRE(channels >= 1 && channels <= cm::kMaxC, "cm_readout_backward: channels=%d must be in [1, %d]", channels, cm::kMaxC);
  CM_REQUIRE(nnodes >= 0 && nnodes < INT32_MAX / 2, "cm_readout_backward: nnodes out of range");
  if (nnodes == 0 || (!grad_h1 && !grad_h2)) return CM_OK;
  CM_REQUIRE(grad_node_energies && w1 && d_h2, "cm_readout_backward: NULL pointer");
  const int64_t total = nnodes * channels;
  hipLaunchKernelGGL(cm::readout_backward_kernel, dim3(static_cast<unsigned>(cm::ceil_div(total, 256))), dim3(256), 0,
                     cm::as_stream(stream), grad_node_energies, w1, d_h2, scale, total, channels, grad_h1, grad_h2);
  return cm::check_launch("cm_readout_backward");
}
