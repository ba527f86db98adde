// The per-node arithmetic of the readouts (fp64), shared by the stand-alone readout kernel (readout.hip) and the kernel
// that runs the readouts between the second layer's product linear and its transpose (node_glue.hip), so that both
// return the same bits.  A group of 256 threads serves 16 nodes: thread t = 16 r + j is hidden unit j of node r.
//
//   e[n]    = scale * ( h1[n] . w1  +  sum_j w2b[j] * act(z_j) ) + shift,     z = h2[n] . W2a,   act(z) = cst * z * sigmoid(z)
//   d2[n,c] = scale * sum_j W2a[c, j] * w2b[j] * act'(z_j)
#pragma once

#include <cmath>

#include "common.hpp"

namespace cm {
namespace readout {

constexpr int kNodes = 16;    // nodes per pass of 256 threads
constexpr int kHidden = 16;   // threads per node = largest hidden width handled
constexpr int kMaxC = 256;
constexpr int kLdW = kMaxC + 2;   // row stride (doubles) of W2a transposed, [hidden][channel]: rows j and j + 1 start 4 banks apart,
                                  // so the 16 hidden units of a node read their 16-byte pieces without conflicts
typedef double d2v __attribute__((ext_vector_type(2)));

// W2a [C, H] -> sW [16][ldw] transposed (rows beyond H zero; ldw doubles per row, even, ldw / 2 odd keeps the 16 hidden
// units' 16-byte reads on different banks), w1 -> sw1; all `nthreads` threads of the workgroup
__device__ __forceinline__ void stage_weights(double *sW, double *sw1, const double *__restrict__ W2a, const double *__restrict__ w1,
                                              int C, int H, int t, int nthreads, int ldw = kLdW) {
  for (int i = t; i < C * kHidden; i += nthreads) {
    const int c = i / kHidden, j = i % kHidden;
    sW[j * ldw + c] = j < H ? W2a[c * H + j] : 0.0;
  }
  for (int c = t; c < C; c += nthreads) sw1[c] = w1[c];
}

// Node energy of node r = t / 16 (valid in every lane of the node's 16 after the reduction; the caller stores it from
// lane j == 0 of live nodes) and sD[t] = w2b[j] act'(z_j).  row1 / row2: the node's rows of h1 / h2 in LDS (16-byte
// aligned when wide).
__device__ __forceinline__ double node_energy(int t, bool live, int C, int H, bool wide, const float *row1, const float *srow,
                                              const double *sW, const double *sw1, const double *__restrict__ w2b, double act_cst,
                                              double scale, double shift, double *sD, int ldw = kLdW) {
  const int j = t % kHidden;
  // first readout: each of the node's 16 threads takes every 16th channel
  double e1 = 0.0, z = 0.0;
  if (live) {
    for (int c = j; c < C; c += kHidden) e1 += static_cast<double>(row1[c]) * sw1[c];
    // four independent partial sums (channels c = 0, 1, 2, 3 modulo 4): the fp64 multiply-add chain is otherwise as long
    // as the channel count.  Four channels per trip: one 16-byte read of the node's row, two of the weight row.
    double z0 = 0.0, z1 = 0.0, z2 = 0.0, z3 = 0.0;
    const double *wrow = sW + j * ldw;
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
  return scale * e + shift;
}

// d e / d h2 of the pass's `rows` nodes: a thread keeps the 16 weights of its channel in registers and serves a share
// of the rows (256 / C row groups; the rows' 16 factors are read by all lanes of a group at once).  store(rr, c, value)
// receives the fp32 derivative of row rr, channel c.  Call after a workgroup barrier behind node_energy (sD complete).
template <class Store>
__device__ __forceinline__ void energy_gradient(int t, int rows, int C, const double *sW, const double *sD, double scale, Store store,
                                                int ldw = kLdW) {
  const int groups = kNodes * kHidden / C;  // at least 1: C <= 256 = threads of the pass
  const int per = (kNodes + groups - 1) / groups;
  const int c = t % C, grp = t / C;
  if (grp < groups) {
    double wq[kHidden];
#pragma unroll
    for (int q = 0; q < kHidden; ++q) wq[q] = sW[q * ldw + c];
    const int r1 = min(rows, (grp + 1) * per);
    for (int rr = grp * per; rr < r1; ++rr) {
      double acc = 0.0;
#pragma unroll
      for (int q = 0; q < kHidden; ++q) acc += wq[q] * sD[rr * kHidden + q];
      store(rr, c, static_cast<float>(scale * acc));
    }
  }
}

}  // namespace readout
}  // namespace cm
