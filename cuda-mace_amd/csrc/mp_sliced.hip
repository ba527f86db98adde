// Forward message passing from edge vectors with the radial table in LDS.
//
//   out[n, m, c] = sum_{e -> n} X[sender[e], c] * Y_m(vec[e]) * R(|vec[e]|)[l(m), c]
//
// The kernels in mp_spline.hip give a wave one receiver node and all 16 components; per edge a lane fetches its 16
// coefficient pieces of the cubic (8 KB per edge over the wave) from the table in L2, and that delivery is what bounds
// them.  Here the work is cut the other way: a workgroup owns two degrees, (0, 3) or (1, 2) -- eight components either
// way, so every workgroup has the same work per edge -- and one slice of 16 channels, and the part of the table it
// needs, (nknots - 1) x 4 coefficients x 2 degrees x 16 channels = 130 KB at 256 knots, stays in its LDS for the whole
// launch.  One workgroup per compute unit; the workgroups of a (pair, slice) split the node range evenly.
//
// Inside a workgroup a quad of four lanes serves one receiver node, four channels per lane, so a wave works on 16 nodes
// at once.  Edges are taken four at a time: lane k of the quad loads edge k of the block, computes its length, knot
// interval, offset and the eight harmonics, and in step j of the block the whole quad handles edge j: the X row piece of
// its sender is one contiguous 64 bytes over the quad.  The edge's values reach the other lanes once per block: the
// offset inside the interval and the eight harmonics of the block's four edges are gathered over the quad by one matrix
// instruction each (quad_gather below), after which every lane holds them for all four steps in plain registers; the two
// byte offsets of an edge (table row, X row) come from lane j through a quad permutation of the DPP operand of the
// address addition, once per step.
//
// LDS layout of the table slice: interval idx at 512 idx bytes; inside it the (a, b, c, d) of degree li (0 / 1: first /
// second of the pair), channel 4 k + 2 p + b of the slice at 256 li + 64 (p + 2 b) + 16 k: the four lanes of a quad read
// 64 contiguous bytes.  A 16-byte LDS read is served 16 lanes, i.e. four quads with unrelated intervals, at a time, and
// the row stride is a multiple of the bank span, so quads that read the same piece position collide.  Which channel a
// register stands for is a matter of addresses only (which 8 bytes of the X row land in it, which pieces are read for
// it, where its sums are stored), so the quads at odd places take their two channel pairs in the other order: an odd
// and an even quad never touch the same banks, two even (or two odd) ones do (a two-way conflict; avoiding it as well
// would need X loads of four bytes).
//
// Everything a step needs from memory is requested ahead, with registers that rotate in three sets so that nothing that
// a load is still on its way into ever has to be copied (a copy would wait for the load): the sender and vector of a
// lane's edge three blocks ahead, the X pieces two blocks ahead (what is in flight per compute unit, against the
// latency of L2 under this load, sets the rate of the X gather), the table pieces of the next step while the current
// one accumulates.  The instruction scheduler, left to itself, moves each request down to the end of the block (it
// shortens the life of the landing registers); scheduling barriers keep every request in its step.
//
// Receiver nodes differ in their edge counts and the 16 nodes of a wave advance together, so a workgroup sorts its nodes
// (4 096 at a time) by their number of edge blocks and its waves draw 16 neighbours of that order at a time from a
// counter in LDS.  Which wave serves a node does not change the node's result: a node's sum runs over its edges in
// list order.
#include <algorithm>
#include <type_traits>

#include "mp_common.hpp"
#include "sh_device.hpp"

namespace cm {
namespace mp {
namespace {

constexpr int kSlThreads = 512;       // two waves per SIMD (three: 168 registers, equal at 25 000 nodes, 8 % slower at 50 000)
constexpr int kSlMaxIntervals = 272;  // 136 KB of table (one row of it is the row of zeros)
constexpr int kSlSub = 4096;          // nodes sorted at a time
constexpr int kSlBins = 64;           // edge blocks per node that the sort tells apart
constexpr int kSlMinNodes = 2048;

struct SlicedArgs {
  const float *X, *vec;
  const int32_t *sender, *first_occ;
  const float *coeffs, *knots;
  int nknots;
  float r_width, r_max;
  int nnodes;
  int64_t nedges;
  int C;
  float *out;
  int nslices;  // C / 16
  int share;    // workgroups per (pair, slice)
};

typedef float f2 __attribute__((ext_vector_type(2)));

// value of `v` in lane J of the reader's quad of four lanes (quad permutation of the DPP operand)
template <int J>
__device__ __forceinline__ unsigned quadu(unsigned v) {
  return static_cast<unsigned>(__builtin_amdgcn_mov_dpp(static_cast<int>(v), J * 0x55, 0xf, 0xf, true));
}

// The value of `v` in each of the four lanes of the reader's quad: element i is lane i's.  One matrix instruction: the
// 4x4x1 form works on 16 independent blocks of four lanes, D_b[i][j] = A_b[i] B_b[j] + C_b[i][j], with A_b[i] taken from
// lane i of the block and row i of D in register i of every lane; B = 1 and C = 0 make it a copy (exact for every
// normal number).  It runs on the matrix pipe, which this kernel does not use otherwise, in place of four moves with a
// DPP operand on the vector pipe, which is the one that bounds the kernel.
__device__ __forceinline__ f4 quad_gather(float v) {
  return __builtin_amdgcn_mfma_f32_4x4x1f32(v, 1.0f, f4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
}

// the two degrees of pair P and their component counts
template <int P>
struct Pair {
  static constexpr int L0 = P == 0 ? 0 : 1, L1 = P == 0 ? 3 : 2;
  static constexpr int M0 = 2 * L0 + 1, M1 = 2 * L1 + 1;
  static_assert(M0 + M1 == 8, "eight components per pair");
  // row of out (component m) that accumulator i stands for
  static constexpr int row(int i) { return i < M0 ? L0 * L0 + i : L1 * L1 + i - M0; }
};

// the eight harmonics of pair P (the unused ones of the full evaluation fall away at compile time)
template <int P>
__device__ __forceinline__ void harmonics(float v0, float v1, float v2, float inv_len, float (&y)[8]) {
  float all[16];
  sh::eval(sh::Direction{v2 * inv_len, v0 * inv_len, v1 * inv_len, inv_len}, all);
#pragma unroll
  for (int i = 0; i < 8; ++i) y[i] = all[Pair<P>::row(i)];
}

// What a lane has prepared for its edge of a block: byte offset of the sender's row in X, byte offset of the knot
// interval in the table slice, offset inside the interval, harmonics.  An edge that does not count (beyond the node's
// range or the cutoff, or with a sender outside the node range) keeps zero harmonics and points at the node's own row
// and at a row of zeros behind the last interval of the table slice.
struct Prepared {
  unsigned xo, io;
  float xr;
  float y[8];
};
// offset inside the interval and harmonics of the four edges of a block, in every lane of the quad
struct Gathered {
  f4 xr;
  f4 y[8];
};
__device__ __forceinline__ Gathered gather(const Prepared &o) {
  Gathered g;
  g.xr = quad_gather(o.xr);
#pragma unroll
  for (int i = 0; i < 8; ++i) g.y[i] = quad_gather(o.y[i]);
  return g;
}
struct Raw {  // what a lane loads for its edge of a block
  int s;
  float v0, v1, v2;
};

// per-lane constants of the channel order (see the head of the file)
struct LaneMap {
  unsigned x[2];    // byte offset inside an X / out row of the lane's two channel pairs, in ITS order
  unsigned lds[2];  // byte offset inside a table row of the piece (first degree, first channel) of each pair
};

// q[4 li + 2 p + b]: (a, b, c, d) of degree li, channel b of the lane's pair p
template <int J>
__device__ __forceinline__ void read_pieces(const char *tab, unsigned io, const LaneMap &m, f4 (&q)[8]) {
  const unsigned row = quadu<J>(io);
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    const char *at = tab + (row + m.lds[p]);
    q[0 + 2 * p + 0] = *reinterpret_cast<const f4 *>(at);
    q[0 + 2 * p + 1] = *reinterpret_cast<const f4 *>(at + 128);
    q[4 + 2 * p + 0] = *reinterpret_cast<const f4 *>(at + 256);
    q[4 + 2 * p + 1] = *reinterpret_cast<const f4 *>(at + 384);
  }
}

template <int J>
__device__ __forceinline__ void request_row(const float *__restrict__ X, unsigned xo, const LaneMap &m, f2 (&x)[2]) {
  const unsigned row = quadu<J>(xo);
  const char *base = reinterpret_cast<const char *>(X);
  x[0] = *reinterpret_cast<const f2 *>(base + (row + m.x[0]));
  x[1] = *reinterpret_cast<const f2 *>(base + (row + m.x[1]));
}

// Steps J .. 3 of a block: `cur` is the block, xin[j] the X values of the edge of step j; as soon as step j has taken
// them, the values of step j of the block after next (`fut`) are requested into xout[j].
template <int P, int J>
__device__ __forceinline__ void edge_step(const float *__restrict__ X, const char *tab, const Prepared &cur, const Gathered &all,
                                          const Prepared &fut, const LaneMap &m, const f2 (&xin)[4][2], f2 (&xout)[4][2],
                                          f4 (&q)[8], float (&acc)[8][4]) {
  const float xs[4] = {xin[J][0].x, xin[J][0].y, xin[J][1].x, xin[J][1].y};
  request_row<J>(X, fut.xo, m, xout[J]);
  const float xr = all.xr[J];
  float y[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) y[i] = all.y[i][J];
  float t[2][4];
#pragma unroll
  for (int li = 0; li < 2; ++li)
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const f4 c = q[4 * li + d];
      t[li][d] = xs[d] * fmaf(xr, fmaf(xr, fmaf(xr, c.w, c.z), c.y), c.x);
    }
  __builtin_amdgcn_sched_barrier(0);
  if constexpr (J + 1 < 4) read_pieces<J + 1>(tab, cur.io, m, q);
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int d = 0; d < 4; ++d) acc[i][d] = fmaf(y[i], t[i < Pair<P>::M0 ? 0 : 1][d], acc[i][d]);
  __builtin_amdgcn_sched_barrier(0);
  if constexpr (J + 1 < 4) edge_step<P, J + 1>(X, tab, cur, all, fut, m, xin, xout, q, acc);
}

// the rounds of one sorted sub-range: nodes lo + order[0 .. cnt)
template <int P>
__device__ __forceinline__ void run_rounds(const SlicedArgs &p, const float *sTab, const float *sKnots,
                                           const unsigned short *sOrder, int *sNext, int lo, int cnt, int slice) {
  const int lane = threadIdx.x % kWave;
  const int k = lane & 3;         // place in the quad: channels 4 k .. 4 k + 3 of the slice
  const int u = (lane >> 2) & 1;  // parity of the quad's place among the four that an LDS access serves together
  const int gw = lane >> 2;       // node of the wave's round
  LaneMap m;
#pragma unroll
  for (int pr = 0; pr < 2; ++pr) {
    m.x[pr] = static_cast<unsigned>(4 * (slice * 16 + 4 * k + 2 * (pr ^ u)));
    m.lds[pr] = static_cast<unsigned>(64 * (pr ^ u) + 16 * k);
  }
  const char *tab = reinterpret_cast<const char *>(sTab);
  const int C = p.C;
  const int last_edge = static_cast<int>(p.nedges) - 1;  // the launcher does not come here without edges
  const unsigned zero_row = static_cast<unsigned>(p.nknots - 1) * 512u;
  const float inv_width = 1.0f / p.r_width;

  for (;;) {
    int base = 0;
    if (lane == 0) base = atomicAdd(sNext, kWave / 4);
    base = __builtin_amdgcn_readfirstlane(base);
    if (base >= cnt) break;
    const int mine = base + gw;
    const int node = mine < cnt ? lo + sOrder[mine] : -1;
    int e0 = 0, e1 = 0;
    if (node >= 0) {
      e0 = p.first_occ[node];
      e1 = p.first_occ[p.nnodes + node];
      clamp_edge_range(e0, e1, p.nedges);
    }
    const int nblk = (e1 - e0 + 3) >> 2;
    const unsigned own_row = static_cast<unsigned>(node >= 0 ? node : 0) * static_cast<unsigned>(4 * C);
    float acc[8][4];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int d = 0; d < 4; ++d) acc[i][d] = 0.f;

    // Unconditional (an edge index beyond the list reads the last edge, and prepare() discards it): loads under a
    // branch would make the later waits cover everything in flight.
    auto request = [&](int blk) {
      const int64_t e = min(e0 + 4 * blk + k, last_edge);
      return Raw{p.sender[e], p.vec[3 * e + 0], p.vec[3 * e + 1], p.vec[3 * e + 2]};
    };
    auto prepare = [&](const Raw &r, int blk) {
      Prepared o;
      const bool valid = e0 + 4 * blk + k < e1;
      // Length and direction from one reciprocal square root (the hardware's, one Newton step: within an ulp) and the
      // interval from a product with 1 / width: the correctly rounded square root and the two divisions they stand for
      // are 40 instructions per edge, and every one of the 16 workgroup types of a piece of the node range prepares
      // every edge.  An edge within rounding of a knot may land in the neighbouring interval, whose cubic continues
      // the spline there (value and two derivatives agree at the knot); one within rounding of the cutoff may be kept
      // or dropped, where the tabulated functions of a model end in zero (their envelope) and a table that does not
      // is cut off at a length that is only known to that rounding anyway.
      const float r2 = fmaf(r.v2, r.v2, fmaf(r.v1, r.v1, r.v0 * r.v0));
      float ir = __builtin_amdgcn_rsqf(r2);
      ir = ir * fmaf(-0.5f * r2 * ir, ir, 1.5f);
      const float len = r2 * ir;  // NaN for a vector of zeros: such an edge does not count
      // without a branch (the interval of an edge that does not count is looked up and dropped): under a branch the
      // knot's way from LDS is waited for on the spot, here it arrives while the harmonics are formed
      int idx = static_cast<int>(len * inv_width);
      idx = idx < 0 ? 0 : (idx > p.nknots - 2 ? p.nknots - 2 : idx);
      const float knot = sKnots[idx];
      const bool live = valid && len <= p.r_max && static_cast<unsigned>(r.s) < static_cast<unsigned>(p.nnodes);
      harmonics<P>(r.v0, r.v1, r.v2, ir, o.y);
#pragma unroll
      for (int i = 0; i < 8; ++i) o.y[i] = live ? o.y[i] : 0.f;
      o.xr = live ? len - knot : 0.f;
      o.xo = live ? __umul24(static_cast<unsigned>(r.s), static_cast<unsigned>(4 * C)) : own_row;  // both below 2^24
      o.io = live ? static_cast<unsigned>(idx) * 512u : zero_row;
      return o;
    };
    auto rows = [&](const Prepared &o, f2 (&x)[4][2]) {
      request_row<0>(p.X, o.xo, m, x[0]);
      request_row<1>(p.X, o.xo, m, x[1]);
      request_row<2>(p.X, o.xo, m, x[2]);
      request_row<3>(p.X, o.xo, m, x[3]);
    };

    // three sets that rotate: block b computes from set b % 3 while the rows of block b + 2 are requested into set
    // (b + 2) % 3 and the raw values of block b + 3 into raw set b % 3
    Raw r0 = request(0), r1 = request(1), r2 = request(2);
    Prepared p0 = prepare(r0, 0), p1 = prepare(r1, 1), p2;
    f2 x0[4][2], x1[4][2], x2[4][2];
    f4 q[8];
    Gathered all;
    rows(p0, x0);
    rows(p1, x1);
    for (int blk = 0;; blk += 3) {
      r0 = request(blk + 3);
      __builtin_amdgcn_sched_barrier(0);
      p2 = prepare(r2, blk + 2);
      read_pieces<0>(tab, p0.io, m, q);
      all = gather(p0);
      __builtin_amdgcn_sched_barrier(0);
      edge_step<P, 0>(p.X, tab, p0, all, p2, m, x0, x2, q, acc);
      if (!__any(blk + 1 < nblk)) break;
      r1 = request(blk + 4);
      __builtin_amdgcn_sched_barrier(0);
      p0 = prepare(r0, blk + 3);
      read_pieces<0>(tab, p1.io, m, q);
      all = gather(p1);
      __builtin_amdgcn_sched_barrier(0);
      edge_step<P, 0>(p.X, tab, p1, all, p0, m, x1, x0, q, acc);
      if (!__any(blk + 2 < nblk)) break;
      r2 = request(blk + 5);
      __builtin_amdgcn_sched_barrier(0);
      p1 = prepare(r1, blk + 4);
      read_pieces<0>(tab, p2.io, m, q);
      all = gather(p2);
      __builtin_amdgcn_sched_barrier(0);
      edge_step<P, 0>(p.X, tab, p2, all, p1, m, x2, x1, q, acc);
      if (!__any(blk + 3 < nblk)) break;
    }

    if (node >= 0) {
      char *op = reinterpret_cast<char *>(p.out + static_cast<int64_t>(node) * 16 * C);
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int pr = 0; pr < 2; ++pr)
          *reinterpret_cast<f2 *>(op + static_cast<int64_t>(Pair<P>::row(i)) * (4 * C) + m.x[pr]) =
              f2{acc[i][2 * pr], acc[i][2 * pr + 1]};
    }
  }
}

__global__ __launch_bounds__(kSlThreads) void mp_edge_forward_sliced_kernel(const SlicedArgs p) {
  __shared__ __attribute__((aligned(16))) float sTab[kSlMaxIntervals * 128];
  __shared__ float sKnots[kSlMaxIntervals + 1];
  __shared__ unsigned short sOrder[kSlSub];
  __shared__ int sHist[kSlBins];
  __shared__ int sNext;

  const int tid = threadIdx.x;
  // Which (pair, slice) and which piece j of the node range.  Consecutive workgroups go to consecutive XCDs (eight of
  // them, each with its own L2): all workgroups of a piece sit on one XCD, so that the edge data and the X rows of the
  // piece are fetched into one L2 only, for as many pieces as divide evenly among the XCDs (all of them at 64, 128 and
  // 256 channels).
  int type, j;
  {
    const int types = 2 * p.nslices;
    const int aligned = (p.share / 8) * 8;  // pieces that go to one XCD each; the others are spread over all of them
    const int b = blockIdx.x;
    if (b < aligned * types) {
      const int xcd = b % 8, q = b / 8;
      type = q % types;
      j = xcd + 8 * (q / types);
    } else {
      const int rest = b - aligned * types;
      type = rest % types;
      j = aligned + rest / types;
    }
  }
  const int slice = type >> 1;
  const int pair = type & 1;
  const int lo = static_cast<int>(static_cast<int64_t>(p.nnodes) * j / p.share);
  const int hi = static_cast<int>(static_cast<int64_t>(p.nnodes) * (j + 1) / p.share);

  // the slice of the table: coeffs[idx][coef][l C + 16 slice + 4 k + 2 pr + b] -> byte 512 idx + 256 li + 64 (pr + 2 b)
  // + 16 k of sTab, (a, b, c, d) together
  const int intervals = p.nknots - 1;
  for (int i = tid; i < intervals * 32; i += kSlThreads) {
    const int idx = i >> 5, coef = (i >> 3) & 3, li = (i >> 2) & 1, k = i & 3;
    const int l = pair == 0 ? (li == 0 ? 0 : 3) : (li == 0 ? 1 : 2);
    const f4 v = ld4(p.coeffs + (static_cast<int64_t>(idx * 4 + coef) * 4 + l) * p.C + slice * 16 + 4 * k);
    float *dst = sTab + idx * 128 + 64 * li + 4 * k + coef;
    dst[0] = v.x;   // pr 0, b 0
    dst[32] = v.y;  // pr 0, b 1
    dst[16] = v.z;  // pr 1, b 0
    dst[48] = v.w;  // pr 1, b 1
  }
  for (int i = tid; i < 128; i += kSlThreads) sTab[intervals * 128 + i] = 0.f;  // the row of edges that do not count
  for (int i = tid; i < p.nknots; i += kSlThreads) sKnots[i] = p.knots[i];

  for (int sub = lo; sub < hi; sub += kSlSub) {
    const int cnt = min(kSlSub, hi - sub);
    __syncthreads();  // every wave has left the previous sub-range (and the table is staged)
    if (tid < kSlBins) sHist[tid] = 0;
    if (tid == 0) sNext = 0;
    __syncthreads();
    // counting sort by the number of edge blocks, most blocks first
    constexpr int kPerThread = (kSlSub + kSlThreads - 1) / kSlThreads;
    int bin[kPerThread];
#pragma unroll
    for (int q = 0; q < kPerThread; ++q) {
      const int i = tid + q * kSlThreads;
      bin[q] = -1;
      if (i < cnt) {
        int e0 = p.first_occ[sub + i], e1 = p.first_occ[p.nnodes + sub + i];
        clamp_edge_range(e0, e1, p.nedges);
        bin[q] = kSlBins - 1 - min((e1 - e0 + 3) >> 2, kSlBins - 1);
        atomicAdd(&sHist[bin[q]], 1);
      }
    }
    __syncthreads();
    if (tid == 0) {
      int run = 0;
      for (int b = 0; b < kSlBins; ++b) {
        const int n = sHist[b];
        sHist[b] = run;
        run += n;
      }
    }
    __syncthreads();
#pragma unroll
    for (int q = 0; q < kPerThread; ++q)
      if (bin[q] >= 0) sOrder[atomicAdd(&sHist[bin[q]], 1)] = static_cast<unsigned short>(tid + q * kSlThreads);
    __syncthreads();
    if (pair == 0)
      run_rounds<0>(p, sTab, sKnots, sOrder, &sNext, sub, cnt, slice);
    else
      run_rounds<1>(p, sTab, sKnots, sOrder, &sNext, sub, cnt, slice);
  }
}

}  // namespace

bool sliced_forward_applies(int64_t nnodes, int channels, int nknots) {
  return nnodes >= kSlMinNodes && nnodes < (1 << 24) && nnodes * channels < (int64_t{1} << 30) && channels % 16 == 0 && nknots >= 2 &&
         nknots - 1 < kSlMaxIntervals && device_compute_units() / (2 * (channels / 16)) >= 2;
}

int launch_sliced_forward(const float *X, const float *vec, const float *knots, const float *coeffs, int nknots, float r_width,
                          float r_max, const int32_t *sender, const int32_t *first_occ, int64_t nnodes, int64_t nedges,
                          int channels, float *out, hipStream_t st) {
  SlicedArgs a{X, vec, sender, first_occ, coeffs, knots, nknots, r_width, r_max, static_cast<int>(nnodes), nedges, channels, out,
               channels / 16, 0};
  a.share = device_compute_units() / (2 * a.nslices);
  hipLaunchKernelGGL(mp_edge_forward_sliced_kernel, dim3(static_cast<unsigned>(a.share * 2 * a.nslices)), dim3(kSlThreads), 0, st, a);
  return check_launch("cm_mp_edge_forward");
}

}  // namespace mp
}  // namespace cm
