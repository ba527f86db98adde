// Invariant message passing with the radial weights evaluated inside the kernels from the cubic-spline
// table, so that R[E, 4, C], its derivative and grad_R never exist in HBM.
//
//   out[n, m, c] = sum_{e -> n} X[sender[e], c] * Y[m, e] * R(r[e])[l(m), c],
//   R(r)[j] = a + b x + c x^2 + d x^3,  (a, b, c, d) = coeffs[idx, :, j],  x = r - r_knots[idx]
//
// Same decomposition as the tabulated-radial kernels (one wave per receiver node, lane = 4 channels,
// node-resident accumulators / gradients in registers, Y and sender staged in LDS); the per-edge knot
// interval and offset are staged next to them.  The coefficient table (2 MB at C = 128) lives in L2:
// per edge and l a lane reads its four 16-byte coefficient pieces, evaluates R_l (and dR_l/dr in the
// backward) and drops them, so only 16 registers of radial data are live at a time.  The backward
// returns the gradient with respect to the edge length directly:
//   g_r[e] = sum_{l, c} X[s, c] * q_l[c] * dR_l/dr[c],   q_l = sum_{m in l} Y[m, e] * grad_out[n, m, c].
//
// The FROM_VEC variants go one step further and take the fp32 edge vectors instead of Y and r: the 16 harmonics and the
// length are computed per edge while the chunk is staged, and the backward turns the reduced gY and g_r of an edge
// straight into the gradient with respect to its vector (harmonics Jacobian + radial part), so Y[16, E], grad_Y and
// grad_r never exist either.  From 2 048 receiver nodes on the forward from edge vectors runs on the kernel of
// mp_sliced.hip, which keeps a workgroup's part of the table in LDS (same arithmetic per edge, sums in list order).
#include <type_traits>

#include "mp_common.hpp"
#include "sh_device.hpp"

// waves per SIMD the register allocator must leave room for.  The backward edge pass runs with a rotated edge loop (the
// next edge's loads are requested before the current edge's reductions), which needs the registers of two waves per SIMD.
#ifndef CM_FUSED_FWD_WAVES
#define CM_FUSED_FWD_WAVES 3
#endif
#ifndef CM_FUSED_BWD_WAVES
#define CM_FUSED_BWD_WAVES 2
#endif

namespace cm {
namespace {

using namespace mp;

struct Spline {
  const float *vec;     // [E, 3] edge vectors (FROM_VEC variants; then r is unused)
  const float *r;       // [E]
  const float *knots;   // [nknots]
  const float *coeffs;  // [nknots - 1, 4, 4C]
  int nknots;
  float r_width;
  float r_max;
};

// Knot interval (or -1 beyond the cutoff) and offset inside it for one edge length.  lds_knots: a copy of the knots in LDS,
// read instead of the one in memory if use_lds.
__device__ __forceinline__ void locate(const Spline &sp, float re, int &idx, float &x, const float *lds_knots = nullptr,
                                       bool use_lds = false) {
  idx = -1;
  x = 0.f;
  if (re <= sp.r_max) {
    idx = static_cast<int>(re / sp.r_width);
    idx = idx < 0 ? 0 : (idx > sp.nknots - 2 ? sp.nknots - 2 : idx);
    // The markers keep each read and its use inside its branch: merged, the two become one read through a generic
    // address, or one subtraction behind a wait for the read of memory, on the path that reads LDS as well.
    if (use_lds) {
      x = re - lds_knots[idx];
      asm volatile("; offset from the knot in LDS" : "+v"(x));
    } else {
      x = re - sp.knots[idx];
      asm volatile("; offset from the knot in memory" : "+v"(x));
    }
  }
}

// Stages up to kChunk LIVE edges of a node -- those inside the cutoff whose sender index is valid -- densely, in their
// original order: sender, Y (as [edge][16]), knot interval, offset inside it, and the position of the edge counted from
// `first` (the value of `base` on entry).  Raw edges are read kChunk at a time until kChunk live ones are staged or the
// node's edges are used up, so a neighbour list with a skin (a quarter of its pairs beyond the cutoff) fills the chunk
// all the same, and the edges beyond the cutoff cost nothing after this point.  `base` advances past every raw edge that
// was consumed; `dead(pass_base, consumed, live_mask, lane_is_dead)` is called once per pass for the consumed edges that
// are not live (the backward writes their zeros there).  Returns the number of staged edges (the same in every lane).
// FROM_VEC: Y and the length come from the edge vector; otherwise from the Y and r arrays.
// `ahead` (AHEAD, FROM_VEC only): sender and vector of edge base + lane, which the caller asked for before it
// called (so that loads it issued in between do not stand in front of them in the queue); used by the first pass.
struct RawEdge {
  int s;
  float v0, v1, v2;
};
template <bool FROM_VEC, bool AHEAD = false, class DeadFn>
__device__ __forceinline__ int stage_edges(const float *__restrict__ Y, const int32_t *__restrict__ sender, const Spline &sp,
                                           int nnodes, int64_t nedges, int &base, int e1, int lane, float *sY, int *sS,
                                           int *sIdx, float *sXr, int *sOrig, DeadFn dead,
                                           RawEdge ahead = RawEdge{-1, 0.f, 0.f, 0.f}, const float *lds_knots = nullptr,
                                           bool use_lds_knots = false) {
  static_assert(FROM_VEC || !AHEAD, "raw edges are handed in for the edge-vector variant only");
  const int first = base;
  int nlive = 0;
  // one pass over up to kChunk raw edges; the first one is written out on its own where its raw edges are handed in, so
  // that its waits are not those of a pass that has just issued its loads
  auto pass = [&](auto use_ahead) {
    const int cnt = min(kChunk, e1 - base);
    int s = -1, idx = -1;
    float x = 0.f;
    float y[16];
#pragma unroll
    for (int m = 0; m < 16; ++m) y[m] = 0.f;
    if (lane < cnt) {
      const int64_t e = base + lane;
      if constexpr (FROM_VEC) {
        float v0, v1, v2;
        if constexpr (decltype(use_ahead)::value) {
          s = ahead.s, v0 = ahead.v0, v1 = ahead.v1, v2 = ahead.v2;
        } else {
          s = sender[e], v0 = sp.vec[3 * e + 0], v1 = sp.vec[3 * e + 1], v2 = sp.vec[3 * e + 2];
        }
        locate(sp, edge_length(v0, v1, v2), idx, x, lds_knots, use_lds_knots);
        sh::eval(sh::direction(v0, v1, v2), y);
      } else {
        s = sender[e];
        locate(sp, sp.r[e], idx, x, lds_knots, use_lds_knots);
#pragma unroll
        for (int m = 0; m < 16; ++m) y[m] = Y[m * nedges + e];
      }
    }
    const bool live = lane < cnt && idx >= 0 && static_cast<unsigned>(s) < static_cast<unsigned>(nnodes);
    const unsigned long long live_mask = __ballot(live);
    const int pos = nlive + __popcll(live_mask & ((1ull << lane) - 1ull));
    const int nlive_pass = __popcll(live_mask);
    // raw edges consumed by this pass: all of them, or those up to the live edge that fills the last place
    int consumed = cnt;
    if (nlive + nlive_pass > kChunk) consumed = __ffsll(static_cast<long long>(__ballot(live && pos == kChunk - 1)));
    if (live && pos < kChunk) {
      sS[pos] = s;
      sIdx[pos] = idx;
      sXr[pos] = x;
      sOrig[pos] = base - first + lane;
#pragma unroll
      for (int q = 0; q < 4; ++q)
        *reinterpret_cast<f4 *>(sY + pos * 16 + 4 * q) = f4{y[4 * q], y[4 * q + 1], y[4 * q + 2], y[4 * q + 3]};
    }
    dead(base, consumed, live_mask, lane < consumed && !live);
    nlive = min(kChunk, nlive + nlive_pass);
    base += consumed;
  };
  if constexpr (AHEAD) {
    if (base < e1) pass(std::true_type{});
  }
  while (nlive < kChunk && base < e1) pass(std::false_type{});
  return nlive;
}

constexpr int kKnotsInLds = 512;  // knots the backward edge pass keeps in LDS (more are read from memory)

// LDS of one wave's staged chunk: Y [kChunk][16], sender, knot interval, offset in it, position (floats / ints)
constexpr int kStageBytes = kChunk * 64 + 4 * kChunk * 4;

template <int L>
struct MRange {
  static constexpr int lo = L * L;
  static constexpr int hi = (L + 1) * (L + 1);
};

// -----------------------------------------------------------------------------------------------
// forward
// -----------------------------------------------------------------------------------------------
// MULTI: a workgroup of up to eight waves per node, each on a part of the node's edge range (launched for few nodes)
template <int C, bool FROM_VEC, bool MULTI>
__global__ __launch_bounds__(MULTI ? 8 * kWave : kWave, (MULTI || Cfg<C, true>::V > 5 ? 2 : CM_FUSED_FWD_WAVES)) void mp_spline_forward_kernel(const float *__restrict__ X,
                                                                 const float *__restrict__ Y, Spline sp,
                                                                 const int32_t *__restrict__ sender,
                                                                 const int32_t *__restrict__ first_occ, int nnodes,
                                                                 int64_t nedges, float *__restrict__ out) {
  using K = Cfg<C, true>;
  using vec = typename K::vec;
  // A workgroup is one wave per part of the node's edge range (MULTI; otherwise one wave and one part: see parts_for).
  // Every wave stages its own edges in its own piece of LDS; the waves meet once, at the end.
  extern __shared__ __attribute__((aligned(16))) unsigned char dyn_lds[];
  const int wave = MULTI ? threadIdx.x / kWave : 0;
  const int parts = MULTI ? blockDim.x / kWave : 1;
  unsigned char *mine = dyn_lds + wave * kStageBytes;
  float *sY = reinterpret_cast<float *>(mine);
  int *sS = reinterpret_cast<int *>(mine + kChunk * 64);
  int *sIdx = sS + kChunk;
  float *sXr = reinterpret_cast<float *>(sIdx + kChunk);
  int *sOrig = reinterpret_cast<int *>(sXr + kChunk);

  const int node = blockIdx.x;
  const int lane = threadIdx.x % kWave;
  const int slot = lane / K::SW;
  const int cl = lane % K::SW;
  const bool active = cl < K::LPE;
  int e0 = first_occ[node];
  int e1 = first_occ[nnodes + node];
  clamp_edge_range(e0, e1, nedges);
  if (parts > 1) {
    const int64_t len = e1 - e0;
    const int lo = e0 + static_cast<int>(len * wave / parts);
    e1 = e0 + static_cast<int>(len * (wave + 1) / parts);
    e0 = lo;
  }

  vec acc[16];
#pragma unroll
  for (int m = 0; m < 16; ++m) acc[m] = zerov<vec>();

  for (int base = e0; base < e1;) {
    wave_lds_fence();  // the staged edges belong to this wave alone
    const int nlive = stage_edges<FROM_VEC>(Y, sender, sp, nnodes, nedges, base, e1, lane, sY, sS, sIdx, sXr, sOrig,
                                            [](int, int, unsigned long long, bool) {});
    wave_lds_fence();
    if (active) {
      // what one edge brings in: the sender's row piece, the 16 coefficient pieces of its knot interval, its harmonics
      struct Edge {
        vec x, coef[16];
        float y[16], xr;
      };
      auto fetch = [&](int j, Edge &e) {
        const int s = sS[j];
        const int idx = sIdx[j];
        e.xr = sXr[j];
        e.x = K::ld(X + (static_cast<unsigned>(s) * C + unsigned(K::off(cl))));
        const f4 *yp = reinterpret_cast<const f4 *>(sY + j * 16);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const f4 v = yp[q];
          e.y[4 * q] = v.x, e.y[4 * q + 1] = v.y, e.y[4 * q + 2] = v.z, e.y[4 * q + 3] = v.w;
        }
        const unsigned co = static_cast<unsigned>(idx) * (16u * C) + unsigned(K::off(cl));  // 32-bit offset from the uniform table base
        // addressed from the middle of the interval's 16C-float row: all 16 pieces lie within +-8C floats of it, which
        // up to C = 128 fits the signed immediate offset of a load, so one address serves them all
        const float *mid = sp.coeffs + (co + 8 * C);
#pragma unroll
        for (int q = 0; q < 16; ++q) e.coef[q] = K::ld(mid + (q * C - 8 * C));  // piece q: coefficient q / 4 of degree q % 4
      };
      auto accumulate = [&](const Edge &e) {
        auto per_l = [&](auto lc) {
          constexpr int L = decltype(lc)::value;
          const vec t = e.x * (e.coef[L] + e.xr * (e.coef[4 + L] + e.xr * (e.coef[8 + L] + e.xr * e.coef[12 + L])));
#pragma unroll
          for (int m = MRange<L>::lo; m < MRange<L>::hi; ++m) acc[m] += e.y[m] * t;
        };
        per_l(std::integral_constant<int, 0>{});
        per_l(std::integral_constant<int, 1>{});
        per_l(std::integral_constant<int, 2>{});
        per_l(std::integral_constant<int, 3>{});
      };
      if constexpr (MULTI && K::V <= 4) {
        // few nodes: a wave's part is a dozen edges, and what it waits for is one memory round trip per trip of this
        // loop, so two edges per slot are requested per trip (same order of the sums; registers for it up to four
        // channels per lane)
        for (int j = slot; j < nlive; j += 2 * K::EPW) {
          Edge e0, e1;
          const bool two = j + K::EPW < nlive;
          fetch(j, e0);
          fetch(two ? j + K::EPW : j, e1);
          __builtin_amdgcn_sched_barrier(0);  // both edges' loads stay ahead of the first edge's arithmetic
          accumulate(e0);
          if (two) accumulate(e1);
        }
      } else {
        // one edge per trip; per degree the four coefficient pieces are loaded, used and dropped (16 registers of
        // radial data live at a time)
        for (int j = slot; j < nlive; j += K::EPW) {
          const int s = sS[j];
          const int idx = sIdx[j];
          const float xr = sXr[j];
          const vec x = K::ld(X + (static_cast<unsigned>(s) * C + unsigned(K::off(cl))));
          float y[16];
          {
            const f4 *yp = reinterpret_cast<const f4 *>(sY + j * 16);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const f4 v = yp[q];
              y[4 * q] = v.x, y[4 * q + 1] = v.y, y[4 * q + 2] = v.z, y[4 * q + 3] = v.w;
            }
          }
          const unsigned co = static_cast<unsigned>(idx) * (16u * C) + unsigned(K::off(cl));
          const float *__restrict__ tab = sp.coeffs;
          auto per_l = [&](auto lc) {
            constexpr int L = decltype(lc)::value;
            const float *mid = tab + (co + 8 * C);
            const vec a = K::ld(mid + (L * C - 8 * C)), b = K::ld(mid + (L * C - 4 * C)), c = K::ld(mid + L * C),
                      d = K::ld(mid + (L * C + 4 * C));
            const vec t = x * (a + xr * (b + xr * (c + xr * d)));
#pragma unroll
            for (int m = MRange<L>::lo; m < MRange<L>::hi; ++m) acc[m] += y[m] * t;
          };
          per_l(std::integral_constant<int, 0>{});
          per_l(std::integral_constant<int, 1>{});
          per_l(std::integral_constant<int, 2>{});
          per_l(std::integral_constant<int, 3>{});
        }
      }
    }
  }

#pragma unroll
  for (int off = kWave / 2; off >= K::SW; off >>= 1) {
#pragma unroll
    for (int m = 0; m < 16; ++m) acc[m] += shfl_downv(acc[m], off);
  }
  if (parts > 1) {
    // sums of the parts, added up by the first wave in the order of the parts (the same on every run)
    float *comb = reinterpret_cast<float *>(dyn_lds + parts * kStageBytes);
    if (wave > 0 && slot == 0 && active) {
      float *cp = comb + (wave - 1) * (16 * C) + K::off(cl);
#pragma unroll
      for (int m = 0; m < 16; ++m) K::st(cp + m * C, acc[m]);
    }
    __syncthreads();
    if (wave > 0) return;
    if (slot == 0 && active) {
      for (int w = 1; w < parts; ++w) {
        const float *cp = comb + (w - 1) * (16 * C) + K::off(cl);
#pragma unroll
        for (int m = 0; m < 16; ++m) acc[m] += K::ld(cp + m * C);
      }
    }
  }
  if (slot == 0 && active) {
    float *op = out + static_cast<int64_t>(node) * (16 * C) + K::off(cl);
#pragma unroll
    for (int m = 0; m < 16; ++m) K::st(op + m * C, acc[m]);
  }
}

// -----------------------------------------------------------------------------------------------
// backward, edge pass: gY, g_r and the per-edge contribution to gX
// -----------------------------------------------------------------------------------------------
template <int C, bool FROM_VEC, bool WANT_GY, bool WANT_GR, bool WANT_GX>
__global__ __launch_bounds__(kWave, CM_FUSED_BWD_WAVES) void mp_spline_backward_edge_kernel(
    const float *__restrict__ X, const float *__restrict__ Y, Spline sp, const float *__restrict__ G,
    const int32_t *__restrict__ sender, const int32_t *__restrict__ first_occ, int nnodes, int64_t nedges,
    float *__restrict__ gY, float *__restrict__ g_r, float *__restrict__ gXe, int parts) {
  using K = Cfg<C>;
  using vec = typename K::vec;
  __shared__ __attribute__((aligned(16))) float sY[kChunk * 16];
  __shared__ int sS[kChunk];
  __shared__ int sIdx[kChunk];
  __shared__ float sXr[kChunk];
  __shared__ int sOrig[kChunk];
  __shared__ float sGY[16 * kChunk];  // [m][edge]
  __shared__ float sGr[kChunk];
  // The knots, where there are at most kKnotsInLds of them: the staging looks one up per edge, and a lookup in memory is
  // waited for behind everything the wave has in flight (the gradient rows from HBM first of all).
  __shared__ float sKnots[kKnotsInLds];

  // one wave per node, or (few nodes: parts_for) per part of a node's edge range: every output of this pass belongs to
  // one edge, so the parts share nothing but the node's gradient rows, which each of them reads
  const int node = parts == 1 ? blockIdx.x : blockIdx.x / parts;
  const int lane = threadIdx.x;
  const int slot = lane / K::SW;
  const int cl = lane % K::SW;
  const bool active = cl < K::LPE;
  const unsigned cla = active ? cl : 0;  // lanes beyond the channel count read lane 0's addresses; their g is zero
  const bool knots_in_lds = sp.nknots <= kKnotsInLds;
  float knot[kKnotsInLds / kWave];
#pragma unroll
  for (int q = 0; q < kKnotsInLds / kWave; ++q) knot[q] = sp.knots[min(lane + kWave * q, sp.nknots - 1)];
  __builtin_amdgcn_sched_barrier(0);
  int e0 = first_occ[node];
  int e1 = first_occ[nnodes + node];
  clamp_edge_range(e0, e1, nedges);
  if (parts > 1) {
    const int part = blockIdx.x % parts;
    const int64_t len = e1 - e0;
    const int lo = e0 + static_cast<int>(len * part / parts);
    e1 = e0 + static_cast<int>(len * (part + 1) / parts);
    e0 = lo;
  }
  if (e0 >= e1) return;

  // Order of the first requests: the raw edges of the first chunk (from L2, and the staging waits for them), then the
  // node's gradient rows (from HBM, read once, not needed before the first edge's arithmetic).  Memory operations retire
  // in issue order, so with the rows in front the staging would wait for them as well.
  RawEdge ahead{-1, 0.f, 0.f, 0.f};
  if constexpr (FROM_VEC) {
    const int64_t e = min(static_cast<int64_t>(e0) + lane, nedges - 1);  // unconditional; lanes beyond the range drop it
    ahead.s = sender[e];
    ahead.v0 = sp.vec[3 * e + 0], ahead.v1 = sp.vec[3 * e + 1], ahead.v2 = sp.vec[3 * e + 2];
    __builtin_amdgcn_sched_barrier(0);
  }
  vec g[16];
  {
    const float *gp = G + static_cast<int64_t>(node) * (16 * C) + K::off(cl);
#pragma unroll
    for (int m = 0; m < 16; ++m) g[m] = active ? K::ld_stream(gp + m * C) : zerov<vec>();  // read once
  }
  __builtin_amdgcn_sched_barrier(0);
  if (knots_in_lds) {
#pragma unroll
    for (int q = 0; q < kKnotsInLds / kWave; ++q) sKnots[lane + kWave * q] = knot[q];
  }

  // The first chunk is written out ahead of the loop over the others (most nodes have no others): at a loop's head the
  // compiler has to assume that the loads a previous iteration left in flight (a slot's last, unused look-ahead) are still
  // on their way into registers the staging reuses, and waits for everything, the gradient rows included.
  int cursor = e0;
  auto chunk = [&](auto first_chunk) {
    const int base = cursor;  // sOrig counts from here
    // (the workgroup is this one wave: ordering its own LDS traffic is all that is needed, and a workgroup barrier would
    // wait for everything in flight first, the gradient rows and the previous chunk's stores included)
    wave_lds_fence();
    // consumed edges that are not live: their gradients are zeros (their rows of gXe stay unwritten: the sender pass
    // reads the rows of live edges only)
    auto dead = [&](int pass_base, int, unsigned long long, bool lane_is_dead) {
      if constexpr (WANT_GY || WANT_GR) {
        if (lane_is_dead) {
          const int64_t e = pass_base + lane;
          if constexpr (FROM_VEC) {
            gY[3 * e + 0] = g_r ? g_r[3 * e + 0] : 0.f;
            gY[3 * e + 1] = g_r ? g_r[3 * e + 1] : 0.f;
            gY[3 * e + 2] = g_r ? g_r[3 * e + 2] : 0.f;
          } else {
            if constexpr (WANT_GY) {
#pragma unroll
              for (int m = 0; m < 16; ++m) gY[m * nedges + e] = 0.f;
            }
            if constexpr (WANT_GR) g_r[e] = 0.f;
          }
        }
      }
    };
    const int nlive = stage_edges<FROM_VEC, FROM_VEC && decltype(first_chunk)::value>(
        Y, sender, sp, nnodes, nedges, cursor, e1, lane, sY, sS, sIdx, sXr, sOrig, dead, ahead, sKnots, knots_in_lds);
    wave_lds_fence();
    // Every lane of a slot takes part in the reductions, so the loop bound is slot-uniform; only live edges are staged.
    // The loop is rotated: the sender row and the 16 coefficient pieces of the NEXT edge are requested right after the
    // arithmetic of the current one, so they travel while the cross-lane reductions (a chain of dependent lane
    // exchanges) run.
    // Two operand sets used in turn (the loop body is written out twice), so that the set being loaded is never copied
    // into the set being consumed.
    struct Operands {
      vec x, ca[4], cb[4], cc[4], cd[4];
      float xr;
    };
    auto fetch = [&](Operands &o, int j) {
      const int s = sS[j];
      const int idx = sIdx[j];
      o.xr = sXr[j];
      o.x = K::ld(X + (static_cast<unsigned>(s) * C + unsigned(K::off(cla))));
      const unsigned co = static_cast<unsigned>(idx) * (16u * C) + unsigned(K::off(cla));
      const float *__restrict__ tab = sp.coeffs;
#pragma unroll
      for (int L = 0; L < 4; ++L) {
        // addressed from the middle of the interval's 16C-float row (offsets within +-8C floats: one address and
        // immediate offsets, up to C = 128)
        const float *mid = tab + (co + 8 * C);
        o.ca[L] = K::ld(mid + (L * C - 8 * C));
        o.cb[L] = K::ld(mid + (L * C - 4 * C));
        o.cc[L] = K::ld(mid + L * C);
        o.cd[L] = K::ld(mid + (L * C + 4 * C));
      }
    };
    auto edge = [&](const Operands &o, int j, Operands &next) {
      float y[16];
      {
        const f4 *yp = reinterpret_cast<const f4 *>(sY + j * 16);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const f4 v = yp[q];
          y[4 * q] = v.x, y[4 * q + 1] = v.y, y[4 * q + 2] = v.z, y[4 * q + 3] = v.w;
        }
      }
      const float xr = o.xr;
      const float xr2 = 2.f * xr, xr3 = 3.f * xr * xr;
      float p[16];
      vec gxe = zerov<vec>();
      vec grq = zerov<vec>();
      auto per_l = [&](auto lc) {
        constexpr int L = decltype(lc)::value;
        const vec a = o.ca[L], b = o.cb[L], c = o.cc[L], d = o.cd[L];
        const vec rl = a + xr * (b + xr * (c + xr * d));
        vec q = zerov<vec>();
#pragma unroll
        for (int m = MRange<L>::lo; m < MRange<L>::hi; ++m) q += y[m] * g[m];
        if constexpr (WANT_GY) {
          const vec t = o.x * rl;
#pragma unroll
          for (int m = MRange<L>::lo; m < MRange<L>::hi; ++m) p[m] = dotv(g[m], t);
        }
        if constexpr (WANT_GX) gxe += rl * q;
        if constexpr (WANT_GR) grq += q * (b + xr2 * c + xr3 * d);  // q_l * dR_l/dr
      };
      per_l(std::integral_constant<int, 0>{});
      per_l(std::integral_constant<int, 1>{});
      per_l(std::integral_constant<int, 2>{});
      per_l(std::integral_constant<int, 3>{});
      float grv = 0.f;
      if constexpr (WANT_GR) grv = hsumv(o.x * grq);

      if constexpr (WANT_GX) {
        // streamed out: 666 MB at the headline size, read once by the sender pass (measured 2 % on the whole step).
        // Issued before the loads of the next edge: memory operations retire in issue order, so a store that is
        // younger than those loads would have to be complete wherever the loop waits for all of them.
        if (active) K::st_stream(gXe + static_cast<int64_t>(base + sOrig[j]) * C + K::off(cl), gxe);
        __builtin_amdgcn_sched_barrier(0);  // keeps the instruction scheduler from sinking the store below the loads
      }
      // Unconditional (the last edge of a slot fetches itself again): loads under a branch would make every later wait
      // assume that they were not issued, i.e. wait for all but the oldest few of them.
      fetch(next, j + K::EPW < nlive ? j + K::EPW : j);
      if constexpr (WANT_GR) {
        const float tot = slot_sum<K::SW>(grv);
        if (cl == 0) sGr[j] = tot;
      }
      if constexpr (WANT_GY) {
        slot_reduce16<K::SW>(p, cl);
        store_reduced16<K::SW>(p, cl, j, sGY);
      }
    };
    Operands opa, opb;
    if (slot < nlive) fetch(opa, slot);
    for (int j = slot; j < nlive; j += 2 * K::EPW) {
      edge(opa, j, opb);
      if (j + K::EPW >= nlive) break;
      edge(opb, j + K::EPW, opa);
    }
    if constexpr (WANT_GY || WANT_GR) {
      wave_lds_fence();
      // lane k < nlive finishes the k-th staged edge
      if (lane < nlive) {
        const int64_t e = base + sOrig[lane];
        if constexpr (FROM_VEC) {
          // gradient with respect to the edge vector: harmonics Jacobian applied to gY, plus g_r along the direction
          // (gY doubles as the output pointer of the [E, 3] vector gradient in this variant)
          const float v0 = sp.vec[3 * e + 0], v1 = sp.vec[3 * e + 1], v2 = sp.vec[3 * e + 2];
          const sh::Direction d = sh::direction(v0, v1, v2);
          float gy[16], gin[3];
#pragma unroll
          for (int m = 0; m < 16; ++m) gy[m] = sGY[m * kChunk + lane];
          sh::vjp(d, gy, gin);
          const float gr = sGr[lane];
          float o0 = gin[0] + gr * d.y, o1 = gin[1] + gr * d.z, o2 = gin[2] + gr * d.x;
          if (g_r) {
            // g_r doubles as an optional [E, 3] addend in this variant (another layer's gradient of the same vectors);
            // the sum is formed from the rounded value, as a separate addition pass would form it
            o0 = __fadd_rn(o0, g_r[3 * e + 0]);
            o1 = __fadd_rn(o1, g_r[3 * e + 1]);
            o2 = __fadd_rn(o2, g_r[3 * e + 2]);
          }
          gY[3 * e + 0] = o0;
          gY[3 * e + 1] = o1;
          gY[3 * e + 2] = o2;
        } else {
          if constexpr (WANT_GY) {
#pragma unroll
            for (int m = 0; m < 16; ++m) gY[m * nedges + e] = sGY[m * kChunk + lane];
          }
          if constexpr (WANT_GR) g_r[e] = sGr[lane];
        }
      }
    }
  };
  chunk(std::true_type{});
  while (cursor < e1) chunk(std::false_type{});
}

template <int C, bool FROM_VEC>
int launch_forward(const float *X, const float *Y, const Spline &sp, const int32_t *sender, const int32_t *first_occ,
                   int64_t nnodes, int64_t nedges, float *out, hipStream_t st) {
  const int parts = parts_for(nnodes, nedges);
  const size_t lds = static_cast<size_t>(parts) * kStageBytes + static_cast<size_t>(parts - 1) * 16 * C * sizeof(float);
  if (parts > 1)
    hipLaunchKernelGGL((mp_spline_forward_kernel<C, FROM_VEC, true>), dim3(static_cast<unsigned>(nnodes)), dim3(kWave * parts), lds, st,
                       X, Y, sp, sender, first_occ, static_cast<int>(nnodes), nedges, out);
  else
    hipLaunchKernelGGL((mp_spline_forward_kernel<C, FROM_VEC, false>), dim3(static_cast<unsigned>(nnodes)), dim3(kWave), lds, st, X, Y,
                       sp, sender, first_occ, static_cast<int>(nnodes), nedges, out);
  return check_launch(FROM_VEC ? "cm_mp_edge_forward" : "cm_mp_spline_forward");
}

template <int C, bool FROM_VEC, bool GY, bool GR, bool GX>
void launch_edge(const float *X, const float *Y, const Spline &sp, const float *G, const int32_t *sender,
                 const int32_t *first_occ, int64_t nnodes, int64_t nedges, float *gY, float *g_r, float *gXe,
                 hipStream_t st) {
  const int parts = parts_for(nnodes, nedges);
  hipLaunchKernelGGL((mp_spline_backward_edge_kernel<C, FROM_VEC, GY, GR, GX>), dim3(static_cast<unsigned>(nnodes * parts)),
                     dim3(kWave), 0, st, X, Y, sp, G, sender, first_occ, static_cast<int>(nnodes), nedges, gY, g_r, gXe, parts);
}

// gY / g_r: outputs of the Y-and-r variant; in the FROM_VEC variant gY is the [E, 3] vector gradient and g_r, when given,
// an [E, 3] addend to it (read only).
template <int C, bool FROM_VEC>
int launch_backward(const float *X, const float *Y, const Spline &sp, const float *G, const int32_t *sender,
                    const int32_t *first_occ, const int32_t *perm, const int32_t *offsets, int64_t nnodes, int64_t nedges,
                    float *gX, float *gY, float *g_r, float *gXe, hipStream_t st) {
  if constexpr (FROM_VEC) {
    if (gY && gX) launch_edge<C, true, true, true, true>(X, Y, sp, G, sender, first_occ, nnodes, nedges, gY, g_r, gXe, st);
    else if (gY) launch_edge<C, true, true, true, false>(X, Y, sp, G, sender, first_occ, nnodes, nedges, gY, g_r, gXe, st);
    else if (gX) launch_edge<C, true, false, false, true>(X, Y, sp, G, sender, first_occ, nnodes, nedges, gY, g_r, gXe, st);
    else return CM_OK;
  } else {
    const int key = (gY ? 4 : 0) | (g_r ? 2 : 0) | (gX ? 1 : 0);
    switch (key) {
      case 7: launch_edge<C, false, true, true, true>(X, Y, sp, G, sender, first_occ, nnodes, nedges, gY, g_r, gXe, st); break;
      case 6: launch_edge<C, false, true, true, false>(X, Y, sp, G, sender, first_occ, nnodes, nedges, gY, g_r, gXe, st); break;
      case 5: launch_edge<C, false, true, false, true>(X, Y, sp, G, sender, first_occ, nnodes, nedges, gY, g_r, gXe, st); break;
      case 4: launch_edge<C, false, true, false, false>(X, Y, sp, G, sender, first_occ, nnodes, nedges, gY, g_r, gXe, st); break;
      case 3: launch_edge<C, false, false, true, true>(X, Y, sp, G, sender, first_occ, nnodes, nedges, gY, g_r, gXe, st); break;
      case 2: launch_edge<C, false, false, true, false>(X, Y, sp, G, sender, first_occ, nnodes, nedges, gY, g_r, gXe, st); break;
      case 1: launch_edge<C, false, false, false, true>(X, Y, sp, G, sender, first_occ, nnodes, nedges, gY, g_r, gXe, st); break;
      default: return CM_OK;
    }
  }
  int rc = check_launch(FROM_VEC ? "cm_mp_edge_backward (edge pass)" : "cm_mp_spline_backward (edge pass)");
  if (rc != CM_OK) return rc;
  if (gX) rc = mp::launch_sender_pass(C, gXe, perm, offsets, nnodes, nedges, gX, st, FROM_VEC ? sp.vec : nullptr,
                                      FROM_VEC ? nullptr : sp.r, sp.r_max);
  return rc;
}

int check_spline(const char *who, const float *r_or_vec, const float *r_knots, const float *coeffs, int nknots,
                 float r_width, int64_t nedges, int64_t nnodes, int channels) {
  // the kernels address X rows and table rows with 32-bit element offsets
  CM_REQUIRE(nnodes * channels < (int64_t{1} << 31) && static_cast<int64_t>(nknots) * 16 * channels < (int64_t{1} << 31),
             "%s: nnodes * channels or the spline table exceeds 32-bit element offsets", who);
  CM_REQUIRE(nknots >= 2, "%s: need at least two knots, got %d", who, nknots);
  CM_REQUIRE(r_width > 0.f, "%s: r_width must be positive", who);
  CM_REQUIRE(nedges == 0 || (r_or_vec && r_knots && coeffs), "%s: NULL spline operand", who);
  return CM_OK;
}

}  // namespace
}  // namespace cm

extern "C" int cm_mp_spline_forward(const float *X, const float *Y, const float *r, const float *r_knots,
                                    const float *coeffs, int nknots, float r_width, float r_max, const int32_t *sender,
                                    const int32_t *first_occ, int64_t nnodes, int64_t nedges, int channels, float *out,
                                    cm_stream_t stream) {
  CM_REQUIRE(cm_channels_supported(channels), "cm_mp_spline_forward: channels=%d must be a multiple of 32 in [32, 256]", channels);
  CM_REQUIRE(nedges >= 0 && nnodes >= 0, "cm_mp_spline_forward: negative size");
  CM_REQUIRE(nedges < INT32_MAX && nnodes < INT32_MAX / 2, "cm_mp_spline_forward: sizes exceed int32 indexing");
  if (nnodes == 0) return CM_OK;
  CM_REQUIRE(X && first_occ && out, "cm_mp_spline_forward: NULL pointer");
  CM_REQUIRE(nedges == 0 || (Y && sender), "cm_mp_spline_forward: NULL edge operand");
  int rc = cm::check_spline("cm_mp_spline_forward", r, r_knots, coeffs, nknots, r_width, nedges, nnodes, channels);
  if (rc != CM_OK) return rc;
  const cm::Spline sp{nullptr, r, r_knots, coeffs, nknots, r_width, r_max};
  rc = CM_EINVAL;
  CM_DISPATCH_C(channels, rc = (cm::launch_forward<C_, false>(X, Y, sp, sender, first_occ, nnodes, nedges, out, cm::as_stream(stream))));
  return rc;
}

extern "C" int cm_mp_spline_backward(const float *X, const float *Y, const float *r, const float *r_knots,
                                     const float *coeffs, int nknots, float r_width, float r_max, const float *grad_out,
                                     const int32_t *sender, const int32_t *first_occ, const int32_t *sender_perm,
                                     const int32_t *sender_offsets, int64_t nnodes, int64_t nedges, int channels,
                                     float *gX, float *gY, float *grad_r, float *edge_scratch, cm_stream_t stream) {
  CM_REQUIRE(cm_channels_supported(channels), "cm_mp_spline_backward: channels=%d must be a multiple of 32 in [32, 256]", channels);
  CM_REQUIRE(nedges >= 0 && nnodes >= 0, "cm_mp_spline_backward: negative size");
  CM_REQUIRE(nedges < INT32_MAX && nnodes < INT32_MAX / 2, "cm_mp_spline_backward: sizes exceed int32 indexing");
  if (nnodes == 0) return CM_OK;
  CM_REQUIRE(X && grad_out && first_occ, "cm_mp_spline_backward: NULL pointer");
  CM_REQUIRE(nedges == 0 || (Y && sender), "cm_mp_spline_backward: NULL edge operand");
  CM_REQUIRE(!gX || (sender_offsets && (nedges == 0 || (sender_perm && edge_scratch))),
             "cm_mp_spline_backward: gX wanted but sender_perm / sender_offsets / edge_scratch missing");
  int rc = cm::check_spline("cm_mp_spline_backward", r, r_knots, coeffs, nknots, r_width, nedges, nnodes, channels);
  if (rc != CM_OK) return rc;
  const cm::Spline sp{nullptr, r, r_knots, coeffs, nknots, r_width, r_max};
  rc = CM_EINVAL;
  CM_DISPATCH_C(channels, rc = (cm::launch_backward<C_, false>(X, Y, sp, grad_out, sender, first_occ, sender_perm, sender_offsets,
                                                               nnodes, nedges, gX, gY, grad_r, edge_scratch, cm::as_stream(stream))));
  return rc;
}

extern "C" int cm_mp_edge_forward(const float *X, const float *vectors, const float *r_knots, const float *coeffs, int nknots,
                                  float r_width, float r_max, const int32_t *sender, const int32_t *first_occ,
                                  int64_t nnodes, int64_t nedges, int channels, float *out, cm_stream_t stream) {
  CM_REQUIRE(cm_channels_supported(channels), "cm_mp_edge_forward: channels=%d must be a multiple of 32 in [32, 256]", channels);
  CM_REQUIRE(nedges >= 0 && nnodes >= 0, "cm_mp_edge_forward: negative size");
  CM_REQUIRE(nedges < INT32_MAX / 3 && nnodes < INT32_MAX / 2, "cm_mp_edge_forward: sizes exceed int32 indexing");
  if (nnodes == 0) return CM_OK;
  CM_REQUIRE(X && first_occ && out, "cm_mp_edge_forward: NULL pointer");
  CM_REQUIRE(nedges == 0 || sender, "cm_mp_edge_forward: NULL edge operand");
  int rc = cm::check_spline("cm_mp_edge_forward", vectors, r_knots, coeffs, nknots, r_width, nedges, nnodes, channels);
  if (rc != CM_OK) return rc;
  if (nedges > 0 && cm::mp::sliced_forward_applies(nnodes, channels, nknots))
    return cm::mp::launch_sliced_forward(X, vectors, r_knots, coeffs, nknots, r_width, r_max, sender, first_occ, nnodes, nedges,
                                         channels, out, cm::as_stream(stream));
  const cm::Spline sp{vectors, nullptr, r_knots, coeffs, nknots, r_width, r_max};
  rc = CM_EINVAL;
  CM_DISPATCH_C(channels, rc = (cm::launch_forward<C_, true>(X, nullptr, sp, sender, first_occ, nnodes, nedges, out, cm::as_stream(stream))));
  return rc;
}

namespace cm {
namespace mp {

// cm_mp_edge_backward without gX whose vector gradient is written as (this layer's gradient + addend[e]): saves the pass
// that adds two layers' gradients of the same edge vectors.  Arguments as checked by the caller (cm_mace_step).
int edge_backward_onto(const float *X, const float *vectors, const float *r_knots, const float *coeffs, int nknots, float r_width,
                       float r_max, const float *grad_out, const int32_t *sender, const int32_t *first_occ, int64_t nnodes,
                       int64_t nedges, int channels, float *grad_vectors, const float *addend, hipStream_t st) {
  if (nnodes == 0) return CM_OK;
  const Spline sp{vectors, nullptr, r_knots, coeffs, nknots, r_width, r_max};
  int rc = CM_EINVAL;
  CM_DISPATCH_C(channels, rc = (launch_backward<C_, true>(X, nullptr, sp, grad_out, sender, first_occ, nullptr, nullptr, nnodes, nedges,
                                                          nullptr, grad_vectors, const_cast<float *>(addend), nullptr, st)));
  return rc;
}

}  // namespace mp
}  // namespace cm

extern "C" int cm_mp_edge_backward(const float *X, const float *vectors, const float *r_knots, const float *coeffs, int nknots,
                                   float r_width, float r_max, const float *grad_out, const int32_t *sender,
                                   const int32_t *first_occ, const int32_t *sender_perm, const int32_t *sender_offsets,
                                   int64_t nnodes, int64_t nedges, int channels, float *gX, float *grad_vectors,
                                   float *edge_scratch, cm_stream_t stream) {
  CM_REQUIRE(cm_channels_supported(channels), "cm_mp_edge_backward: channels=%d must be a multiple of 32 in [32, 256]", channels);
  CM_REQUIRE(nedges >= 0 && nnodes >= 0, "cm_mp_edge_backward: negative size");
  CM_REQUIRE(nedges < INT32_MAX / 3 && nnodes < INT32_MAX / 2, "cm_mp_edge_backward: sizes exceed int32 indexing");
  if (nnodes == 0) return CM_OK;
  CM_REQUIRE(X && grad_out && first_occ, "cm_mp_edge_backward: NULL pointer");
  CM_REQUIRE(nedges == 0 || sender, "cm_mp_edge_backward: NULL edge operand");
  CM_REQUIRE(!gX || (sender_offsets && (nedges == 0 || (sender_perm && edge_scratch))),
             "cm_mp_edge_backward: gX wanted but sender_perm / sender_offsets / edge_scratch missing");
  int rc = cm::check_spline("cm_mp_edge_backward", vectors, r_knots, coeffs, nknots, r_width, nedges, nnodes, channels);
  if (rc != CM_OK) return rc;
  const cm::Spline sp{vectors, nullptr, r_knots, coeffs, nknots, r_width, r_max};
  rc = CM_EINVAL;
  CM_DISPATCH_C(channels, rc = (cm::launch_backward<C_, true>(X, nullptr, sp, grad_out, sender, first_occ, sender_perm,
                                                              sender_offsets, nnodes, nedges, gX, grad_vectors, nullptr,
                                                              edge_scratch, cm::as_stream(stream))));
  return rc;
}
