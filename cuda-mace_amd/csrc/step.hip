// One energy + forces evaluation of the two-layer invariant model: the library enqueues every kernel of the step
// itself, forward and then the hand-written backward chain, through the same entry points a caller could use one by
// one.  Nothing here computes; this file is the order of the launches and the layout of the workspace.
//
// Forward                                         Backward (seed -1 on every node energy: the chain delivers forces)
//   vec        = pos[snd] - pos[rcv] + shift        g1 = -scale w1 (every node), g2 = -dE/dh2 (never stored: the sign
//                                                             goes into the scale of the linears that read dE/dh2)
//   live       = edge ranges up to the last pair
//                inside the cutoff (forward MP only)
//   M1         = MP(X1, vec, spline 0)              gB2       = g2 . Wprod2^T
//   A          = mix0(M1)        (per element)      gA        = (gB2 * grad2) . Wmix1^T      (contraction backward folded)
//   B1, grad1  = contraction 0 (A)                  gX2, gv2  = MP backward(X2, vec, spline 1, gA)
//   h1         = B1 . Wprod1                        gh1       = gX2 . Wup^T + g1 ;  gh1 += skip^T(g2)
//   sc         = skip(h1)        (per element)      gB1       = gh1 . Wprod1^T
//   X2         = h1 . Wup                           gA        = (gB1 * grad1) . Wmix0^T      (per element)
//   M2         = MP(X2, vec, spline 1)              gv1       = MP backward(X1, vec, spline 0, gA)   (no gX: X1 is constant)
//   A          = mix1(M2)                           forces    = geometry backward(gv1 + gv2)
//   B2, grad2  = contraction 1 (A)                  virials   = 1/2 sum_e (vec (x) gv + gv (x) vec), per node, then per graph
//   h2         = B2 . Wprod2 + sc                               (on request)
//   E_n, dE/dh2, feats = readouts(h1, h2);  E_graph = sum over the graph's nodes
// With node weights (cm_mace_graph.node_weights) E_graph = sum_n weight[n] E_n and the seed of node n is -weight[n]: g1's
// rows and the rows of dE/dh2 are multiplied by the node's weight before the chain starts.
#include <cstdlib>
#include <mutex>
#include <vector>

#include "common.hpp"
#include "mp_common.hpp"
#include "node_glue.hpp"
#include "readout.hpp"

namespace cm {
namespace {

// ---- optional per-stage timing: events on the launch stream around chosen stages of the step --------------------
constexpr int kStages = 25;
struct Pending {
  int stage;
  hipEvent_t start, stop;
};
std::mutex g_timing_mutex;
unsigned g_timing_mask = 0;  // bit s set: stage s is bracketed by events
std::vector<Pending> g_pending;
std::vector<hipEvent_t> g_event_pool;
double g_stage_ms[kStages] = {};
int64_t g_stage_launches[kStages] = {};

hipEvent_t take_event() {
  if (!g_event_pool.empty()) {
    hipEvent_t e = g_event_pool.back();
    g_event_pool.pop_back();
    return e;
  }
  hipEvent_t e = nullptr;
  (void)hipEventCreate(&e);
  return e;
}

// Brackets one stage with events when its bit is set; used only through CM_STAGE below.
struct StageTimer {
  hipStream_t st;
  int stage;
  hipEvent_t start = nullptr;
  StageTimer(hipStream_t s, int stage_, unsigned mask) : st(s), stage(stage_) {
    if (mask >> stage & 1u) {
      std::lock_guard<std::mutex> lock(g_timing_mutex);
      start = take_event();
      if (start) (void)hipEventRecord(start, st);
    }
  }
  ~StageTimer() {
    if (!start) return;
    std::lock_guard<std::mutex> lock(g_timing_mutex);
    hipEvent_t stop = take_event();
    if (stop) {
      (void)hipEventRecord(stop, st);
      g_pending.push_back({stage, start, stop});
    } else {
      g_event_pool.push_back(start);
    }
  }
};

__global__ void fill_f64_kernel(double *p, int64_t n, double value) {
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x)
    p[i] = value;
}

// p[i] = src[i], or zero without a source
__global__ void copy_or_zero_f64_kernel(double *p, const double *src, int64_t n) {
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x)
    p[i] = src ? src[i] : 0.0;
}

// g1[n, c] = -weight[n] * scale * w1[c]: the gradient of -sum(weight * node energies) with respect to the first layer's
// features (the linear readout); without weights the same row for every node
__global__ void seed_linear_readout_kernel(float *__restrict__ g1, const double *__restrict__ w1, double scale,
                                           const double *__restrict__ node_weights, int64_t total, int C) {
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x)
    g1[i] = static_cast<float>(-1.0 * scale * w1[i % C] * (node_weights ? node_weights[i / C] : 1.0));
}

// rows of x [nnodes, C] times the node's weight (the second readout's derivative, when node energies carry weights)
__global__ void weight_rows_kernel(float *__restrict__ x, const double *__restrict__ node_weights, int64_t total, int C) {
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x)
    x[i] = static_cast<float>(static_cast<double>(x[i]) * node_weights[i / C]);
}

// Edge vectors and the edge range of every receiver node cut back to its last edge inside the cutoff, one launch.
// Thread i forms the vector of edge i (fp64 difference of the positions plus the shift, rounded once to fp32: the
// arithmetic of cm_edge_geometry_forward) and clears the vector gradients of an edge beyond the cutoff (the backward edge
// passes skip the edges behind a node's mark, and write the same zeros for those before it).  The thread of a receiver's
// last edge closes the receiver's range: live[n] = first_occ[n], live[nnodes + n] = one past the last edge e of the node
// with |vec[e]| <= r_max (the node's first edge if there is none).  The message-passing kernels, forward and backward,
// skip the edges behind that mark, which contribute exact zeros.  A Verlet list holds a third more pairs than the cutoff
// takes in; the model orders each node's pairs with those of the skin shell last, nearest first, so that most of them
// fall behind the mark.  The closing thread reads the mark off the workgroup's ballots of "inside the cutoff" where the
// node's edges up to the mark lie among the workgroup's 256; otherwise it walks back from the workgroup's first edge,
// forming those vectors again (a walk over all of a node's tail, one line of memory per lane and access, cost a list
// with a skin 60 us per step).  The length is the one the message-passing kernels compute from the same fp32 vector.
__device__ __forceinline__ int walk_back_to_live_edge(const double *__restrict__ pos, const int32_t *__restrict__ a,
                                                      const int32_t *__restrict__ b, const double *__restrict__ shifts,
                                                      const int32_t *__restrict__ rows, int nnodes, float r_max, int e0, int e) {
  constexpr int kAhead = 4;  // edges per trip, their operands requested together
  bool found = false;
  while (e > e0 && !found) {
    float len[kAhead];
#pragma unroll
    for (int u = 0; u < kAhead; ++u) {
      const int64_t q = max(e - 1 - u, e0);  // below the range: the first edge again, never looked at
      double w[3];
      edge_vector_f64(pos, a, b, shifts, rows, q, nnodes, w);
      len[u] = mp::edge_length(static_cast<float>(w[0]), static_cast<float>(w[1]), static_cast<float>(w[2]));
    }
#pragma unroll
    for (int u = 0; u < kAhead; ++u) {
      if (found || e <= e0) continue;
      if (len[u] <= r_max)
        found = true;
      else
        --e;
    }
  }
  return e;
}

__global__ __launch_bounds__(256) void geometry_live_range_kernel(const double *__restrict__ pos, const int32_t *__restrict__ a,
                                                                  const int32_t *__restrict__ b, const double *__restrict__ shifts,
                                                                  const int32_t *__restrict__ rows, const int32_t *__restrict__ first_occ,
                                                                  float r_max, int nnodes, int64_t nedges, float *__restrict__ vec,
                                                                  int32_t *__restrict__ live, float *__restrict__ gv1,
                                                                  float *__restrict__ gv2) {
  const int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  const int lane = threadIdx.x % kWave;
  bool inside = false;
  int recv = -1, next_recv = -2;
  if (i < nedges) {
    double v[3];
    edge_vector_f64(pos, a, b, shifts, rows, i, nnodes, v);
    const float v0 = static_cast<float>(v[0]), v1 = static_cast<float>(v[1]), v2 = static_cast<float>(v[2]);
    vec[3 * i + 0] = v0;
    vec[3 * i + 1] = v1;
    vec[3 * i + 2] = v2;
    inside = mp::edge_length(v0, v1, v2) <= r_max;
    if (!inside) {
      gv1[3 * i + 0] = gv1[3 * i + 1] = gv1[3 * i + 2] = 0.f;
      gv2[3 * i + 0] = gv2[3 * i + 1] = gv2[3 * i + 2] = 0.f;
    }
    recv = a[i];
    next_recv = i + 1 < nedges ? a[i + 1] : -2;
  }
  // "inside the cutoff" of the workgroup's 256 consecutive edges, one word per wave (every thread arrives here)
  __shared__ unsigned long long s_inside[4];
  const int wave = threadIdx.x / kWave;
  const unsigned long long inside_mask = __ballot(inside);
  if (lane == 0) s_inside[wave] = inside_mask;
  __syncthreads();
  if (i < nedges && recv != next_recv && static_cast<unsigned>(recv) < static_cast<unsigned>(nnodes)) {
    int e0 = first_occ[recv], e1 = first_occ[nnodes + recv];
    clamp_edge_range(e0, e1, nedges);
    int e;
    if (e1 == i + 1) {  // this is the last edge of the receiver's range, as in every sorted list
      const int64_t group_first = i - threadIdx.x;  // first edge of the workgroup
      e = -1;
      // the node's edges in this workgroup, from this wave down: the highest one inside the cutoff
      for (int w = wave; w >= 0 && e < 0; --w) {
        const int64_t wave_first = group_first + w * kWave;
        if (wave_first + kWave <= e0) break;  // the node's range begins above this wave
        const int hi = w == wave ? lane : kWave - 1;
        const int lo = e0 > wave_first ? static_cast<int>(e0 - wave_first) : 0;
        const unsigned long long upto = hi == kWave - 1 ? ~0ull : (1ull << (hi + 1)) - 1ull;
        const unsigned long long mine = s_inside[w] & upto & ~((1ull << lo) - 1ull);
        if (mine != 0) e = static_cast<int>(wave_first) + (63 - __clzll(static_cast<long long>(mine))) + 1;
      }
      if (e < 0)
        e = e0 >= group_first ? e0
                              : walk_back_to_live_edge(pos, a, b, shifts, rows, nnodes, r_max, e0, static_cast<int>(group_first));
    } else {
      e = walk_back_to_live_edge(pos, a, b, shifts, rows, nnodes, r_max, e0, e1);
    }
    live[recv] = e0;
    live[nnodes + recv] = e;
  }
  if (i < nnodes) {  // a node without edges: an empty range
    const int n = static_cast<int>(i);
    int e0 = first_occ[n], e1 = first_occ[nnodes + n];
    clamp_edge_range(e0, e1, nedges);
    if (e0 >= e1) {
      live[n] = e0;
      live[nnodes + n] = e0;
    }
  }
}

// out[g] = sum of x over the nodes ptr[g] .. ptr[g + 1]: one workgroup per graph, every thread a strided partial sum, a
// tree over the partials: the same order on every run.
constexpr int kSumThreads = 1024;
__global__ __launch_bounds__(kSumThreads) void segment_sum_f64_kernel(const double *__restrict__ x, const double *__restrict__ weights,
                                                                     const int32_t *__restrict__ ptr, double *__restrict__ out,
                                                                     const double *__restrict__ graph_e0, double *__restrict__ total) {
  __shared__ double part[kSumThreads];
  const int lo = ptr[blockIdx.x], hi = ptr[blockIdx.x + 1];
  auto term = [&](int i) { return weights ? weights[i] * x[i] : x[i]; };
  // four strided partial sums per thread, their loads requested together (one sum waits for memory once per element)
  double s0 = 0.0, s1 = 0.0, s2 = 0.0, s3 = 0.0;
  int i = lo + threadIdx.x;
  for (; i + 3 * kSumThreads < hi; i += 4 * kSumThreads) {
    const double t0 = term(i), t1 = term(i + kSumThreads), t2 = term(i + 2 * kSumThreads), t3 = term(i + 3 * kSumThreads);
    s0 += t0, s1 += t1, s2 += t2, s3 += t3;
  }
  for (; i < hi; i += kSumThreads) s0 += term(i);
  part[threadIdx.x] = (s0 + s1) + (s2 + s3);
  __syncthreads();
  for (int d = kSumThreads / 2; d > 0; d >>= 1) {
    if (threadIdx.x < d) part[threadIdx.x] += part[threadIdx.x + d];
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    out[blockIdx.x] = part[0];
    if (total) total[blockIdx.x] = part[0] + (graph_e0 ? graph_e0[blockIdx.x] : 0.0);
  }
}

// Virials from the per-edge gradients the backward chain ends with: under a symmetric strain every edge vector becomes
// vec + vec . strain, so -dE/d strain = 1/2 sum_e (vec_e (x) gv_e + gv_e (x) vec_e) with gv_e = -dE/d vec_e, which is what
// the chain delivers.  Two levels, both in a fixed order: per receiver node (eight lanes share a node's edges), then per
// graph.  node_virial [nnodes, 6]: xx, yy, zz, yz, xz, xy.
__global__ __launch_bounds__(256) void node_virial_kernel(const float *__restrict__ vec, const float *__restrict__ gv,
                                                          const int32_t *__restrict__ first_occ, int nnodes, int64_t nedges,
                                                          double *__restrict__ node_virial) {
  const int64_t t = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  const int n = static_cast<int>(t >> 3), sub = static_cast<int>(t & 7);
  double acc[6] = {0.0, 0.0, 0.0, 0.0, 0.0, 0.0};
  if (n < nnodes) {
    int e0 = first_occ[n], e1 = first_occ[nnodes + n];
    clamp_edge_range(e0, e1, nedges);
    for (int64_t e = e0 + sub; e < e1; e += 8) {
      const double v0 = vec[3 * e + 0], v1 = vec[3 * e + 1], v2 = vec[3 * e + 2];
      const double g0 = gv[3 * e + 0], g1 = gv[3 * e + 1], g2 = gv[3 * e + 2];
      acc[0] += v0 * g0, acc[1] += v1 * g1, acc[2] += v2 * g2;
      acc[3] += 0.5 * (v1 * g2 + v2 * g1), acc[4] += 0.5 * (v0 * g2 + v2 * g0), acc[5] += 0.5 * (v0 * g1 + v1 * g0);
    }
  }
#pragma unroll
  for (int k = 0; k < 6; ++k) {
    acc[k] += __shfl_xor(acc[k], 1);
    acc[k] += __shfl_xor(acc[k], 2);
    acc[k] += __shfl_xor(acc[k], 4);
  }
  if (n < nnodes && sub == 0) {
#pragma unroll
    for (int k = 0; k < 6; ++k) node_virial[6 * static_cast<int64_t>(n) + k] = acc[k];
  }
}

// virials[g] (3 x 3, symmetric) = sum of node_virial over the graph's nodes; one workgroup per graph, strided partial sums
// and a tree over them
__global__ __launch_bounds__(kSumThreads) void graph_virial_kernel(const double *__restrict__ node_virial,
                                                                   const int32_t *__restrict__ ptr, double *__restrict__ virials) {
  __shared__ double part[6][kSumThreads];
  const int lo = ptr[blockIdx.x], hi = ptr[blockIdx.x + 1];
  double s[6] = {0.0, 0.0, 0.0, 0.0, 0.0, 0.0};
  for (int i = lo + threadIdx.x; i < hi; i += kSumThreads) {
#pragma unroll
    for (int k = 0; k < 6; ++k) s[k] += node_virial[6 * static_cast<int64_t>(i) + k];
  }
#pragma unroll
  for (int k = 0; k < 6; ++k) part[k][threadIdx.x] = s[k];
  __syncthreads();
  for (int d = kSumThreads / 2; d > 0; d >>= 1) {
    if (threadIdx.x < d) {
#pragma unroll
      for (int k = 0; k < 6; ++k) part[k][threadIdx.x] += part[k][threadIdx.x + d];
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    double *o = virials + 9 * static_cast<int64_t>(blockIdx.x);
    o[0] = part[0][0], o[4] = part[1][0], o[8] = part[2][0];
    o[5] = o[7] = part[3][0];
    o[2] = o[6] = part[4][0];
    o[1] = o[3] = part[5][0];
  }
}

// A fixed amount of dependent-free fp32 multiply-adds per lane, nothing else: what a box's vector ALUs deliver, for
// telling boxes apart when the step's VALU-bound kernels differ between runs.
__global__ __launch_bounds__(256) void probe_fma_kernel(float *out, int iters) {
  float a[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) a[k] = 1.0f + 0.001f * static_cast<float>(threadIdx.x + k);
  const float m = 0.999f, c = 0.0005f;
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int k = 0; k < 8; ++k) a[k] = fmaf(a[k], m, c);
  }
  float sum = 0.f;
#pragma unroll
  for (int k = 0; k < 8; ++k) sum += a[k];
  if (sum == 123.456f) out[0] = sum;  // never true: keeps the loop
}

inline size_t align256(size_t n) { return (n + 255) & ~static_cast<size_t>(255); }

// Carves the workspace; the same walk sizes it (base == nullptr) and lays it out.
struct Layout {
  float *vec, *gv1, *gv2, *bufM1, *bufM2, *bufA, *edge_scratch;
  float *B1, *h1, *sc, *X2, *B2, *h2, *d_h2, *g1, *gB, *gX2, *gh1a, *gh1;
  int32_t *live;         // [2 N] edge ranges cut back to the last edge inside the cutoff
  double *node_virial;   // [N, 6]
  size_t bytes;

  Layout(void *base, int64_t N, int64_t E, int C) {
    size_t at = 0;
    auto take = [&](size_t n) {
      char *p = base ? static_cast<char *>(base) + at : nullptr;
      at += align256(n);
      return p;
    };
    auto f = [&](int64_t n) { return reinterpret_cast<float *>(take(static_cast<size_t>(n) * sizeof(float))); };
    const int64_t NC = N * C;
    vec = f(3 * E), gv1 = f(3 * E), gv2 = f(3 * E);
    bufM1 = f(16 * NC), bufM2 = f(16 * NC), bufA = f(16 * NC);
    edge_scratch = f(E * C);
    B1 = f(NC), h1 = f(NC), sc = f(NC), X2 = f(NC), B2 = f(NC), h2 = f(NC), d_h2 = f(NC);
    g1 = f(NC), gB = f(NC), gX2 = f(NC), gh1a = f(NC), gh1 = f(NC);
    live = reinterpret_cast<int32_t *>(take(static_cast<size_t>(2 * N) * sizeof(int32_t)));
    node_virial = reinterpret_cast<double *>(take(static_cast<size_t>(6 * N) * sizeof(double)));
    bytes = at;
  }
};

}  // namespace
}  // namespace cm

extern "C" int cm_probe_fma(float *out, int workgroups, int iters, cm_stream_t stream) {
  CM_REQUIRE(out && workgroups > 0 && iters > 0, "cm_probe_fma: NULL output or empty launch");
  hipLaunchKernelGGL(cm::probe_fma_kernel, dim3(static_cast<unsigned>(workgroups)), dim3(256), 0, cm::as_stream(stream), out, iters);
  return cm::check_launch("cm_probe_fma");
}

extern "C" size_t cm_mace_step_workspace(int64_t nnodes, int64_t nedges, int channels) {
  if (nnodes < 0 || nedges < 0 || channels <= 0) return 0;
  return cm::Layout(nullptr, nnodes, nedges, channels).bytes;
}

// Runs one stage; with the stage's timing bit set, between two events recorded on the stream.
#define CM_STAGE(id, call)                          \
  do {                                              \
    cm::StageTimer timer_(st, (id), timing_mask);   \
    const int rc_ = (call);                         \
    if (rc_ != CM_OK) return rc_;                   \
  } while (0)

extern "C" int cm_mace_step_timing(unsigned stage_mask) {
  std::lock_guard<std::mutex> lock(cm::g_timing_mutex);
  cm::g_timing_mask = stage_mask & ((1u << cm::kStages) - 1u);
  for (cm::Pending &p : cm::g_pending) {
    cm::g_event_pool.push_back(p.start);
    cm::g_event_pool.push_back(p.stop);
  }
  cm::g_pending.clear();
  for (int s = 0; s < cm::kStages; ++s) cm::g_stage_ms[s] = 0.0, cm::g_stage_launches[s] = 0;
  return CM_OK;
}

extern "C" int cm_mace_step_timing_read(double *total_ms, int64_t *launches, int capacity) {
  CM_REQUIRE(total_ms && launches && capacity >= cm::kStages, "cm_mace_step_timing_read: need room for %d stages", cm::kStages);
  std::lock_guard<std::mutex> lock(cm::g_timing_mutex);
  for (cm::Pending &p : cm::g_pending) {
    float ms = 0.f;
    if (hipEventSynchronize(p.stop) == hipSuccess && hipEventElapsedTime(&ms, p.start, p.stop) == hipSuccess) {
      cm::g_stage_ms[p.stage] += ms;
      cm::g_stage_launches[p.stage] += 1;
    }
    cm::g_event_pool.push_back(p.start);
    cm::g_event_pool.push_back(p.stop);
  }
  cm::g_pending.clear();
  for (int s = 0; s < cm::kStages; ++s) total_ms[s] = cm::g_stage_ms[s], launches[s] = cm::g_stage_launches[s];
  return cm::kStages;
}

extern "C" int cm_mace_step(const cm_mace_weights *w, const cm_mace_graph *g, const double *positions, const double *shifts,
                            void *workspace, size_t workspace_bytes, double *interaction_energy, double *node_energy,
                            double *forces, double *node_feats, double *virials, double *total_energy, double *total_node_energy,
                            cm_stream_t stream) {
  CM_REQUIRE(w && g, "cm_mace_step: NULL weights or graph");
  const int64_t N = g->nnodes, E = g->nedges;
  const int C = w->channels, ne = w->nelements;
  CM_REQUIRE(N >= 0 && E >= 0 && g->ngraphs >= 1, "cm_mace_step: negative size or no graph");
  CM_REQUIRE(cm_channels_supported(C), "cm_mace_step: channels=%d must be a multiple of 32 in [32, 256]", C);
  CM_REQUIRE(ne >= 1, "cm_mace_step: nelements must be at least 1");
  CM_REQUIRE(interaction_energy && g->graph_ptr, "cm_mace_step: NULL energy output or graph_ptr");
  hipStream_t st = cm::as_stream(stream);
  unsigned timing_mask;
  {
    std::lock_guard<std::mutex> lock(cm::g_timing_mutex);
    timing_mask = cm::g_timing_mask;
  }
  if (timing_mask != 0) {
    // events recorded into a capture cannot be read back: a captured step is not timed
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) timing_mask = 0;
  }
  if (N == 0) {
    hipLaunchKernelGGL(cm::fill_f64_kernel, dim3(1), dim3(64), 0, st, interaction_energy, static_cast<int64_t>(g->ngraphs), 0.0);
    if (virials)
      hipLaunchKernelGGL(cm::fill_f64_kernel, dim3(1), dim3(64), 0, st, virials, static_cast<int64_t>(9) * g->ngraphs, 0.0);
    if (total_energy)
      hipLaunchKernelGGL(cm::copy_or_zero_f64_kernel, dim3(1), dim3(64), 0, st, total_energy, g->graph_e0, static_cast<int64_t>(g->ngraphs));
    return cm::check_launch("cm_mace_step");
  }
  CM_REQUIRE(positions && node_energy && forces, "cm_mace_step: NULL positions or output");
  CM_REQUIRE(N < INT32_MAX / 4 && E < INT32_MAX, "cm_mace_step: sizes out of range");
  CM_REQUIRE(E == 0 || shifts, "cm_mace_step: NULL shifts");
  CM_REQUIRE(g->first_occ && g->sender_offsets && g->elem_perm && g->elem_offsets && g->onehot_perm && g->onehot_offsets && g->X1,
             "cm_mace_step: NULL graph structure");
  CM_REQUIRE(E == 0 || (g->receiver && g->sender && g->sender_perm), "cm_mace_step: NULL edge list");
  for (int t = 0; t < 2; ++t)
    CM_REQUIRE(w->spline[t] && w->mix_WT[t] && w->mix_W[t] && w->T3[t] && w->T2[t] && w->T1[t] && w->prod_WT[t] && w->prod_W[t] &&
                   (w->mono3[t] == nullptr) == (w->mono2[t] == nullptr),
               "cm_mace_step: NULL weight of layer %d", t);
  CM_REQUIRE(w->r_knots && w->up_WT && w->up_W && w->skip_WT && w->skip_W && w->w1 && w->W2a && w->w2b, "cm_mace_step: NULL weight");
  const cm::Layout L(workspace, N, E, C);
  if (workspace == nullptr || workspace_bytes < L.bytes) {
    cm::set_error("cm_mace_step: workspace of %zu bytes, need %zu", workspace_bytes, L.bytes);
    return CM_ENOSPC;
  }
  CM_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0, "cm_mace_step: workspace must be 256-byte aligned");
  const int32_t *oh_perm = g->onehot_perm, *oh_off = g->onehot_offsets;
  const int32_t *el_perm = g->elem_perm, *el_off = g->elem_offsets;
  const float *none = nullptr;

  // ---- forward ----
  if (E > 0) {
    cm::StageTimer timer_(st, 0, timing_mask);
    hipLaunchKernelGGL(cm::geometry_live_range_kernel, dim3(static_cast<unsigned>(cm::ceil_div(std::max(N, E), 256))), dim3(256), 0, st,
                       positions, g->receiver, g->sender, shifts, g->node_rows, g->first_occ, w->r_max, static_cast<int>(N), E, L.vec,
                       L.live, L.gv1, L.gv2);
  }
  const int32_t *fo_live = E > 0 ? L.live : g->first_occ;
  const float *X[2] = {g->X1, L.X2};
  float *bufM[2] = {L.bufM1, L.bufM2};
  float *B[2] = {L.B1, L.B2};
  float *h[2] = {L.h1, L.h2};
  // the three [N, C] products between the layers (and their three transposes in the backward) as one launch each
  const char *glue_env = getenv("CM_STEP_GLUE");  // development switch: smallest node count that takes the chained kernels; -1: none
  const int glue_min = glue_env ? atoi(glue_env) : 0;
  const bool glue = cm_node_glue_supported(C) != 0 && glue_min >= 0 && N >= glue_min;
  for (int t = 0; t < 2; ++t) {
    if (t == 1 && !glue) {
      // residual skip connection per element and linear_up, both of the first layer's output
      CM_STAGE(5, cm_linear(L.h1, w->skip_WT, oh_perm, oh_off, N, ne + 1, 1, 1, C, C, w->skip_scale, none, none, L.sc, stream));
      CM_STAGE(6, cm_linear(L.h1, w->up_WT, nullptr, nullptr, N, 1, 0, 1, C, C, 1.0f, none, none, L.X2, stream));
    }
    CM_STAGE(t == 0 ? 1 : 7, cm_mp_edge_forward(X[t], L.vec, w->r_knots, w->spline[t], w->nknots, w->r_width, w->r_max, g->sender, fo_live, N,
                               E, C, bufM[t], stream));
    if (t == 0)
      CM_STAGE(2, cm_linear(bufM[t], w->mix_WT[t], oh_perm, oh_off, N, ne + 1, 1, 16, C, C, w->mix_scale[t], none, none, L.bufA, stream));
    else
      CM_STAGE(8, cm_linear(bufM[t], w->mix_WT[t], nullptr, nullptr, N, 1, 0, 16, C, C, w->mix_scale[t], none, none, L.bufA, stream));
    // the contraction's gradient table takes the place of the message, which is no longer needed
    CM_STAGE(t == 0 ? 3 : 9, cm_symcon_forward(L.bufA, el_perm, el_off, w->mono3[t], w->n3[t], w->mono2[t], w->n2[t], w->T3[t], w->T2[t], w->T1[t], N,
                              ne, C, B[t], bufM[t], stream));
    if (t == 0 && glue)
      CM_STAGE(4, cm_node_glue_forward(L.B1, w->prod_WT[0], w->skip_WT, w->up_WT, oh_perm, oh_off, N, ne + 1, C, w->skip_scale, L.h1, L.sc,
                                       L.X2, stream));
    else
      CM_STAGE(t == 0 ? 4 : 10, cm_linear(B[t], w->prod_WT[t], nullptr, nullptr, N, 1, 0, 1, C, C, 1.0f, none, t == 1 ? L.sc : none, h[t], stream));
  }
  CM_STAGE(11, cm::readout_forward_with_totals(L.h1, L.h2, w->w1, w->W2a, w->w2b, w->act_cst, w->scale, w->shift, N, C, w->hidden,
                                               node_energy, L.d_h2, node_feats, g->node_rows, g->node_e0, total_node_energy, st));
  if (!glue) {  // with the chained kernels the sums ride in the backward chain's launch
    cm::StageTimer timer_(st, 12, timing_mask);
    hipLaunchKernelGGL(cm::segment_sum_f64_kernel, dim3(g->ngraphs), dim3(cm::kSumThreads), 0, st, node_energy, g->node_weights,
                       g->graph_ptr, interaction_energy, g->graph_e0, total_energy);
  }

  // ---- backward: d(-sum of node energies) / d positions ----
  // The seed is -1 on every node energy (-weight[n] with node weights), so the readouts' backward needs no pass of its
  // own: the gradient with respect to the second layer's features is -d_h2 (the sign goes into the scale of the two
  // linears that consume it, which is exact; node weights scale its rows first), the one with respect to the first
  // layer's is a constant row (times the node's weight).
  if (!glue || g->node_weights) {  // the chained kernel forms the constant rows itself
    cm::StageTimer timer_(st, 13, timing_mask);
    const dim3 grid(static_cast<unsigned>(std::min<int64_t>(cm::ceil_div(N * C, 256), 2048)));
    if (!glue)
      hipLaunchKernelGGL(cm::seed_linear_readout_kernel, grid, dim3(256), 0, st, L.g1, w->w1, w->scale, g->node_weights,
                         static_cast<int64_t>(N) * C, C);
    if (g->node_weights)
      hipLaunchKernelGGL(cm::weight_rows_kernel, grid, dim3(256), 0, st, L.d_h2, g->node_weights, static_cast<int64_t>(N) * C, C);
  }
  // layer 1 (second interaction)
  CM_STAGE(14, cm_linear(L.d_h2, w->prod_W[1], nullptr, nullptr, N, 1, 0, 1, C, C, -1.0f, none, none, L.gB, stream));
  CM_STAGE(15, cm_linear(L.bufM2, w->mix_W[1], nullptr, nullptr, N, 1, 0, 16, C, C, w->mix_scale[1], L.gB, none, L.bufA, stream));
  CM_STAGE(16, cm_mp_edge_backward(L.X2, L.vec, w->r_knots, w->spline[1], w->nknots, w->r_width, w->r_max, L.bufA, g->sender,
                              fo_live, g->sender_perm, g->sender_offsets, N, E, C, L.gX2, L.gv2, L.edge_scratch, stream));
  // layer 0 (first interaction): its input features depend on the species alone, so no gradient with respect to them
  if (glue) {
    CM_STAGE(17, cm::node_glue_backward_with_energy_sums(L.gX2, L.d_h2, w->up_W, w->skip_W, w->prod_W[0], w->w1, w->scale, g->node_weights,
                                                         oh_perm, oh_off, N, ne + 1, C, w->skip_scale, L.gB, node_energy, g->graph_ptr,
                                                         g->ngraphs, interaction_energy, g->graph_e0, total_energy, st));
  } else {
    CM_STAGE(17, cm_linear(L.gX2, w->up_W, nullptr, nullptr, N, 1, 0, 1, C, C, 1.0f, none, L.g1, L.gh1a, stream));
    CM_STAGE(18, cm_linear(L.d_h2, w->skip_W, oh_perm, oh_off, N, ne + 1, 1, 1, C, C, -w->skip_scale, none, L.gh1a, L.gh1, stream));
    CM_STAGE(19, cm_linear(L.gh1, w->prod_W[0], nullptr, nullptr, N, 1, 0, 1, C, C, 1.0f, none, none, L.gB, stream));
  }
  CM_STAGE(20, cm_linear(L.bufM1, w->mix_W[0], oh_perm, oh_off, N, ne + 1, 1, 16, C, C, w->mix_scale[0], L.gB, none, L.bufA, stream));
  // its vector gradient is written onto the second layer's: gv1 = (this layer's) + gv2
  CM_STAGE(21, cm::mp::edge_backward_onto(g->X1, L.vec, w->r_knots, w->spline[0], w->nknots, w->r_width, w->r_max, L.bufA, g->sender,
                                         fo_live, N, E, C, L.gv1, L.gv2, st));
  CM_STAGE(23, cm_edge_geometry_backward(positions, g->receiver, g->sender, shifts, g->node_rows, g->first_occ, g->sender_perm,
                                    g->sender_offsets, L.gv1, nullptr, N, E, forces, nullptr, stream));
  if (virials) {
    cm::StageTimer timer_(st, 24, timing_mask);
    if (N > 0)
      hipLaunchKernelGGL(cm::node_virial_kernel, dim3(static_cast<unsigned>(cm::ceil_div(8 * N, 256))), dim3(256), 0, st, L.vec, L.gv1,
                       g->first_occ, static_cast<int>(N), E, L.node_virial);
    hipLaunchKernelGGL(cm::graph_virial_kernel, dim3(g->ngraphs), dim3(cm::kSumThreads), 0, st, L.node_virial, g->graph_ptr, virials);
  }
  return cm::check_launch("cm_mace_step");
}
