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

__global__ void fill_zero_i32_kernel(int32_t *p, int64_t n) {
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x)
    p[i] = 0;
}

// status[0] = 1 if receiver[e - 1] > receiver[e] anywhere, status[1] = 1 if a value lies outside [0, nnodes); both
// are cleared by the fill launched before this kernel.  Offending threads store the same value: no atomics needed.
__global__ void receiver_list_status_kernel(const int32_t *__restrict__ receiver, int64_t nedges, int nnodes,
                                            int32_t *__restrict__ status) {
  const int64_t e = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  if (e >= nedges) return;
  const int cur = receiver[e];
  if (e > 0 && receiver[e - 1] > cur) status[0] = 1;
  if (cur < 0 || cur >= nnodes) status[1] = 1;
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
  int e0 = first_occ[node];
  int e1 = first_occ[nnodes + node];
  clamp_edge_range(e0, e1, nedges);

  vec acc[16];
#pragma unroll
  for (int m = 0; m < 16; ++m) acc[m] = zerov<vec>();

  for (int base = e0; base < e1; base += kChunk) {
    const int cnt = min(kChunk, e1 - base);
    wave_lds_fence();  // the workgroup is this one wave
    stage_chunk(Y, sender, nedges, base, cnt, lane, sY, sS);
    wave_lds_fence();
    if (active) {
      auto one = [&](int j) {
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
      };
      // Edges in blocks of eight (from 128 channels on), four, two, one per slot: the loads of a block are requested
      // together (8 x 4 rows of R in flight per wave keep the stream at 5.9 TB/s where 2 x 4 give 5.5), and a node's
      // last edges take the largest block that still fits instead of one edge at a time.  A block's rows and the 16
      // accumulators have to fit the register file: 5 V and 16 V registers for V channels per lane, so five channels
      // per lane (160 channels) stop at blocks of four and seven (224 channels) at blocks of two.
      int j = slot;
      if constexpr (C >= 128 && K::V <= 4) {
        for (; j + 7 * K::EPW < cnt; j += 8 * K::EPW) {
#pragma unroll
          for (int u = 0; u < 8; ++u) one(j + u * K::EPW);
        }
      }
      if constexpr (K::V <= 5) {
        for (; j + 3 * K::EPW < cnt; j += 4 * K::EPW) {
#pragma unroll
          for (int u = 0; u < 4; ++u) one(j + u * K::EPW);
        }
      }
      for (; j + K::EPW < cnt; j += 2 * K::EPW) {
        one(j);
        one(j + K::EPW);
      }
      if (j < cnt) one(j);
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
// LIVE: 0 = every row of gXe is read; 1 / 2 = only rows of edges within r_max, by the edge vector / the edge length
// (the spline-fused edge pass writes no others).
//
// A slot (the lanes that carry one row) takes four edges per iteration.  Three loads depend on each other per edge --
// its index from the sender-sorted view, its vector or length (LIVE), its row -- so the loop is pipelined over
// iterations: iteration i issues the rows of batch i, the vectors of batch i + 1 and the indices of batch i + 2
// together and uses what iteration i - 1 issued: one memory latency per iteration instead of three.  Every load is
// unconditional: an edge that is not to be read (beyond the list's end, beyond the cutoff, out of range) loads the row
// of the slot's last good edge again, a cache hit, and its value is dropped by a select.  The loads are issued from
// inline assembly and waited for once per iteration by an explicit wait at the end of the iteration that issued them,
// with the loaded registers passed through the waiting statement so that no use can move above it and every value that
// crosses the loop's back edge has arrived: left to itself the compiler sinks each load to its first use in
// the next iteration and waits for it there, which puts the three latencies back in a row.  Registers that are still
// being loaded are never copied (the build scans the generated code of this kernel for any instruction that touches
// a register between the load issued into it and the wait); the batches change roles after the wait.  The summation
// order is fixed.
__device__ __forceinline__ void issue_load(int &dst, const int32_t *p) {
  asm volatile("global_load_dword %0, %1, off" : "=v"(dst) : "v"(p) : "memory");
}
__device__ __forceinline__ void issue_load(float &dst, const float *p) {
  asm volatile("global_load_dword %0, %1, off" : "=v"(dst) : "v"(p) : "memory");
}
__device__ __forceinline__ void issue_load(f3 &dst, const float *p) {
  asm volatile("global_load_dwordx3 %0, %1, off" : "=v"(dst) : "v"(p) : "memory");
}
__device__ __forceinline__ void issue_load_stream(float &dst, const float *p) {
  asm volatile("global_load_dword %0, %1, off nt" : "=v"(dst) : "v"(p) : "memory");
}
__device__ __forceinline__ void issue_load_stream(f4 &dst, const float *p) {
  asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(dst) : "v"(p) : "memory");
}
// Marks the point from which a register that a hand-issued load lands in holds the loaded value; the comment it leaves
// in the assembly is read by the build's scan of the generated code (see the head of the sender kernel).
template <class T>
__device__ __forceinline__ void arrived(T &v) {
  asm volatile("; landed %0" : "+v"(v));
}

//
// MULTI (few senders, see parts_for): a workgroup of up to eight waves per sender, each on a part of the sender's range;
// the parts' sums are added by the first wave in the order of the parts.
template <int C, int LIVE, bool MULTI>
__global__ __launch_bounds__(MULTI ? 8 * kWave : kWave) void mp_backward_sender_kernel(
    const float *__restrict__ gXe, const int32_t *__restrict__ perm,
    const int32_t *__restrict__ offsets, int nnodes, int64_t nedges, const float *__restrict__ live_by, float r_max,
    float *__restrict__ gX) {
  using K = Cfg<C, false, true>;  // a pure row stream: 16 bytes per lane at every channel count
  using vec = typename K::vec;
  constexpr int B = 4;            // edges per slot and iteration
  constexpr int STEP = B * K::EPW;
  __shared__ __attribute__((aligned(16))) float comb[MULTI ? 7 * C : 1];
  const int node = blockIdx.x;
  const int lane = threadIdx.x % kWave;
  const int wave = MULTI ? threadIdx.x / kWave : 0;
  const int parts = MULTI ? blockDim.x / kWave : 1;
  const int slot = lane / K::SW;
  const int cl = lane % K::SW;
  const bool active = cl < K::LPE;
  int k0 = offsets[node];
  int k1 = offsets[node + 1];
  if (MULTI) {
    const int64_t len = k1 - k0;
    const int lo = k0 + static_cast<int>(len * wave / parts);
    k1 = k0 + static_cast<int>(len * (wave + 1) / parts);
    k0 = lo;
  }
  vec acc = zerov<vec>();
  if (active && k0 < k1 && nedges > 0) {
    const int klast = k1 - 1;
    const int emax = static_cast<int>(nedges - 1);
    int e_cur[B], e_nxt[B], e_aft[B];   // indices of batches i, i + 1 (arrived) and i + 2 (being loaded)
    f3 lv_cur[B], lv_nxt[B];    // LIVE 1: vectors of batch i (arrived) and i + 1 (being loaded)
    float lr_cur[B], lr_nxt[B];  // LIVE 2: lengths of the same
    f4 rows4[B];                        // rows of the previous batch (four channels per lane: one 16-byte load)
    float rowsf[B][K::V];               // the same for the other channel counts per lane (dword loads)
    bool take[B];
    auto issue_indices = [&](int kk, int (&e)[B]) {
#pragma unroll
      for (int j = 0; j < B; ++j) issue_load(e[j], perm + min(kk + j * K::EPW, klast));
    };
    auto issue_live = [&](const int (&e)[B]) {  // into lv_nxt / lr_nxt
      if constexpr (LIVE != 0) {
#pragma unroll
        for (int j = 0; j < B; ++j) {
          const int ec = min(max(e[j], 0), emax);
          if constexpr (LIVE == 1) issue_load(lv_nxt[j], live_by + 3 * static_cast<int64_t>(ec));
          else issue_load(lr_nxt[j], live_by + ec);
        }
      }
    };
    auto issue_rows = [&](const int (&e)[B]) {
#pragma unroll
      for (int j = 0; j < B; ++j) {
        const float *p = gXe + static_cast<int64_t>(e[j]) * C + K::off(cl);
        if constexpr (K::V == 4) {
          issue_load_stream(rows4[j], p);
        } else {
#pragma unroll
          for (int q = 0; q < K::V; ++q) issue_load_stream(rowsf[j][q], p + q * K::ES);
        }
      }
    };
    auto wait_all = [&](auto &...regs) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      (arrived(regs), ...);
    };
    auto arrived_rows = [&]() {
#pragma unroll
      for (int j = 0; j < B; ++j) {
        if constexpr (K::V == 4) {
          arrived(rows4[j]);
        } else {
#pragma unroll
          for (int q = 0; q < K::V; ++q) arrived(rowsf[j][q]);
        }
      }
    };
    auto row = [&](int j) -> vec {  // the row if it is to be taken, zeros otherwise
      vec r;
      if constexpr (K::V == 4) {
        r = rows4[j];
      } else {
#pragma unroll
        for (int q = 0; q < K::V; ++q) r[q] = rowsf[j][q];
      }
      return take[j] ? r : zerov<vec>();
    };

    auto wait_for_everything = [&]() {
      // One wait for all that is in flight; every register a load was issued into passes through this point, so that
      // whatever the compiler does with it afterwards (a copy across the loop's back edge included) sees the loaded value.
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      arrived_rows();
#pragma unroll
      for (int j = 0; j < B; ++j) {
        arrived(e_aft[j]);
        if constexpr (LIVE == 1) arrived(lv_nxt[j]);
        if constexpr (LIVE == 2) arrived(lr_nxt[j]);
      }
    };

    int k = k0 + slot;
    // prologue: indices of batches 0 and 1, then the vectors of batch 0
    issue_indices(k, e_cur);
    issue_indices(k + STEP, e_aft);
    wait_all(e_cur[0], e_cur[1], e_cur[2], e_cur[3], e_aft[0], e_aft[1], e_aft[2], e_aft[3]);
    int good = min(max(e_cur[0], 0), emax);  // a row that may always be read
#pragma unroll
    for (int j = 0; j < B; ++j) {
      rows4[j] = zero4();
#pragma unroll
      for (int q = 0; q < K::V; ++q) rowsf[j][q] = 0.f;
      take[j] = false;
      e_nxt[j] = e_cur[j];  // the loop head finds batch 0 in e_nxt / lv_nxt and batch 1 in e_aft
    }
    issue_live(e_nxt);  // lands in lv_nxt / lr_nxt: the loop's first act is to move it to the current set
    wait_for_everything();
    for (; k < k1; k += STEP) {
      // everything has arrived: rows of the previous batch, vectors of this one, indices of the next one
      acc += (row(0) + row(1)) + (row(2) + row(3));
#pragma unroll
      for (int j = 0; j < B; ++j) {
        e_cur[j] = e_nxt[j];
        e_nxt[j] = e_aft[j];
        if constexpr (LIVE == 1) lv_cur[j] = lv_nxt[j];
        if constexpr (LIVE == 2) lr_cur[j] = lr_nxt[j];
      }
#pragma unroll
      for (int j = 0; j < B; ++j) {
        bool ok = (k + j * K::EPW < k1) & (static_cast<unsigned>(e_cur[j]) <= static_cast<unsigned>(emax));
        if constexpr (LIVE == 1) ok = ok & (edge_length(lv_cur[j].x, lv_cur[j].y, lv_cur[j].z) <= r_max);
        if constexpr (LIVE == 2) ok = ok & (lr_cur[j] <= r_max);
        take[j] = ok;
        good = ok ? e_cur[j] : good;
        e_cur[j] = ok ? e_cur[j] : good;
      }
      // issue: rows of this batch, vectors of the next, indices of the one after; then the iteration's one wait
      issue_rows(e_cur);
      issue_live(e_nxt);
      issue_indices(k + 2 * STEP, e_aft);
      wait_for_everything();
    }
    acc += (row(0) + row(1)) + (row(2) + row(3));
  }
#pragma unroll
  for (int off = kWave / 2; off >= K::SW; off >>= 1) acc += shfl_downv(acc, off);
  if (MULTI) {
    if (wave > 0 && slot == 0 && active) K::st(comb + (wave - 1) * C + K::off(cl), acc);
    __syncthreads();
    if (wave > 0) return;
    if (slot == 0 && active)
      for (int w = 1; w < parts; ++w) acc += K::ld(comb + (w - 1) * C + K::off(cl));
  }
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
                  float *gX, hipStream_t st, const float *live_vec, const float *live_r, float r_max) {
  const int parts = parts_for(nnodes, nedges);
  const dim3 grid(static_cast<unsigned>(nnodes)), block(parts * kWave);
#define CM_SENDER(LIVE_, by_, rmax_)                                                                                                   \
  do {                                                                                                                                 \
    if (parts > 1)                                                                                                                     \
      hipLaunchKernelGGL((mp_backward_sender_kernel<C, LIVE_, true>), grid, block, 0, st, gXe, perm, offsets, static_cast<int>(nnodes), \
                         nedges, by_, rmax_, gX);                                                                                      \
    else                                                                                                                               \
      hipLaunchKernelGGL((mp_backward_sender_kernel<C, LIVE_, false>), grid, block, 0, st, gXe, perm, offsets,                         \
                         static_cast<int>(nnodes), nedges, by_, rmax_, gX);                                                            \
  } while (0)
  if (live_vec)
    CM_SENDER(1, live_vec, r_max);
  else if (live_r)
    CM_SENDER(2, live_r, r_max);
  else
    CM_SENDER(0, static_cast<const float *>(nullptr), 0.f);
#undef CM_SENDER
  return check_launch("cm_mp_backward (sender pass)");
}

}  // namespace

int mp::launch_sender_pass(int channels, const float *gXe, const int32_t *perm, const int32_t *offsets, int64_t nnodes,
                           int64_t nedges, float *gX, hipStream_t st, const float *live_vec, const float *live_r,
                           float r_max) {
  int rc = CM_EINVAL;
  CM_DISPATCH_C(channels, rc = launch_sender<C_>(gXe, perm, offsets, nnodes, nedges, gX, st, live_vec, live_r, r_max));
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
  // a list that is not sorted leaves entries unwritten: they then read 0, an empty range, instead of what the buffer held
  hipLaunchKernelGGL(cm::fill_zero_i32_kernel, dim3(static_cast<unsigned>(std::min<int64_t>(cm::ceil_div(2 * nnodes, block), 1024))),
                     dim3(block), 0, cm::as_stream(stream), first_occ, 2 * nnodes);
  hipLaunchKernelGGL(cm::first_occurences_kernel, dim3(grid), dim3(block), 0, cm::as_stream(stream), receiver,
                     static_cast<int>(nedges), static_cast<int>(nnodes), first_occ);
  return cm::check_launch("cm_first_occurences");
}

extern "C" int cm_receiver_list_status(const int32_t *receiver, int64_t nedges, int64_t nnodes, int32_t *status,
                                       cm_stream_t stream) {
  CM_REQUIRE(nedges >= 0 && nnodes >= 0, "cm_receiver_list_status: negative size");
  CM_REQUIRE(nedges < INT32_MAX && nnodes < INT32_MAX / 2, "cm_receiver_list_status: sizes exceed int32 indexing");
  CM_REQUIRE(status != nullptr, "cm_receiver_list_status: status is NULL");
  CM_REQUIRE(nedges == 0 || receiver != nullptr, "cm_receiver_list_status: receiver is NULL");
  hipLaunchKernelGGL(cm::fill_zero_i32_kernel, dim3(1), dim3(64), 0, cm::as_stream(stream), status, 2);
  if (nedges > 0)
    hipLaunchKernelGGL(cm::receiver_list_status_kernel, dim3(static_cast<unsigned>(cm::ceil_div(nedges, 256))), dim3(256), 0,
                       cm::as_stream(stream), receiver, nedges, static_cast<int>(nnodes), status);
  return cm::check_launch("cm_receiver_list_status");
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
