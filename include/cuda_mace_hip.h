/*
 * C ABI of libcuda_mace_hip.so: the invariant-MACE hot path as hand-written HIP kernels for
 * gfx950 (MI355X).  Plain pointers and sizes only; every pointer is DEVICE memory unless a
 * comment says otherwise; every tensor is contiguous row-major fp32 / int32.  Each entry point
 * enqueues its kernels on `stream` (a hipStream_t passed as void*, NULL = the default stream),
 * returns without synchronising, and returns 0 on success or a negative CM_E* code after
 * storing a message retrievable with cm_last_error().  Argument checking happens on the host
 * before anything is launched; no entry point allocates or frees device memory.
 *
 * The reference exposes this path as TorchScript custom classes whose C++ launchers are the
 * jit_* free functions cited below (paths relative to the reference tree); each entry point
 * here replaces the launcher + kernel pair named in its comment.
 */
#ifndef CUDA_MACE_HIP_H
#define CUDA_MACE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CM_OK 0
#define CM_EINVAL (-22)   /* bad shape / null pointer / unsupported channel count */
#define CM_ELAUNCH (-5)   /* the HIP runtime refused a launch */
#define CM_ENOSPC (-28)   /* caller's workspace too small */

typedef void *cm_stream_t;

/* ABI version, bumped on any signature change. */
int cm_abi_version(void);
/* Message of the calling thread's most recent failure ("" if none). Host pointer, do not free. */
const char *cm_last_error(void);
/* 1 if `channels` is a supported feature width (multiple of 32, 32..256), else 0. */
int cm_channels_supported(int channels);

/* ---------------------------------------------------------------------------------------------
 * Profiler ranges.  The reference opens an NVTX range named "cuda_mace" around every autograd forward and backward
 * (PUSH_RANGE / POP_RANGE, include/utils.h:9-21; e.g. src/linear.cpp:15, :24).  Here the ranges are ROCTx ranges,
 * emitted only when the environment variable CUDA_MACE_TRACE is set to a non-zero value at the first call; the
 * marker library is looked up at run time.  cm_trace_push / cm_trace_pop do nothing otherwise.
 */
int cm_trace_enabled(void);
void cm_trace_push(const char *name);
void cm_trace_pop(void);

/* ---------------------------------------------------------------------------------------------
 * CSR offsets of a non-decreasing receiver list.
 * Replaces jit_calculate_first_occurences (jit_wrappers/src/invariant_message_passing_wrapper.cpp:19-70)
 * and calculate_first_occurences_kernel_ptr (cuda/src/invariant_message_passing_impl.cu:8-72).
 *   receiver   int32 [nedges], non-decreasing, values in [0, nnodes)
 *   first_occ  int32 [2 * nnodes]: [n] = first edge of node n, [nnodes + n] = one past its last.
 * Nodes without edges get start == end == insertion point (the reference leaves them undefined).
 */
int cm_first_occurences(const int32_t *receiver, int64_t nedges, int64_t nnodes,
                        int32_t *first_occ, cm_stream_t stream);
/* Checks what cm_first_occurences assumes of its input (the reference does not check it either: an unsorted list
 * silently gives wrong sums there, jit_wrappers/src/invariant_message_passing_wrapper.cpp:19-70).
 *   status int32 [2] (device): [0] = 1 if the list decreases somewhere, [1] = 1 if a value lies outside [0, nnodes).
 * cm_first_occurences itself clamps out-of-range values and gives empty ranges to nodes an unsorted list skips, and
 * every kernel that reads first_occ forces the ranges into [0, nedges], so a bad list gives wrong sums, never an
 * access outside the edge arrays.  The Python binding runs this check when CUDA_MACE_DEBUG is set. */
int cm_receiver_list_status(const int32_t *receiver, int64_t nedges, int64_t nnodes, int32_t *status,
                            cm_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Stable counting sort of item indices by key: perm lists items by non-decreasing key, ties in
 * original order; offsets[k] = number of items with key < k (offsets has nkeys + 1 entries).
 * Used for the sender-sorted view of the edge list, which takes the place of the reference's
 * N x N reverse-edge table (jit_wrappers/src/invariant_message_passing_wrapper.cpp:91-93;
 * cuda/src/invariant_message_passing_impl.cu:112-116, 331-336), and for grouping nodes by
 * element, which takes the place of the per-element torch::where + host sync in
 * jit_elemental_linear (jit_wrappers/src/linear_wrapper.cpp:137-145).
 *   keys int32 [n] in [0, nkeys); perm int32 [n]; offsets int32 [nkeys + 1];
 *   workspace: cm_stable_key_sort_workspace(n, nkeys) bytes of device memory.
 * Cost: linear in n up to 64 keys (any bucket size).  Above 64 keys the items of a bucket are ranked by comparing
 * them with each other, so the cost also grows with the square of the largest bucket: meant for neighbour lists,
 * where a bucket is one atom's edges (tens of items; 1.3 million edges over 25 000 senders take 0.1 ms), not for
 * keys that put a large part of the items into one bucket (430 000 of 1.7 million items in one bucket: 25 ms).
 */
size_t cm_stable_key_sort_workspace(int64_t n, int64_t nkeys);
int cm_stable_key_sort(const int32_t *keys, int64_t n, int64_t nkeys, int32_t *perm,
                       int32_t *offsets, void *workspace, size_t workspace_bytes,
                       cm_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * cm_stable_key_sort without a workspace argument, for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * Same operands and result as cm_stable_key_sort; the counters, cursors and bucketed item list live in a buffer of
 * cm_stable_key_sort_static_capacity() bytes (32 MiB) that is part of the library image on every GPU, so the call
 * allocates nothing.  It returns CM_ENOSPC when cm_stable_key_sort_workspace(n, nkeys) = 4 * (n + 2 * nkeys) bytes
 * (rounded up to 256) exceeds that capacity.  All calls on one GPU share that GPU's buffer: calls that may overlap
 * on one GPU (different streams, different threads) race and must be serialised by the caller.
 * The first use on a GPU looks the buffer's address up (a runtime query, not to be made while a stream is capturing):
 * before a capture, call cm_stable_key_sort_static_capacity() with that GPU current (it performs the lookup) or make
 * one sort call; after that a call enqueues kernels only and can be recorded into a HIP graph.
 */
size_t cm_stable_key_sort_static_capacity(void);
int cm_stable_key_sort_static(const int32_t *keys, int64_t n, int64_t nkeys, int32_t *perm,
                              int32_t *offsets, cm_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Invariant message passing, forward.
 * Replaces jit_forward_message_passing (jit_wrappers/src/invariant_message_passing_wrapper.cpp:72-155)
 * and inv_tp_kernel_ptr (cuda/src/invariant_message_passing_impl.cu:74-165).
 *   out[n, m, c] = sum_{e in [first_occ[n], first_occ[nnodes + n])} X[sender[e], c] * Y[m, e] * R[e, l(m), c]
 *   X [nnodes, channels]; Y [16, nedges]; R [nedges, 4, channels]; sender int32 [nedges];
 *   first_occ from cm_first_occurences; out [nnodes, 16, channels] (rows of edgeless nodes = 0).
 * No N x N side table is produced.
 */
int cm_mp_forward(const float *X, const float *Y, const float *R, const int32_t *sender,
                  const int32_t *first_occ, int64_t nnodes, int64_t nedges, int channels,
                  float *out, cm_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Invariant message passing, backward.
 * Replaces jit_backward_message_passing (jit_wrappers/src/invariant_message_passing_wrapper.cpp:157-284),
 * backward_edge_inv_tp_kernel_ptr (cuda/src/invariant_message_passing_impl.cu:167-294) and
 * backward_node_inv_tp_kernel_ptr (:296-399).
 *   grad_out [nnodes, 16, channels]
 *   gY [16, nedges]           (may be NULL: not computed)
 *   gR [nedges, 4, channels]  (may be NULL: not computed)
 *   gX [nnodes, channels]     (may be NULL: not computed).  When gX is wanted the caller also
 *      passes the sender-sorted view (sender_perm [nedges], sender_offsets [nnodes + 1] from
 *      cm_stable_key_sort(sender, nedges, nnodes, ...)) and edge_scratch, fp32
 *      [nedges, channels], which receives the per-edge contributions that the second kernel
 *      sums per sender.  Works for any directed multigraph.
 */
int cm_mp_backward(const float *X, const float *Y, const float *R, const float *grad_out,
                   const int32_t *sender, const int32_t *first_occ, const int32_t *sender_perm,
                   const int32_t *sender_offsets, int64_t nnodes, int64_t nedges, int channels,
                   float *gX, float *gY, float *gR, float *edge_scratch, cm_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Invariant message passing with one radial weight per component instead of one per degree:
 *   out[n, m, c] = sum_{e -> n} X[sender[e], c] * Y[m, e] * R[e, m, c],     R [nedges, 16, channels]
 * The reference's kernels index the weight of component m as radial[edge * 4 * C + floor(sqrt(m)) * C + c]
 * (cuda/src/invariant_message_passing_impl.cu:138, :246-262, :365-371); these two entry points are cm_mp_forward /
 * cm_mp_backward for callers that hold a weight per component (gR is then [nedges, 16, channels]); every other
 * operand, the NULL conventions and the sender-sorted view are the same.
 */
int cm_mp_forward_per_m(const float *X, const float *Y, const float *R, const int32_t *sender,
                        const int32_t *first_occ, int64_t nnodes, int64_t nedges, int channels, float *out,
                        cm_stream_t stream);
int cm_mp_backward_per_m(const float *X, const float *Y, const float *R, const float *grad_out, const int32_t *sender,
                         const int32_t *first_occ, const int32_t *sender_perm, const int32_t *sender_offsets,
                         int64_t nnodes, int64_t nedges, int channels, float *gX, float *gY, float *gR,
                         float *edge_scratch, cm_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Message passing with the radial weights evaluated in-kernel from the cubic-spline table:
 *   out[n, m, c] = sum_{e -> n} X[sender[e], c] * Y[m, e] * R(r[e])[l(m) * channels + c]
 * with R(r) exactly what cm_spline_forward computes (coeffs [nknots - 1, 4, 4 * channels], zero beyond
 * r_max).  It fuses the reference's CubicSpline call and its InvariantMessagePassingTP call
 * (models/InvariantMACE.py:320 and :105-112; kernels cuda/src/cubic_spline_impl.cu:5-107 and
 * cuda/src/invariant_message_passing_impl.cu:74-399) so that R[nedges, 4, channels], dR/dr and grad_R are
 * never written to or read from HBM.  The backward returns grad_r[e] = sum_j grad_R[e, j] * dR/dr[e, j]
 * directly (may be NULL), next to gY and gX as in cm_mp_backward.
 * Edges with r[e] > r_max (the skin of a Verlet list) and edges whose sender index is out of range contribute nothing
 * and get zero gradients; their rows of edge_scratch are neither written nor read.
 */
int cm_mp_spline_forward(const float *X, const float *Y, const float *r, const float *r_knots,
                         const float *coeffs, int nknots, float r_width, float r_max,
                         const int32_t *sender, const int32_t *first_occ, int64_t nnodes,
                         int64_t nedges, int channels, float *out, cm_stream_t stream);
int cm_mp_spline_backward(const float *X, const float *Y, const float *r, const float *r_knots,
                          const float *coeffs, int nknots, float r_width, float r_max,
                          const float *grad_out, const int32_t *sender, const int32_t *first_occ,
                          const int32_t *sender_perm, const int32_t *sender_offsets, int64_t nnodes,
                          int64_t nedges, int channels, float *gX, float *gY, float *grad_r,
                          float *edge_scratch, cm_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Message passing straight from the edge vectors: the 16 harmonics (cm_sh_forward's) and the length are computed per
 * edge inside the kernels next to the radial spline, i.e. cm_mp_spline_forward with Y = SH(vectors), r = |vectors|.
 * Fuses the reference's SphericalHarmonics, CubicSpline and InvariantMessagePassingTP calls
 * (models/InvariantMACE.py:306, 320, 105-112); Y[16, nedges], grad_Y and grad_r never exist.
 *   vectors fp32 [nedges, 3].  Backward: grad_vectors fp32 [nedges, 3] (may be NULL) is the full gradient with respect
 *   to the edge vector, harmonics Jacobian and radial part included; gX as in cm_mp_backward.
 */
int cm_mp_edge_forward(const float *X, const float *vectors, const float *r_knots, const float *coeffs,
                       int nknots, float r_width, float r_max, const int32_t *sender,
                       const int32_t *first_occ, int64_t nnodes, int64_t nedges, int channels,
                       float *out, cm_stream_t stream);
int cm_mp_edge_backward(const float *X, const float *vectors, const float *r_knots, const float *coeffs,
                        int nknots, float r_width, float r_max, const float *grad_out,
                        const int32_t *sender, const int32_t *first_occ, const int32_t *sender_perm,
                        const int32_t *sender_offsets, int64_t nnodes, int64_t nedges, int channels,
                        float *gX, float *grad_vectors, float *edge_scratch, cm_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Real spherical harmonics l <= 3 of normalised edge vectors, sqrt(4 pi) ("component")
 * normalisation, input axes permuted as (x, y, z) = (in[2], in[0], in[1]).
 * Replaces jit_spherical_harmonics / jit_spherical_harmonics_backward
 * (jit_wrappers/src/spherical_harmonics_wrapper.cpp:15-83, 85-137) and
 * spherical_harmonics_kernel_ptr / spherical_harmonics_backward_kernel_ptr
 * (cuda/src/spherical_harmonics_impl.cu:21-282, 284-334).
 *   xyz [nedges, 3] -> Y [16, nedges];  backward: grad_Y [16, nedges] -> grad_xyz [nedges, 3]
 * The backward recomputes the Jacobian from xyz instead of reading a stored [16, 3, nedges] one.
 */
int cm_sh_forward(const float *xyz, int64_t nedges, float *Y, cm_stream_t stream);
int cm_sh_backward(const float *xyz, const float *grad_Y, int64_t nedges, float *grad_xyz,
                   cm_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Edge vectors and lengths from positions, and the scatter of per-edge gradients back to atoms.
 * Replaces the upstream helper the reference model calls at models/InvariantMACE.py:297-301
 * (get_edge_vectors_and_lengths, positions[edge_index[1]] - positions[edge_index[0]] + shifts, evaluated
 * there by generic indexing kernels whose backward is a sort-based index_put) and the casts at :303-304, :320.
 *   positions fp64 [nnodes, 3]; row_a = edge_index[0] (non-decreasing), row_b = edge_index[1], int32 [nedges];
 *   shifts fp64 [nedges, 3] -> vectors fp32 [nedges, 3] = pos[row_b] - pos[row_a] + shifts (computed in
 *   fp64, rounded once), lengths fp32 [nedges].
 * Backward: g = grad_vectors + grad_lengths * vec / |vec| per edge (either gradient may be NULL);
 *   grad_positions[n] = sum_{e: row_b[e] = n} g - sum_{e: row_a[e] = n} g   (fp64 [nnodes, 3], may be NULL)
 *   grad_shifts[e] = g                                                     (fp64 [nedges, 3], may be NULL)
 *   a_first_occ = cm_first_occurences(row_a); b_perm / b_offsets = cm_stable_key_sort(row_b, nedges, nnodes).
 *   node_rows int32 [nnodes] or NULL: when given, atom n of the edge lists is row node_rows[n] of positions and of
 *   grad_positions (a permutation), so a caller that relabels its atoms keeps positions and forces in its own order.
 */
int cm_edge_geometry_forward(const double *positions, const int32_t *row_a, const int32_t *row_b,
                             const double *shifts, const int32_t *node_rows, int64_t nnodes, int64_t nedges,
                             float *vectors, float *lengths, cm_stream_t stream);
int cm_edge_geometry_backward(const double *positions, const int32_t *row_a, const int32_t *row_b,
                              const double *shifts, const int32_t *node_rows, const int32_t *a_first_occ,
                              const int32_t *b_perm, const int32_t *b_offsets, const float *grad_vectors,
                              const float *grad_lengths, int64_t nnodes, int64_t nedges,
                              double *grad_positions, double *grad_shifts, cm_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Tabulated radial functions: natural cubic spline, R[e, j] = a + b x + c x^2 + d x^3 with
 * x = r[e] - r_knots[idx], idx = clamp(int(r[e] / r_width), 0, nknots - 2); zero when r[e] > r_max.
 * Replaces jit_evaluate_spline / jit_backward_spline (jit_wrappers/src/cubic_spline_wrapper.cpp:14-97,
 * 99-153) and evaluate_spline_kernel_ptr / backward_spline_kernel_ptr
 * (cuda/src/cubic_spline_impl.cu:5-66, 68-107).
 *   r [nedges]; r_knots [nknots]; coeffs [nknots - 1, 4, noutputs]; R_out [nedges, noutputs];
 *   R_deriv [nedges, noutputs] or NULL.  noutputs must be a multiple of 4.
 * Backward: grad_r[e] = sum_j grad_R[e, j] * dR/dr[e, j], with dR/dr recomputed from the table.
 */
int cm_spline_forward(const float *r, const float *r_knots, const float *coeffs, int64_t nedges,
                      int nknots, int noutputs, float r_width, float r_max, float *R_out,
                      float *R_deriv, cm_stream_t stream);
int cm_spline_backward(const float *r, const float *r_knots, const float *coeffs,
                       const float *grad_R, int64_t nedges, int nknots, int noutputs,
                       float r_width, float r_max, float *grad_r, cm_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Channel-mixing linear layers on fp32 MFMA: OUT[n, m, :] = scale * X[n, m, :] . W[g(n)][l(m)].
 * The reference hard-codes scale = 1/sqrt(K) (cuda/src/linear_impl.cu:33), also in the backward, where
 * that is the true gradient only for square layers; here the caller passes the factor.
 * Replaces jit_linear and jit_elemental_linear (jit_wrappers/src/linear_wrapper.cpp:23-95, 97-191) and
 * linear_kernel_ptr / elemental_linear_kernel_ptr (cuda/src/linear_impl.cu:16-133, 134-255).
 *   X [nnodes, ncomp, K]; OUT [nnodes, ncomp, Nout]; ncomp = 16 (l(m) = floor(sqrt(m)), four weight blocks per
 *   group) or ncomp = 1 (scalar features, one weight block per group: the reference leaves that case to
 *   torch.matmul / the upstream e3nn tensor product, models/InvariantMACE.py:41-53, 133, 149).
 *   W_T [ngroups, 4 or 1, Nout, K]: the TRANSPOSED weight blocks, W_T[g][l][j][k] = W[g][l][k][j].  The
 *   reference keeps both W and W_T as module buffers (ops/linear.py:47-51); the forward passes its
 *   weights_transposed buffer here and the backward with respect to X passes its weights buffer.
 *   Plain linear: ngroups = 1, node_perm = group_offsets = NULL.
 *   Per-element linear: node_perm int32 [nnodes] lists nodes grouped by element and
 *   group_offsets int32 [ngroups + 1] delimits the groups (cm_stable_key_sort on the element
 *   index); rows of nodes that are in no group are not written.  With zero_last_group != 0 the last of the
 *   ngroups groups has no weights (W_T holds ngroups - 1 groups) and its rows are written as zeros: that is
 *   where nodes whose one-hot row names no element go.
 *   K and Nout: multiples of 32 in [32, 256].
 *   row_scale fp32 [nnodes, K] or NULL: when given, X[n, m, k] is multiplied by row_scale[n, k] as it is read.
 *   That is the backward of the symmetric contraction (gX[n, m, k] = grad_out[n, k] * grad[n, m, k],
 *   cuda/src/symmetric_contraction_impl.cu:198-234) folded into the backward of the linear layer that precedes
 *   the contraction: pass grad as X and grad_out as row_scale, and no [nnodes, 16, K] product is written.
 *   residual fp32 [nnodes, ncomp, Nout] or NULL: when given, it is added to the written rows (OUT = scale X W +
 *   residual; the model's "linear of the product plus skip connection", models/InvariantMACE.py:41-53 followed by the
 *   product block's addition of sc, in one pass).  residual may be OUT itself (in-place accumulation).
 */
int cm_linear(const float *X, const float *W_T, const int32_t *node_perm,
              const int32_t *group_offsets, int64_t nnodes, int ngroups, int zero_last_group,
              int ncomp, int K, int Nout, float scale, const float *row_scale, const float *residual,
              float *OUT, cm_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Symmetric contraction, correlation 3, scalar (L = 0) output, with its analytic gradient.
 * Replaces jit_symmetric_contraction_forward / _backward
 * (jit_wrappers/src/symmetric_contraction_wrapper.cpp:15-156, 158-205) and
 * symmetric_contraction_kernel / symm_contraction_backward_kernel
 * (cuda/src/symmetric_contraction_impl.cu:6-196, 198-234).
 *
 * The cubic form is evaluated over monomials x_i x_j x_k, i <= j <= k:
 *   out[n, c] = sum_t T3[e, t, c] x_i(t) x_j(t) x_k(t) + sum_q T2[e, q, c] x_i(q) x_j(q)
 *             + T1[e, c] x_0,     e = atom_types[n], x_i = X[n, i, c]
 * cm_symcon_tables builds T3/T2/T1 on the device from the reference's packed sparse U tables and
 * its per-element weights (ops/symmetric_contraction.py:91-232): for every monomial the packed
 * entries (i, j, k, path) that map onto it are listed in CSR form by the host.
 *   mono3_ijk  int32 [n3]  : i | j << 8 | k << 16, sorted triples
 *   term3_off  int32 [n3+1], term3_path int32 [nt3], term3_val fp32 [nt3]: CSR of (path, U value)
 *   same for the quadratic part (mono2_ij: i | j << 8).
 *   W3 [ne, P3, C], W2 [ne, P2, C], W1 [ne, P1, C] (only path 0 of W1 is used, as in the reference)
 *   T3 [ne, n3, C], T2 [ne, n2, C], T1 [ne, C]
 */
int cm_symcon_tables(const int32_t *term3_off, const int32_t *term3_path, const float *term3_val,
                     int n3, const int32_t *term2_off, const int32_t *term2_path,
                     const float *term2_val, int n2, const float *W3, const float *W2,
                     const float *W1, int nelements, int P3, int P2, int P1, int channels,
                     float *T3, float *T2, float *T1, cm_stream_t stream);
/*   X [nnodes, 16, C]; atom_types int32 [nnodes] in [0, nelements);
 *   node_perm / group_offsets: nodes grouped by element (cm_stable_key_sort on atom_types);
 *   out [nnodes, C]; grad [nnodes, 16, C] or NULL (d out[n, c] / d X[n, i, c]). */
int cm_symcon_forward(const float *X, const int32_t *node_perm, const int32_t *group_offsets,
                      const int32_t *mono3_ijk, int n3, const int32_t *mono2_ij, int n2,
                      const float *T3, const float *T2, const float *T1, int64_t nnodes,
                      int nelements, int channels, float *out, float *grad, cm_stream_t stream);
/* The monomial lists of the l_max = 3, scalar-output coupling tensors are also compiled into the library
 * (sorted triples / pairs in lexicographic order).  Passing mono3_ijk = mono2_ij = NULL to cm_symcon_forward
 * selects a kernel unrolled over that built-in structure (n3, n2 and the row order of T3, T2 must then be the
 * built-in ones).  cm_symcon_builtin_structure copies the lists to HOST buffers (either may be NULL) and
 * returns their lengths, so that a caller can check that the tables it was given have this structure. */
int cm_symcon_builtin_structure(int32_t *mono3_ijk_host, int capacity3, int32_t *mono2_ij_host,
                                int capacity2, int *n3, int *n2);
/*   gX[n, i, c] = grad_out[n, c] * grad[n, i, c] */
int cm_symcon_backward(const float *grad, const float *grad_out, int64_t nnodes, int channels,
                       float *gX, cm_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * fp64 variants.  The reference dispatches message passing, spherical harmonics, the cubic spline and the symmetric
 * contraction on float and double (AT_DISPATCH_FLOATING_TYPES at
 * jit_wrappers/src/invariant_message_passing_wrapper.cpp:102 and :189, spherical_harmonics_wrapper.cpp:36 and :105,
 * cubic_spline_wrapper.cpp:50 and :123, symmetric_contraction_wrapper.cpp:68); its linears are float only
 * (linear_wrapper.cpp:67).  Each entry point below is the double instantiation of the fp32 one of the same name:
 * same operands, shapes, NULL conventions and index arguments, every floating-point buffer in double.
 * cm_spline_*_f64 accept any noutputs > 0.
 */
int cm_mp_forward_f64(const double *X, const double *Y, const double *R, const int32_t *sender,
                      const int32_t *first_occ, int64_t nnodes, int64_t nedges, int channels,
                      double *out, cm_stream_t stream);
int cm_mp_backward_f64(const double *X, const double *Y, const double *R, const double *grad_out,
                       const int32_t *sender, const int32_t *first_occ, const int32_t *sender_perm,
                       const int32_t *sender_offsets, int64_t nnodes, int64_t nedges, int channels,
                       double *gX, double *gY, double *gR, double *edge_scratch, cm_stream_t stream);
int cm_sh_forward_f64(const double *xyz, int64_t nedges, double *Y, cm_stream_t stream);
int cm_sh_backward_f64(const double *xyz, const double *grad_Y, int64_t nedges, double *grad_xyz,
                       cm_stream_t stream);
int cm_spline_forward_f64(const double *r, const double *r_knots, const double *coeffs, int64_t nedges,
                          int nknots, int noutputs, double r_width, double r_max, double *R_out,
                          double *R_deriv, cm_stream_t stream);
int cm_spline_backward_f64(const double *r, const double *r_knots, const double *coeffs,
                           const double *grad_R, int64_t nedges, int nknots, int noutputs,
                           double r_width, double r_max, double *grad_r, cm_stream_t stream);
int cm_symcon_tables_f64(const int32_t *term3_off, const int32_t *term3_path, const double *term3_val,
                         int n3, const int32_t *term2_off, const int32_t *term2_path,
                         const double *term2_val, int n2, const double *W3, const double *W2,
                         const double *W1, int nelements, int P3, int P2, int P1, int channels,
                         double *T3, double *T2, double *T1, cm_stream_t stream);
int cm_symcon_forward_f64(const double *X, const int32_t *node_perm, const int32_t *group_offsets,
                          const int32_t *mono3_ijk, int n3, const int32_t *mono2_ij, int n2,
                          const double *T3, const double *T2, const double *T1, int64_t nnodes,
                          int nelements, int channels, double *out, double *grad, cm_stream_t stream);
int cm_symcon_backward_f64(const double *grad, const double *grad_out, int64_t nnodes, int channels,
                           double *gX, cm_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Neighbour list on the device: all ordered pairs (i, j, S) with |r_j - r_i + S . cell| < cutoff, (j, S) != (i, 0),
 * sorted lexicographically by (i, j, Sx, Sy, Sz) -- the step before the path.  The reference leaves it to the
 * host: its model consumes data["edge_index"] / ["shifts"] built upstream (models/InvariantMACE.py:297-301) and its
 * tests obtain them from a CPU neighbour search through the upstream data loader (tests/test_utils.py:62-105).
 * Row i of the result is non-decreasing, which is what cm_first_occurences and the message-passing kernels need.
 *   positions fp64 [nnodes, 3] (atoms may lie outside the cell); cell fp64 [3, 3] row vectors (device pointer;
 *   may be NULL without periodic axes); pbc_x/y/z: periodicity along the cell vectors; cutoff > 0.
 * The accept test is v = (r_j - r_i) + (Sx c0 + Sy c1 + Sz c2), v0 v0 + v1 v1 + v2 v2 < cutoff^2, evaluated in fp64
 * left to right without fused multiply-adds.
 * Two calls, because the number of pairs is known only after the first:
 *   cm_neighbour_list_count: builds the cell list in `workspace` (cm_neighbour_list_workspace(nnodes, max_cells)
 *     bytes; max_cells bounds the number of bins, nnodes is a good value) and writes offsets int32 [nnodes + 1]
 *     (offsets[i] = first pair of atom i, offsets[nnodes] = number of pairs) and status int32 [1] (0 = ok,
 *     1 = periodic axis with a singular cell, 2 = a periodic axis thinner than cutoff / 32; offsets are then
 *     all zero).
 *   cm_neighbour_list_fill: after the caller has read offsets[nnodes] = nedges and provided edge_scratch int32
 *     [4 * nedges], writes row_i, row_j int32 [nedges] and unit_shifts int32 [nedges, 3].  `workspace` must be
 *     the one the count call filled, untouched, with the same positions, cutoff, nnodes and max_cells.
 */
size_t cm_neighbour_list_workspace(int64_t nnodes, int64_t max_cells);
int cm_neighbour_list_count(const double *positions, const double *cell, int pbc_x, int pbc_y, int pbc_z,
                            double cutoff, int64_t nnodes, int64_t max_cells, void *workspace,
                            size_t workspace_bytes, int32_t *offsets, int32_t *status, cm_stream_t stream);
int cm_neighbour_list_fill(const double *positions, double cutoff, int64_t nnodes, int64_t max_cells,
                           const void *workspace, const int32_t *offsets, int64_t nedges, int32_t *edge_scratch,
                           int32_t *row_i, int32_t *row_j, int32_t *unit_shifts, cm_stream_t stream);

/*
 * The test a molecular-dynamics driver makes before it reuses a list built out to cutoff + skin: out_sq[0] (fp64,
 * device memory) = the largest squared distance between an atom's row of `positions` and of `reference` (the
 * positions the list was built from), both fp64 [nnodes, 3]; +inf when a coordinate is NaN, 0 without atoms.  The
 * list stays valid while that is at most (skin / 2)^2.  No counterpart in the reference, which leaves the list to
 * its callers (tests/test_utils.py:62-105 rebuild it on the host for every evaluation).  Two small launches, no
 * workspace, nothing read back.
 */
int cm_max_displacement(const double *positions, const double *reference, int64_t nnodes, double *out_sq,
                        cm_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Readouts of the two-layer invariant model, scale / shift and their derivative in one pass, fp64 arithmetic on the
 * fp32 node features.  Replaces the upstream readout modules the reference keeps in fp64 and the casts around them
 * (models/InvariantMACE.py:196, 330-337, 343): a dozen small fp64 GEMM / element-wise launches per direction.
 *   h1, h2 fp32 [nnodes, channels]: node features after the first / second layer;
 *   w1 fp64 [channels]: linear readout of h1 (1/sqrt(fan_in) folded in);
 *   W2a fp64 [channels, hidden], w2b fp64 [hidden] (hidden <= 16): the one-hidden-layer readout of h2 with
 *   act(z) = act_cst * z * sigmoid(z) (1/sqrt(fan_in) folded into both);
 *   node_energies[n] = scale * (h1[n] . w1 + sum_j w2b[j] act((h2[n] . W2a)_j)) + shift        fp64 [nnodes]
 *   d_h2 fp32 [nnodes, channels] = d node_energies[n] / d h2[n, c]   (d / d h1 is scale * w1, not stored)
 *   node_feats64 fp64 [nnodes, 2 * channels] = [h1 | h2], or NULL; with feats_rows int32 [nnodes] (a permutation; may
 *   be NULL) the features of node n go to row feats_rows[n].
 * Backward: grad_h1[n, c] = g[n] * scale * w1[c], grad_h2[n, c] = g[n] * d_h2[n, c] (either may be NULL).
 */
int cm_readout_forward(const float *h1, const float *h2, const double *w1, const double *W2a, const double *w2b,
                       double act_cst, double scale, double shift, int64_t nnodes, int channels, int hidden,
                       double *node_energies, float *d_h2, double *node_feats64, const int32_t *feats_rows,
                       cm_stream_t stream);
int cm_readout_backward(const double *grad_node_energies, const double *w1, const float *d_h2, double scale,
                        int64_t nnodes, int channels, float *grad_h1, float *grad_h2, cm_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Index structures of one neighbour list in one call, without a host synchronisation (no counterpart in the reference,
 * which takes the list as upstream's host-side search returns it, tests/test_utils.py:62-105, and builds its N x N
 * reverse-edge table inside every forward call, jit_wrappers/src/invariant_message_passing_wrapper.cpp:91-93).
 *   in:  positions fp64 [nnodes, 3]; the list row_i (non-decreasing, in [0, nnodes)), row_j int32 [nedges] with
 *        shifts fp64 [nedges, 3] (vector of a pair = positions[row_j] - positions[row_i] + shift);
 *        graph_of_node int32 [nnodes] (non-decreasing) or NULL for one graph; r_max: the model's cutoff;
 *        bins: cells per axis of the grid the atoms are ordered by (1 .. 64; ngraphs * bins^3 < 2^24; cells are at
 *        least r_max / 2 wide and cover the bounding box of the positions)
 *   out: node_perm [nnodes]: atom a of the new order is atom node_perm[a] of the caller (atoms sorted by graph, grid
 *        cell, original index); node_inverse [nnodes] its inverse;
 *        receiver / sender int32 [nedges]: the list in the new labels, sorted by receiver (= new label of row_i); inside a
 *        receiver's segment the pairs within r_max by sender label, then the others by length; ties keep the list's order;
 *        edge_perm [nedges]: pair e of the new list is pair edge_perm[e] of the caller's; shifts_out fp64 [nedges, 3];
 *        first_occ [2 nnodes] = cm_first_occurences(receiver);
 *        sender_perm [nedges], sender_offsets [nnodes + 1] = cm_stable_key_sort(sender, nedges, nnodes).
 *   workspace: cm_graph_prepare_workspace(nnodes, nedges, ngraphs, bins) bytes, 256-byte aligned.
 * Every output is a function of the inputs alone (fixed orders throughout): the same list gives the same bits. */
size_t cm_graph_prepare_workspace(int64_t nnodes, int64_t nedges, int ngraphs, int bins);
int cm_graph_prepare(const double *positions, const int32_t *row_i, const int32_t *row_j, const double *shifts,
                     const int32_t *graph_of_node, int64_t nnodes, int64_t nedges, int ngraphs, double r_max, int bins,
                     int32_t *node_perm, int32_t *node_inverse, int32_t *receiver, int32_t *sender, int32_t *edge_perm,
                     double *shifts_out, int32_t *first_occ, int32_t *sender_perm, int32_t *sender_offsets, void *workspace,
                     size_t workspace_bytes, cm_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * The three [nnodes, C] x [C, C] linears between the two interaction layers as one launch per direction: the product's
 * linear and linear_up (the reference's linear_matmul, models/InvariantMACE.py:41-53) and the per-element skip
 * connection between them (element_linear_to_cuda, :56-74; called at :145-150 and :330).  A workgroup takes 128 nodes
 * of one element through the chain with the intermediate rows in LDS; same arithmetic, rounding points and results as
 * the three cm_linear calls it stands for.  channels = 32, 64, 96 or 128 (cm_node_glue_supported).
 *   node_perm / group_offsets: nodes grouped by element, ngroups = nelements + 1 with the last group holding the nodes
 *   without an element (their skip connection is zero), as cm_linear takes them with zero_last_group.
 * Forward:  h1 = B1 . prod_W;  sc = skip_scale * h1 . skip_W[element];  X2 = h1 . up_W       (all fp32 [nnodes, C];
 *   weights passed transposed, [C out, C in], skip_WT [nelements, C, C]).
 * Backward: gB1 = (gX2 . up_W^T + g1 - skip_scale * d_h2 . skip_W[element]^T) . prod_W^T with
 *   g1[n, c] = -node_weights[n] * scale * w1[c] (node_weights may be NULL = 1): the gradient of minus the weighted sum of
 *   node energies (cm_readout_forward's d_h2, scale, w1) through the chain; weights passed plain, [C in, C out].
 */
int cm_node_glue_supported(int channels);
int cm_node_glue_forward(const float *B1, const float *prod_WT, const float *skip_WT, const float *up_WT,
                         const int32_t *node_perm, const int32_t *group_offsets, int64_t nnodes, int ngroups, int channels,
                         float skip_scale, float *h1, float *sc, float *X2, cm_stream_t stream);
int cm_node_glue_backward(const float *gX2, const float *d_h2, const float *up_W, const float *skip_W, const float *prod_W,
                          const double *w1, double scale, const double *node_weights, const int32_t *node_perm,
                          const int32_t *group_offsets, int64_t nnodes, int ngroups, int channels, float skip_scale,
                          float *gB1, cm_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * One energy + forces evaluation of the two-layer invariant model as a single call: every kernel of the step, forward
 * and backward, enqueued back to back by the library itself.  It replaces, for inference, what the reference runs as a
 * Python forward over its TorchScript classes followed by an autograd backward (models/InvariantMACE.py:246-379:
 * interactions :76-160, products :330, readouts :336, scale/shift :344, forces through get_outputs :354): same kernels,
 * same order, same numbers as that sequence, without a Python interpreter or an autograd engine between the launches
 * (18 launches up to 128 channels, 25 beyond; host cost of a step drops from ~0.4 ms to well under 0.1 ms).
 *
 * cm_mace_weights: the model's frozen weights in the layouts the op modules hold them (device pointers).
 *   spline[t]      [nknots - 1, 4, 4C]   radial spline table of layer t (cm_spline_forward's coeffs)
 *   mix_WT/mix_W   channel mixing between message passing and contraction, transposed / plain blocks with mix_scale:
 *                  layer 0 per element [ne, 4, C, C] (the per-l linear composed with the per-element linear,
 *                  models/InvariantMACE.py:56-74, 113-116), layer 1 [4, C, C]; 1 / avg_num_neighbors folded in
 *   T3/T2/T1       contraction coefficient tables of layer t (cm_symcon_tables); mono3/mono2 NULL selects the
 *                  built-in l_max = 3 structure, otherwise the monomial lists with n3/n2 entries
 *   prod_WT/prod_W [C, C] linear after the contraction (1/sqrt(C) folded in), both orientations
 *   up_WT/up_W     [C, C] linear_up of layer 1 (the second layer; layer 0's acts on species-only features, see X1)
 *   skip_WT/skip_W [ne, C, C] residual skip connection of the second layer per element, with skip_scale
 *   w1, W2a [C, hidden], w2b [hidden], act_cst, scale, shift: cm_readout_forward's operands
 * cm_mace_graph: what depends on the neighbour list and the species only (device pointers; rebuilt when they change).
 *   receiver (non-decreasing) / sender int32 [nedges]; first_occ = cm_first_occurences(receiver);
 *   sender_perm / sender_offsets = cm_stable_key_sort(sender, nedges, nnodes);
 *   elem_perm / elem_offsets = cm_stable_key_sort(element index, nnodes, ne)           [nnodes], [ne + 1]
 *   onehot_perm / onehot_offsets: the same grouping with one more, empty-weight group for atoms whose one-hot row
 *     names no element [nnodes], [ne + 2] (pass the element grouping with a closing repeated offset if there are none)
 *   node_rows int32 [nnodes] or NULL: atom n of the lists is row node_rows[n] of positions / forces / node_feats
 *   graph_ptr int32 [ngraphs + 1]: node range of every graph of the batch, in the order of the lists
 *   X1 fp32 [nnodes, C]: linear_up(node_embedding(species)) of the first layer
 *   node_weights fp64 [nnodes] (in the order of the lists) or NULL: weight of every node energy in interaction_energy
 *     and in the quantity the forces derive from, sum_n node_weights[n] * node_energy[n]; what the rank of a
 *     domain-decomposed MD code needs (1 for its own atoms, 0 for ghost copies: upstream MACE's LAMMPS wrapper,
 *     mace/calculators/lammps_mace.py; the reference has no counterpart).  NULL is all ones, bit for bit.
 *   node_e0 fp64 [nnodes] (in the order of the lists) / graph_e0 fp64 [ngraphs], or NULL = zeros: what total_node_energy /
 *     total_energy add to the interaction part, i.e. the atomic reference energies of the species and their (weighted)
 *     sum per graph (models/InvariantMACE.py:287-293 computes them per call; they depend on the species alone)
 * Per call: positions fp64 [nnodes, 3], shifts fp64 [nedges, 3]; outputs interaction_energy fp64 [ngraphs] ((weighted) sum
 * of the node energies of each graph, in a fixed order), node_energy fp64 [nnodes] (interaction part, unweighted, in
 * list order), forces fp64 [nnodes, 3] = -d(sum of interaction_energy)/d positions (rows of the caller when node_rows is given), node_feats fp64
 * [nnodes, 2C] or NULL, virials fp64 [ngraphs, 3, 3] or NULL = minus the derivative of each graph's energy with respect to a
 * symmetric strain of its positions and cell (what models/InvariantMACE.py:273-285 obtains by differentiating through
 * get_symmetric_displacement), formed from the per-edge gradients as 1/2 sum_e (vec_e (x) g_e + g_e (x) vec_e), g_e =
 * -dE/d vec_e.  total_energy fp64 [ngraphs] or NULL = interaction_energy + graph_e0; total_node_energy fp64 [nnodes] or NULL
 * = node_energy + node_e0, atom n of the lists written to row node_rows[n] (what the reference returns as "energy" and
 * "node_energy", models/InvariantMACE.py:350-352, without a launch of their own).  workspace: cm_mace_step_workspace(nnodes, nedges, channels) bytes, 256-byte aligned; its
 * contents are scratch.  Nothing is allocated, so the call can be captured into a HIP graph.
 */
typedef struct cm_mace_weights {
  int channels, nelements, nknots, hidden;
  float r_width, r_max;
  const float *r_knots;
  const float *spline[2];
  const float *mix_WT[2], *mix_W[2];
  float mix_scale[2];
  const float *T3[2], *T2[2], *T1[2];
  const int32_t *mono3[2], *mono2[2];
  int n3[2], n2[2];
  const float *prod_WT[2], *prod_W[2];
  const float *up_WT, *up_W;
  const float *skip_WT, *skip_W;
  float skip_scale;
  const double *w1, *W2a, *w2b;
  double act_cst, scale, shift;
} cm_mace_weights;

typedef struct cm_mace_graph {
  int64_t nnodes, nedges;
  int ngraphs;
  const int32_t *receiver, *sender, *first_occ, *sender_perm, *sender_offsets;
  const int32_t *elem_perm, *elem_offsets, *onehot_perm, *onehot_offsets;
  const int32_t *node_rows, *graph_ptr;
  const float *X1;
  const double *node_weights;
  const double *node_e0, *graph_e0;
} cm_mace_graph;

/* Per-stage timing of cm_mace_step (off by default): with bit s of stage_mask set, stage s of every later step is
 * bracketed by two events recorded on the launch stream; cm_mace_step_timing_read waits for the outstanding events and
 * returns, per stage, the accumulated milliseconds and the number of timed launches since the mask was set (arrays of
 * at least 25 entries; the return value is the number of stages).  Setting a mask resets the accumulators.  A step
 * enqueued while its stream is capturing is not timed (events recorded into a capture cannot be read back).  Stages: 0 edge geometry and live edge ranges; 1 / 7 message passing forward of layer
 * 0 / 1; 2 / 8 channel mixing; 3 / 9 contraction; 4 / 10 linear after it; 5 skip connection; 6 linear_up; 11 readouts; 12 energy sums per graph;
 * 13 seeds of the backward chain; 14 / 19 linear after the contraction, backward; 15 / 20 channel mixing backward (contraction
 * backward folded in); 16 message passing backward of layer 1 (edge pass + sender pass); 21 of layer 0 (edge pass
 * only); 17 linear_up backward; 18 skip backward; 22 sum of the two layers' per-edge gradients; 23 edge geometry backward
 * (forces); 24 virials. */
int cm_mace_step_timing(unsigned stage_mask);
/* A control launch for benchmarks (no counterpart in the reference): `workgroups` workgroups of 256 lanes, each lane
 * 8 * iters independent fp32 multiply-adds and nothing else (2 * 8 * iters * 256 * workgroups flop); out: one float the
 * kernel never writes.  Timed by the caller, it tells what the vector ALUs of this box deliver. */
int cm_probe_fma(float *out, int workgroups, int iters, cm_stream_t stream);
int cm_mace_step_timing_read(double *total_ms, int64_t *launches, int capacity);
size_t cm_mace_step_workspace(int64_t nnodes, int64_t nedges, int channels);
int cm_mace_step(const cm_mace_weights *weights, const cm_mace_graph *graph, const double *positions, const double *shifts,
                 void *workspace, size_t workspace_bytes, double *interaction_energy, double *node_energy, double *forces,
                 double *node_feats, double *virials, double *total_energy, double *total_node_energy, cm_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* CUDA_MACE_HIP_H */
