"""torch.autograd functions of the ops that go beyond the reference's interface; forward and backward are C-ABI calls.

The six ops of the reference (message passing, spherical harmonics, cubic spline, linear, elemental linear, symmetric
contraction) are TorchScript custom classes implemented in csrc/torch_classes.cpp.  This module holds the fused
variants the model uses by default -- message passing with the radial spline (and the harmonics) evaluated in-kernel,
and the edge-geometry step -- plus the host-side regrouping of the packed coupling tables for direct users of the C ABI.

Index structures that depend only on the neighbour list (CSR offsets, the sender-sorted edge view) are cached on the
tensor object they were derived from, guarded by its version counter, so they are built once per neighbour list
instead of once per call.
"""
from __future__ import annotations

import functools
import weakref

import numpy as np
import torch

from .. import _cabi as cabi

F32, I32 = torch.float32, torch.int32


def _require(cond, msg):
    if not cond:
        raise RuntimeError(msg)


_TRACE = bool(cabi.lib.cm_trace_enabled())  # decided once: CUDA_MACE_TRACE must be set before the import


def _traced(name: str):
    """Profiler range around an autograd forward / backward (the reference's PUSH_RANGE / POP_RANGE, include/utils.h:9-21);
    the function is returned unchanged when tracing is off."""

    def decorate(fn):
        if not _TRACE:
            return fn
        label = ("cuda_mace:" + name).encode()

        @functools.wraps(fn)
        def wrapper(*args, **kwargs):
            cabi.lib.cm_trace_push(label)
            try:
                return fn(*args, **kwargs)
            finally:
                cabi.lib.cm_trace_pop()

        return wrapper

    return decorate


def _cached(owner: torch.Tensor, slot: str, key, build):
    """Value derived from `owner`, rebuilt when owner was modified in place or `key` differs."""
    tag = (owner._version, owner.data_ptr(), key)
    hit = owner.__dict__.get(slot)
    if hit is not None and hit[0] == tag:
        return hit[1]
    val = build()
    owner.__dict__[slot] = (tag, val)
    return val


def _cached_for(owner: torch.Tensor, slot: str, other, build):
    """Value derived from `owner` and `other` (a tensor, or any object that stands for a set of weights), kept on
    `owner`; rebuilt when either was modified in place or `other` is another object.  The entry holds a reference to
    `other`, so neither its address nor its id can be recycled under the cache."""
    hit = owner.__dict__.get(slot)
    tag = (owner._version, owner.data_ptr(), getattr(other, "_version", 0))
    if hit is not None and hit[0] is other and hit[1] == tag:
        return hit[2]
    val = build()
    owner.__dict__[slot] = (other, tag, val)
    return val


class _PerToken(weakref.WeakKeyDictionary):
    """Cache entries per weights token; a copy or a pickle of the tensor that carries it starts empty (the entries
    hold device addresses and belong to live model objects)."""

    def __reduce__(self):
        return (_PerToken, ())

    def __deepcopy__(self, memo):
        return _PerToken()

    def __copy__(self):
        return _PerToken()


def _cached_per(owner: torch.Tensor, slot: str, token, other, build):
    """As `_cached_for`, with one entry per `token` (an object that stands for one model's weights) kept on `owner`.
    Tokens are held weakly: an entry disappears with its model, so the id of a dead token can never be taken for a
    live one's, and several models evaluated on the same tensors do not evict each other."""
    table = owner.__dict__.get(slot)
    if table is None:
        table = owner.__dict__[slot] = _PerToken()
    tag = (owner._version, owner.data_ptr(), getattr(other, "_version", 0))
    hit = table.get(token)
    if hit is not None and hit[0] is other and hit[1] == tag:
        return hit[2]
    val = build()
    table[token] = (other, tag, val)
    return val


def csr_of(receiver: torch.Tensor, nnodes: int) -> torch.Tensor:
    return _cached(receiver, "_cm_csr", nnodes, lambda: cabi.first_occurences(receiver, nnodes))


def sender_view_of(sender: torch.Tensor, nnodes: int):
    return _cached(sender, "_cm_sender_view", nnodes, lambda: cabi.stable_key_sort(sender, nnodes))


def groups_of(atom_types: torch.Tensor, nelements: int):
    """(node_perm, group_offsets) listing nodes element by element."""
    return _cached(atom_types, "_cm_groups", nelements, lambda: cabi.stable_key_sort(atom_types, nelements))


def groups_of_one_hot(one_hot: torch.Tensor):
    """Nodes grouped by the column where one_hot == 1 (rows without such a column end up in no group)."""

    def build():
        ne = one_hot.shape[1]
        mask = one_hot == 1
        elem = mask.to(torch.int8).argmax(dim=1).to(I32)
        elem = torch.where(mask.any(dim=1), elem, torch.full_like(elem, ne))
        return cabi.stable_key_sort(elem.contiguous(), ne + 1)  # group ne collects the rows without an element

    return _cached(one_hot, "_cm_groups", None, build)


# ------------------------------------------------------------------------------------------------
class InvariantMessagePassingSplineTPAutograd(torch.autograd.Function):
    """Message passing whose radial weights are evaluated in-kernel from the spline table: equivalent to
    CubicSplineAutograd followed by InvariantMessagePassingTPAutograd, without R / grad_R in memory.
    Differentiable in X, Y and the edge lengths r."""

    @staticmethod
    @_traced("message_passing_spline forward")
    def forward(ctx, X, Y, r, r_knots, coeffs, r_width, r_max, sender_list, receiver_list, nnodes):
        _require(X.dtype == F32 and Y.dtype == F32 and r.dtype == F32 and coeffs.dtype == F32 and r_knots.dtype == F32,
                 "fused message passing: fp32 tensors expected")
        _require(sender_list.dtype == I32 and receiver_list.dtype == I32, "fused message passing: int32 edge lists expected")
        _require(Y.dim() == 2 and Y.shape[0] == 16, "fused message passing: Y must be [16, nedges]")
        _require(X.dim() == 2 and X.shape[1] % 32 == 0, "fused message passing: X must be [nnodes, C] with C % 32 == 0")
        nnodes = int(nnodes)
        first_occ = csr_of(receiver_list, nnodes)
        Xc, Yc, rc = X.contiguous(), Y.contiguous(), r.contiguous().view(-1)
        out = cabi.mp_spline_forward(Xc, Yc, rc, r_knots, coeffs, r_width, r_max, sender_list, first_occ, nnodes)
        ctx.save_for_backward(Xc, Yc, rc, r_knots, coeffs, sender_list, first_occ)
        ctx.nnodes, ctx.r_width, ctx.r_max, ctx.r_shape = nnodes, float(r_width), float(r_max), r.shape
        return out

    @staticmethod
    @_traced("message_passing_spline backward")
    def backward(ctx, grad_out):
        X, Y, r, r_knots, coeffs, sender, first_occ = ctx.saved_tensors
        need_x, need_y, need_r = ctx.needs_input_grad[:3]
        perm = off = None
        if need_x:
            perm, off = sender_view_of(sender, ctx.nnodes)
        gX, gY, gr = cabi.mp_spline_backward(X, Y, r, r_knots, coeffs, ctx.r_width, ctx.r_max, grad_out.contiguous(), sender,
                                             first_occ, perm, off, ctx.nnodes, need_gX=need_x, need_gY=need_y, need_gr=need_r)
        if gr is not None:
            gr = gr.view(ctx.r_shape)
        return gX, gY, gr, None, None, None, None, None, None, None


# ------------------------------------------------------------------------------------------------
class InvariantMessagePassingEdgeTPAutograd(torch.autograd.Function):
    """Message passing straight from the edge vectors: harmonics, length and radial spline are evaluated in-kernel.
    Equivalent to SphericalHarmonicsAutograd + CubicSplineAutograd + InvariantMessagePassingTPAutograd on
    (vectors, |vectors|); differentiable in X and the vectors."""

    @staticmethod
    @_traced("message_passing_edges forward")
    def forward(ctx, X, vectors, r_knots, coeffs, r_width, r_max, sender_list, receiver_list, nnodes):
        _require(X.dtype == F32 and vectors.dtype == F32 and coeffs.dtype == F32 and r_knots.dtype == F32,
                 "edge message passing: fp32 tensors expected")
        _require(sender_list.dtype == I32 and receiver_list.dtype == I32, "edge message passing: int32 edge lists expected")
        _require(vectors.dim() == 2 and vectors.shape[1] == 3, "edge message passing: vectors must be [nedges, 3]")
        _require(X.dim() == 2 and X.shape[1] % 32 == 0, "edge message passing: X must be [nnodes, C] with C % 32 == 0")
        nnodes = int(nnodes)
        first_occ = csr_of(receiver_list, nnodes)
        Xc, vc = X.contiguous(), vectors.contiguous()
        out = cabi.mp_edge_forward(Xc, vc, r_knots, coeffs, r_width, r_max, sender_list, first_occ, nnodes)
        ctx.save_for_backward(Xc, vc, r_knots, coeffs, sender_list, first_occ)
        ctx.nnodes, ctx.r_width, ctx.r_max = nnodes, float(r_width), float(r_max)
        return out

    @staticmethod
    @_traced("message_passing_edges backward")
    def backward(ctx, grad_out):
        X, vectors, r_knots, coeffs, sender, first_occ = ctx.saved_tensors
        need_x, need_v = ctx.needs_input_grad[:2]
        perm = off = None
        if need_x:
            perm, off = sender_view_of(sender, ctx.nnodes)
        gX, gvec = cabi.mp_edge_backward(X, vectors, r_knots, coeffs, ctx.r_width, ctx.r_max, grad_out.contiguous(), sender,
                                         first_occ, perm, off, ctx.nnodes, need_gX=need_x, need_gvec=need_v)
        return gX, gvec, None, None, None, None, None, None, None


# ------------------------------------------------------------------------------------------------
class EdgeGeometryAutograd(torch.autograd.Function):
    """(positions [N,3], shifts [E,3], row_a int32 [E] non-decreasing, row_b int32 [E], node_rows int32 [N] or None) ->
    (vectors fp32 [E,3], lengths fp32 [E]) with vectors = positions[row_b] - positions[row_a] + shifts evaluated in fp64.
    With node_rows, atom n of the edge lists is row node_rows[n] of positions (and of its gradient).
    Differentiable in positions and shifts; the backward scatters edge gradients to atoms over the CSR of row_a
    and the sorted view of row_b (the same index structures message passing uses), in fp64, without atomics."""

    @staticmethod
    @_traced("edge_geometry forward")
    def forward(ctx, positions, shifts, row_a, row_b, node_rows):
        _require(row_a.dtype == I32 and row_b.dtype == I32, "edge geometry: int32 edge lists expected")
        _require(positions.dim() == 2 and positions.shape[1] == 3, "edge geometry: positions must be [nnodes, 3]")
        _require(node_rows is None or (node_rows.dtype == I32 and node_rows.numel() == positions.shape[0]),
                 "edge geometry: node_rows must be int32 [nnodes]")
        pos64 = positions.detach().double().contiguous()
        sh64 = shifts.detach().double().contiguous()
        vec, length = cabi.edge_geometry_forward(pos64, row_a, row_b, sh64, node_rows)
        ctx.save_for_backward(pos64, sh64, row_a, row_b)
        ctx.node_rows = node_rows
        ctx.dtypes = (positions.dtype, shifts.dtype)
        ctx.set_materialize_grads(False)  # an unused output arrives as None in backward, not as zeros
        return vec, length

    @staticmethod
    @_traced("edge_geometry backward")
    def backward(ctx, grad_vec, grad_len):
        if grad_vec is None and grad_len is None:
            return None, None, None, None, None
        pos64, sh64, row_a, row_b = ctx.saved_tensors
        need_pos, need_shift = ctx.needs_input_grad[:2]
        nnodes = pos64.shape[0]
        first_occ = csr_of(row_a, nnodes)
        perm, off = sender_view_of(row_b, nnodes)
        gv = grad_vec.contiguous() if grad_vec is not None else None
        gl = grad_len.contiguous() if grad_len is not None else None
        gpos, gshift = cabi.edge_geometry_backward(pos64, row_a, row_b, sh64, first_occ, perm, off, gv, gl,
                                                   need_positions=need_pos, need_shifts=need_shift, node_rows=ctx.node_rows)
        if gpos is not None:
            gpos = gpos.to(ctx.dtypes[0])
        if gshift is not None:
            gshift = gshift.to(ctx.dtypes[1])
        return gpos, gshift, None, None, None


class LinearContractionAutograd(torch.autograd.Function):
    """Per-l (or per-element, per-l) linear followed by the symmetric contraction, as one autograd node:

        Y = linear(X),  out = contraction(Y)          forward (Y is dropped, the contraction's gradient table kept)
        gX = linear^T(grad_out[:, None, :] * grad)    backward, ONE kernel: the contraction's backward is folded into
                                                      the operand load of the linear's backward

    Same numbers as Linear / ElementalLinear -> SymmetricContraction; saves the [N,16,C] write and read between the two
    backward kernels.  X [N,16,K]; W_T / W the transposed / plain weight blocks ([4,..] or [ne,4,..]) with `scale`;
    lin_groups = (perm, offsets) for per-element weights or None; sym_groups = nodes grouped by element;
    tables = (mono3, mono2, T3, T2, T1, builtin)."""

    @staticmethod
    @_traced("linear_contraction forward")
    def forward(ctx, X, W_T, W, scale, lin_groups, sym_groups, tables):
        mono3, mono2, T3, T2, T1, builtin = tables
        lp, lo = lin_groups if lin_groups is not None else (None, None)
        # per-element weights: the grouping by one-hot row has one more group than there are weight blocks, for rows
        # that name no element; those rows come out as zeros
        Y = cabi.linear(X.contiguous(), W_T, lp, lo, scale, zero_last_group=lin_groups is not None)
        out, grad = cabi.symcon_forward(Y, sym_groups[0], sym_groups[1], mono3, mono2, T3, T2, T1, want_grad=True,
                                        builtin=builtin, zero_init=False)
        ctx.save_for_backward(grad, W)
        ctx.scale, ctx.lin_groups = scale, lin_groups
        return out

    @staticmethod
    @_traced("linear_contraction backward")
    def backward(ctx, grad_out):
        grad, W = ctx.saved_tensors
        lp, lo = ctx.lin_groups if ctx.lin_groups is not None else (None, None)
        gX = cabi.linear(grad, W, lp, lo, ctx.scale, zero_last_group=ctx.lin_groups is not None,
                         row_scale=grad_out.contiguous())
        return gX, None, None, None, None, None, None


class ScalarLinearAutograd(torch.autograd.Function):
    """Y = X . W (+ residual) for scalar features X [N, K] on the MFMA linear kernel (one component per node); W_T [N', K]
    and W [K, N'] are the two orientations of the same weights (forward uses W_T, the backward W).  The optional
    residual [N, N'] is added in the kernel's epilogue; its gradient is the incoming one."""

    @staticmethod
    @_traced("scalar_linear forward")
    def forward(ctx, X, W_T, W, residual):  # always four arguments (residual may be None): backward returns four
        ctx.save_for_backward(W)
        return cabi.linear(X.contiguous(), W_T, scale=1.0, residual=None if residual is None else residual.contiguous())

    @staticmethod
    @_traced("scalar_linear backward")
    def backward(ctx, grad):
        (W,) = ctx.saved_tensors
        gX = cabi.linear(grad.contiguous(), W, scale=1.0) if ctx.needs_input_grad[0] else None
        return gX, None, None, (grad if ctx.needs_input_grad[3] else None)


class ReadoutEnergyAutograd(torch.autograd.Function):
    """(h1, h2 fp32 [N, C]) -> (node energies fp64 [N], node_feats fp64 [N, 2C]): both readouts, scale and shift in one
    kernel; the derivative with respect to h2 is produced by the same pass and only scaled in the backward.  feats_rows
    (int32 permutation, optional) places the features of node n in row feats_rows[n] of node_feats."""

    @staticmethod
    @_traced("readout forward")
    def forward(ctx, h1, h2, w1, W2a, w2b, act_cst, scale, shift, feats_rows=None):
        es, d2, feats = cabi.readout_forward(h1.detach().contiguous(), h2.detach().contiguous(), w1, W2a, w2b, act_cst, scale, shift,
                                             feats_rows=feats_rows)
        ctx.save_for_backward(w1, d2)
        ctx.scale = float(scale)
        ctx.mark_non_differentiable(feats)
        ctx.set_materialize_grads(False)  # no [N, 2C] tensor of zeros is made for the gradient of feats in every backward
        return es, feats

    @staticmethod
    @_traced("readout backward")
    def backward(ctx, grad_es, _grad_feats):
        w1, d2 = ctx.saved_tensors
        if grad_es is None:
            return (None,) * 9
        g1, g2 = cabi.readout_backward(grad_es.contiguous(), w1, d2, ctx.scale, ctx.needs_input_grad[0], ctx.needs_input_grad[1])
        return g1, g2, None, None, None, None, None, None, None


# ------------------------------------------------------------------------------------------------
def monomials_from_packed(U3_num, U3_idx, U3_val, U2_num, U2_idx, U2_val):
    """Host pass over the packed sparse coupling tables (format of ops/symmetric_contraction.py:91-187):
    groups the entries (i, j, k, path, value) by the sorted index triple they multiply and returns CSR
    arrays (mono, offsets, path, value) for the cubic and the quadratic part."""
    n3 = U3_num.cpu().numpy().astype(np.int64)
    i3 = U3_idx.cpu().numpy().astype(np.int64)
    v3 = U3_val.cpu().numpy().astype(np.float64)
    n2 = U2_num.cpu().numpy().astype(np.int64)
    i2 = U2_idx.cpu().numpy().astype(np.int64)
    v2 = U2_val.cpu().numpy().astype(np.float64)
    terms3, terms2 = {}, {}
    for i in range(16):
        for j in range(16):
            for t in range(int(n3[i, j])):
                word = int(i3[t, i, j])
                k, p = (word >> 8) & 0xFF, word & 0xFF
                bucket = terms3.setdefault(tuple(sorted((i, j, k))), {})
                bucket[p] = bucket.get(p, 0.0) + float(v3[t, i, j])
            if int(n2[i, j]) > 0:
                bucket = terms2.setdefault(tuple(sorted((i, j))), {})
                p = int(i2[i, j])
                bucket[p] = bucket.get(p, 0.0) + float(v2[i, j])

    def pack(terms, shifts):
        mono, off, path, val = [], [0], [], []
        for key in sorted(terms):
            mono.append(sum(idx << s for idx, s in zip(key, shifts)))
            for p in sorted(terms[key]):
                path.append(p)
                val.append(terms[key][p])
            off.append(len(path))
        return (np.asarray(mono, np.int32), np.asarray(off, np.int32), np.asarray(path, np.int32), np.asarray(val, np.float32))

    return pack(terms3, (0, 8, 16)), pack(terms2, (0, 8))
