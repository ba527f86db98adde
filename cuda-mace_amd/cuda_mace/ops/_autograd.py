"""torch.autograd functions of the six ops; forward and backward are C-ABI calls.

Counterparts of the reference's torch::autograd::Function classes (src/invariant_message_passing.cpp:12-59,
src/spherical_harmonics.cpp:12-50, src/cubic_spline.cpp:13-52, src/linear.cpp:9-103,
src/symmetric_contraction.cpp:12-84): same inputs, same differentiable arguments (MP: X, Y, radial;
SH: xyz; spline: r; linears: X; contraction: X), `None` for everything else, first order only.

Index structures that depend only on the neighbour list or on the species (CSR offsets, the
sender-sorted edge view, nodes grouped by element) and tables that depend only on the weights are
cached on the tensor object they were derived from, guarded by its version counter, so they are
built once per neighbour list / model instead of once per call.
"""
from __future__ import annotations

import numpy as np
import torch

from .. import _cabi as cabi

F32, I32 = torch.float32, torch.int32


def _require(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _cached(owner: torch.Tensor, slot: str, key, build):
    """Value derived from `owner`, rebuilt when owner was modified in place or `key` differs."""
    tag = (owner._version, owner.data_ptr(), key)
    hit = owner.__dict__.get(slot)
    if hit is not None and hit[0] == tag:
        return hit[1]
    val = build()
    owner.__dict__[slot] = (tag, val)
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
class InvariantMessagePassingTPAutograd(torch.autograd.Function):
    @staticmethod
    def forward(ctx, X, Y, radial, sender_list, receiver_list, nnodes):
        _require(X.dtype == F32 and Y.dtype == F32 and radial.dtype == F32, "message passing: fp32 tensors expected")
        _require(sender_list.dtype == I32 and receiver_list.dtype == I32, "message passing: int32 edge lists expected")
        _require(Y.dim() == 2 and Y.shape[0] == 16, "message passing: Y must be [16, nedges]")
        _require(X.dim() == 2 and X.shape[1] % 32 == 0, "message passing: X must be [nnodes, C] with C % 32 == 0")
        nnodes = int(nnodes)
        first_occ = csr_of(receiver_list, nnodes)
        Xc, Yc, Rc = X.contiguous(), Y.contiguous(), radial.contiguous()
        out = cabi.mp_forward(Xc, Yc, Rc, sender_list, first_occ, nnodes)
        ctx.save_for_backward(Xc, Yc, Rc, sender_list, first_occ)
        ctx.nnodes = nnodes
        ctx.radial_shape = radial.shape
        return out

    @staticmethod
    def backward(ctx, grad_out):
        X, Y, R, sender, first_occ = ctx.saved_tensors
        need_x, need_y, need_r = ctx.needs_input_grad[:3]
        perm = off = None
        if need_x:
            perm, off = sender_view_of(sender, ctx.nnodes)
        gX, gY, gR = cabi.mp_backward(X, Y, R, grad_out.contiguous(), sender, first_occ, perm, off, ctx.nnodes,
                                      need_gX=need_x, need_gY=need_y, need_gR=need_r)
        if gR is not None:
            gR = gR.view(ctx.radial_shape)
        return gX, gY, gR, None, None, None


# ------------------------------------------------------------------------------------------------
class InvariantMessagePassingSplineTPAutograd(torch.autograd.Function):
    """Message passing whose radial weights are evaluated in-kernel from the spline table: equivalent to
    CubicSplineAutograd followed by InvariantMessagePassingTPAutograd, without R / grad_R in memory.
    Differentiable in X, Y and the edge lengths r."""

    @staticmethod
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
    """(positions [N,3], shifts [E,3], row_a int32 [E] non-decreasing, row_b int32 [E]) -> (vectors fp32 [E,3],
    lengths fp32 [E]) with vectors = positions[row_b] - positions[row_a] + shifts evaluated in fp64.
    Differentiable in positions and shifts; the backward scatters edge gradients to atoms over the CSR of row_a
    and the sorted view of row_b (the same index structures message passing uses), in fp64, without atomics."""

    @staticmethod
    def forward(ctx, positions, shifts, row_a, row_b):
        _require(row_a.dtype == I32 and row_b.dtype == I32, "edge geometry: int32 edge lists expected")
        _require(positions.dim() == 2 and positions.shape[1] == 3, "edge geometry: positions must be [nnodes, 3]")
        pos64 = positions.detach().double().contiguous()
        sh64 = shifts.detach().double().contiguous()
        vec, length = cabi.edge_geometry_forward(pos64, row_a, row_b, sh64)
        ctx.save_for_backward(pos64, sh64, row_a, row_b)
        ctx.dtypes = (positions.dtype, shifts.dtype)
        ctx.mark_non_differentiable()
        return vec, length

    @staticmethod
    def backward(ctx, grad_vec, grad_len):
        pos64, sh64, row_a, row_b = ctx.saved_tensors
        need_pos, need_shift = ctx.needs_input_grad[:2]
        nnodes = pos64.shape[0]
        first_occ = csr_of(row_a, nnodes)
        perm, off = sender_view_of(row_b, nnodes)
        gv = grad_vec.contiguous() if grad_vec is not None else None
        gl = grad_len.contiguous() if grad_len is not None else None
        gpos, gshift = cabi.edge_geometry_backward(pos64, row_a, row_b, sh64, first_occ, perm, off, gv, gl,
                                                   need_positions=need_pos, need_shifts=need_shift)
        if gpos is not None:
            gpos = gpos.to(ctx.dtypes[0])
        if gshift is not None:
            gshift = gshift.to(ctx.dtypes[1])
        return gpos, gshift, None, None


# ------------------------------------------------------------------------------------------------
class SphericalHarmonicsAutograd(torch.autograd.Function):
    @staticmethod
    def forward(ctx, xyz):
        _require(xyz.dtype == F32, "spherical harmonics: fp32 input expected")
        _require(xyz.dim() == 2 and xyz.shape[1] == 3, "spherical harmonics: xyz must be [nedges, 3]")
        x = xyz.contiguous()
        ctx.save_for_backward(x)
        return cabi.sh_forward(x)

    @staticmethod
    def backward(ctx, grad_Y):
        (x,) = ctx.saved_tensors
        return cabi.sh_backward(x, grad_Y.contiguous())


# ------------------------------------------------------------------------------------------------
class CubicSplineAutograd(torch.autograd.Function):
    @staticmethod
    def forward(ctx, r, r_knots, coeffs, r_width, r_max):
        _require(r.dtype == F32 and r_knots.dtype == F32 and coeffs.dtype == F32, "cubic spline: fp32 tensors expected")
        rc = r.contiguous().view(-1)
        ctx.save_for_backward(rc, r_knots, coeffs)
        ctx.r_width, ctx.r_max, ctx.r_shape = float(r_width), float(r_max), r.shape
        return cabi.spline_forward(rc, r_knots, coeffs, r_width, r_max)

    @staticmethod
    def backward(ctx, grad_R):
        r, r_knots, coeffs = ctx.saved_tensors
        g = cabi.spline_backward(r, r_knots, coeffs, grad_R.contiguous(), ctx.r_width, ctx.r_max)
        return g.view(ctx.r_shape), None, None, None, None


# ------------------------------------------------------------------------------------------------
class LinearAutograd(torch.autograd.Function):
    @staticmethod
    def forward(ctx, X, W, W_T):
        _require(X.dtype == F32 and W.dtype == F32 and W_T.dtype == F32, "linear: fp32 tensors expected")
        _require(X.dim() == 3 and X.shape[1] == 16, "linear: X must be [nnodes, 16, K]")
        ctx.save_for_backward(W)
        ctx.scale = 1.0 / float(X.shape[2]) ** 0.5
        return cabi.linear(X.contiguous(), W_T, scale=ctx.scale)

    @staticmethod
    def backward(ctx, grad_out):
        (W,) = ctx.saved_tensors
        # dX = scale * g . W^T: the operand the kernel wants is the transpose of W^T, i.e. W itself
        return cabi.linear(grad_out.contiguous(), W, scale=ctx.scale), None, None


class ElementalLinearAutograd(torch.autograd.Function):
    @staticmethod
    def forward(ctx, X, W, W_T, one_hot_encoding):
        _require(X.dtype == F32 and W.dtype == F32 and W_T.dtype == F32, "elemental linear: fp32 tensors expected")
        _require((X.dim() == 3 and X.shape[1] == 16) or X.dim() == 2, "elemental linear: X must be [nnodes, 16, K] or [nnodes, K]")
        _require(one_hot_encoding.dim() == 2 and one_hot_encoding.shape[1] == W.shape[0],
                 "elemental linear: one_hot must be [nnodes, nelements]")
        perm, off = groups_of_one_hot(one_hot_encoding)
        ctx.save_for_backward(W, perm, off)
        ctx.scale = 1.0 / float(X.shape[-1]) ** 0.5
        return cabi.linear(X.contiguous(), W_T, perm, off, scale=ctx.scale, zero_last_group=True)

    @staticmethod
    def backward(ctx, grad_out):
        W, perm, off = ctx.saved_tensors
        return cabi.linear(grad_out.contiguous(), W, perm, off, scale=ctx.scale, zero_last_group=True), None, None, None


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


class SymmetricContractionAutograd(torch.autograd.Function):
    @staticmethod
    def forward(ctx, X, atom_types, U3_max_nonsparse, U3_num_nonzero, U3_indices, U3_values, U2_num_nonzero,
                U2_indices, U2_values, U1_num_nonzero, U1_index, W3, W2, W1, W3_size, W2_size, W1_size):
        _require(X.dtype == F32 and W3.dtype == F32, "symmetric contraction: fp32 tensors expected")
        _require(X.dim() == 3 and X.shape[1] == 16 and X.shape[2] % 32 == 0,
                 "symmetric contraction: X must be [nnodes, 16, C] with C % 32 == 0")
        _require(atom_types.dtype == I32, "symmetric contraction: int32 atom_types expected")
        # element indices must lie in [0, nelements), as in the reference (which would read weights out of bounds
        # otherwise); rows of nodes with an index outside that range are left unwritten here
        dev = X.device

        def build_structure():
            (m3, o3, p3, v3), (m2, o2, p2, v2) = monomials_from_packed(
                U3_num_nonzero, U3_indices, U3_values, U2_num_nonzero, U2_indices, U2_values)
            b3, b2 = cabi.symcon_builtin_structure()
            builtin = bool(np.array_equal(m3, b3) and np.array_equal(m2, b2))
            return tuple(torch.from_numpy(a).to(dev) for a in (m3, o3, p3, v3, m2, o2, p2, v2)) + (builtin,)

        key = tuple((t.data_ptr(), t._version) for t in (U3_num_nonzero, U3_values, U2_num_nonzero, U2_indices, U2_values))
        m3, o3, p3, v3, m2, o2, p2, v2, builtin = _cached(U3_indices, "_cm_monomials", key, build_structure)

        # weights are [nlout = 1, nelements, npaths, C]; only the scalar output block exists
        w3 = W3.reshape(-1, W3.shape[-2], W3.shape[-1])[:, : int(W3_size)].contiguous()
        w2 = W2.reshape(-1, W2.shape[-2], W2.shape[-1])[:, : int(W2_size)].contiguous()
        w1 = W1.reshape(-1, W1.shape[-2], W1.shape[-1])[:, : int(W1_size)].contiguous()
        ne = w3.shape[0]
        wkey = tuple((t.data_ptr(), t._version) for t in (W2, W1)) + (int(W3_size), int(W2_size), int(W1_size), key)
        T3, T2, T1 = _cached(W3, "_cm_tables", wkey, lambda: cabi.symcon_tables(o3, p3, v3, o2, p2, v2, w3, w2, w1))

        perm, off = groups_of(atom_types, ne)
        want_grad = X.requires_grad
        out, grad = cabi.symcon_forward(X.contiguous(), perm, off, m3, m2, T3, T2, T1, want_grad=want_grad, builtin=builtin, zero_init=False)
        if want_grad:
            ctx.save_for_backward(grad)
        return out.view(X.shape[0], 1, X.shape[2])

    @staticmethod
    def backward(ctx, grad_out):
        (grad,) = ctx.saved_tensors
        N, _, C = grad.shape
        gX = cabi.symcon_backward(grad, grad_out.contiguous().view(N, C))
        return (gX,) + (None,) * 16
