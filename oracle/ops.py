"""fp64 CPU restatement of the reference's op semantics.  TEST INFRASTRUCTURE ONLY.

Every function works on CPU torch tensors (any float dtype; tests use fp64) and is
written from the mathematical definition, not from the kernels' loop structure.
Citations are relative to the reference tree.
"""
from __future__ import annotations

import math

import numpy as np
import torch

# l(m) for the 16 real spherical-harmonic components m = 0..15: floor(sqrt(m)).
L_OF_M = torch.tensor([0, 1, 1, 1, 2, 2, 2, 2, 2, 3, 3, 3, 3, 3, 3, 3], dtype=torch.long)


# ----------------------------------------------------------------------------------------
# index kernels (bit-exact)
# ----------------------------------------------------------------------------------------
def first_occurences(receiver: torch.Tensor, nnodes: int) -> torch.Tensor:
    """CSR offsets of a non-decreasing receiver list: out[n] = first edge of node n,
    out[nnodes + n] = one past its last edge.

    Follows cuda/src/invariant_message_passing_impl.cu:8-72 and
    jit_wrappers/src/invariant_message_passing_wrapper.cpp:19-70 for nodes that own at least
    one edge.  The reference leaves nodes without edges uninitialised; here they get the
    standard CSR convention start == end == insertion point.
    """
    r = receiver.detach().cpu().numpy().astype(np.int64)
    nodes = np.arange(nnodes, dtype=np.int64)
    start = np.searchsorted(r, nodes, side="left")
    end = np.searchsorted(r, nodes, side="right")
    return torch.from_numpy(np.concatenate([start, end]).astype(np.int32))


def stable_key_sort(keys: torch.Tensor, nkeys: int):
    """Stable counting sort of item indices by integer key in [0, nkeys).

    Returns (perm int32 [n], offsets int32 [nkeys + 1]) with keys[perm] non-decreasing, ties in
    original order, and offsets[k] = number of items whose key is < k.  This is the
    sender-sorted view of the edge list that replaces the reference's N x N reverse-edge map
    (jit_wrappers/src/invariant_message_passing_wrapper.cpp:91-93,
    cuda/src/invariant_message_passing_impl.cu:112-116, 331-336).
    """
    k = keys.detach().cpu().numpy().astype(np.int64)
    perm = np.argsort(k, kind="stable").astype(np.int32)
    counts = np.bincount(k, minlength=nkeys)
    offsets = np.zeros(nkeys + 1, dtype=np.int64)
    offsets[1:] = np.cumsum(counts)
    return torch.from_numpy(perm), torch.from_numpy(offsets.astype(np.int32))


# ----------------------------------------------------------------------------------------
# invariant message passing
# ----------------------------------------------------------------------------------------
def mp_forward(X, Y, R, sender, receiver, nnodes: int):
    """out[n, m, c] = sum_{e: receiver[e] = n} X[sender[e], c] * Y[m, e] * R[e, l(m), c].

    X [N, C], Y [16, E], R [E, 4, C] -> [N, 16, C] (R [E, 16, C]: one weight per component m instead of per degree
    l(m), a variant the reference does not have).  Definition of the op computed by
    cuda/src/invariant_message_passing_impl.cu:74-165 (no normalisation factor, Y laid out
    [16, E], one radial weight per l shared by its 2l+1 components), as the reference's own
    test builds it from a per-edge tensor product followed by a scatter-sum
    (tests/invariant_message_passing.py:93-120).  Nodes without edges give zero rows.
    """
    s = sender.long()
    r = receiver.long()
    Rm = R if R.shape[1] == 16 else R[:, L_OF_M, :]  # a weight per component, or the reference's weight per degree
    msg = X[s][:, None, :] * Y.t()[:, :, None] * Rm  # [E, 16, C]
    out = torch.zeros(nnodes, 16, X.shape[1], dtype=X.dtype)
    out.index_add_(0, r, msg)
    return out


def mp_backward(X, Y, R, grad_out, sender, receiver):
    """Closed-form gradients of mp_forward (the three outputs of
    cuda/src/invariant_message_passing_impl.cu:167-294 and :296-399):

      gR[e, l, c] = X[s_e, c] * sum_{m in l} Y[m, e] * g[r_e, m, c]
      gY[m, e]    = sum_c g[r_e, m, c] * R[e, l(m), c] * X[s_e, c]
      gX[n, c]    = sum_{e: s_e = n} sum_m g[r_e, m, c] * R[e, l(m), c] * Y[m, e]

    gX is written for an arbitrary directed multigraph; the reference finds the transposed
    edges through a symmetric-graph lookup instead.
    """
    s = sender.long()
    r = receiver.long()
    g = grad_out[r]  # [E, 16, C]
    Yt = Y.t()  # [E, 16]
    Xs = X[s]  # [E, C]
    if R.shape[1] == 16:  # a weight per component: no sum over the components of a degree
        yg = g * Yt[:, :, None]
        gX = torch.zeros_like(X)
        gX.index_add_(0, s, (R * yg).sum(1))
        return gX, (g * R * Xs[:, None, :]).sum(-1).t().contiguous(), Xs[:, None, :] * yg
    q = torch.zeros(R.shape, dtype=X.dtype)  # [E, 4, C]: sum_{m in l} Y g
    q.index_add_(1, L_OF_M, g * Yt[:, :, None])
    gR = Xs[:, None, :] * q
    gY = (g * R[:, L_OF_M, :] * Xs[:, None, :]).sum(-1).t().contiguous()
    gXe = (R * q).sum(1)  # [E, C]
    gX = torch.zeros_like(X)
    gX.index_add_(0, s, gXe)
    return gX, gY, gR


# ----------------------------------------------------------------------------------------
# real spherical harmonics l <= 3
# ----------------------------------------------------------------------------------------
def spherical_harmonics(xyz: torch.Tensor) -> torch.Tensor:
    """16 real spherical harmonics of the normalised edge vector, "component" normalised
    (sum_{m in l} Y_lm^2 = 2l + 1), laid out [16, E].

    Follows cuda/src/spherical_harmonics_impl.cu:56-127: the input columns are permuted to
    (x, y, z) = (in_2, in_0, in_1) and the standard real harmonics in the order m = -l..l are
    multiplied by sqrt(4 pi).  Constants are written in closed form rather than as the
    kernel's decimals.
    """
    v = xyz / xyz.norm(dim=-1, keepdim=True)
    x, y, z = v[:, 2], v[:, 0], v[:, 1]
    x2, y2, z2 = x * x, y * y, z * z
    s3, s5, s7, s15 = math.sqrt(3.0), math.sqrt(5.0), math.sqrt(7.0), math.sqrt(15.0)
    s105 = math.sqrt(105.0)
    out = [
        torch.ones_like(x),
        s3 * y,
        s3 * z,
        s3 * x,
        s15 * x * y,
        s15 * y * z,
        0.5 * s5 * (2 * z2 - x2 - y2),
        s15 * x * z,
        0.5 * s15 * (x2 - y2),
        math.sqrt(35.0 / 8.0) * y * (3 * x2 - y2),
        s105 * x * y * z,
        math.sqrt(21.0 / 8.0) * y * (4 * z2 - x2 - y2),
        0.5 * s7 * z * (2 * z2 - 3 * x2 - 3 * y2),
        math.sqrt(21.0 / 8.0) * x * (4 * z2 - x2 - y2),
        0.5 * s105 * z * (x2 - y2),
        math.sqrt(35.0 / 8.0) * x * (x2 - 3 * y2),
    ]
    return torch.stack(out, dim=0)


def spherical_harmonics_backward(xyz: torch.Tensor, grad_Y: torch.Tensor) -> torch.Tensor:
    """d/dxyz of sum(grad_Y * spherical_harmonics(xyz)) by autograd; what
    cuda/src/spherical_harmonics_impl.cu:239-268 and :284-334 compute through the stored
    Jacobian (derivative with respect to the un-normalised input, in input axis order)."""
    x = xyz.detach().clone().requires_grad_(True)
    (spherical_harmonics(x) * grad_Y).sum().backward()
    return x.grad


# ----------------------------------------------------------------------------------------
# cubic spline
# ----------------------------------------------------------------------------------------
def spline_coefficients(r_knots: torch.Tensor, R: torch.Tensor) -> torch.Tensor:
    """Natural cubic spline through (r_knots[k], R[k, :]) as coefficients[k, (a, b, c, d), j] of
    a + b x + c x^2 + d x^3 with x = r - r_knots[k]; same quantity as
    ops/cubic_spline.py:41-84, obtained here from scipy."""
    from scipy.interpolate import CubicSpline

    cs = CubicSpline(r_knots.double().numpy(), R.double().numpy(), axis=0, bc_type="natural")
    c = torch.from_numpy(np.ascontiguousarray(cs.c))  # [4, K-1, J], highest power first
    return torch.stack([c[3], c[2], c[1], c[0]], dim=1).contiguous()


def spline_eval(r, r_knots, coeffs, r_width: float, r_max: float, deriv: bool = False):
    """R[e, j] (and dR/dr) from the coefficient table; zero beyond r_max.
    Follows cuda/src/cubic_spline_impl.cu:5-66."""
    nint = coeffs.shape[0]
    idx = torch.clamp((r / r_width).floor().long(), 0, nint - 1)
    x = (r - r_knots[idx])[:, None]
    a, b, c, d = (coeffs[idx, k, :] for k in range(4))
    inside = (r <= r_max)[:, None].to(r.dtype)
    val = (a + x * (b + x * (c + x * d))) * inside
    if not deriv:
        return val
    der = (b + x * (2 * c + 3 * x * d)) * inside
    return val, der


def spline_backward(grad_R, dR):
    """dr[e] = sum_j grad_R[e, j] * dR[e, j]; cuda/src/cubic_spline_impl.cu:68-107."""
    return (grad_R * dR).sum(-1)


# ----------------------------------------------------------------------------------------
# channel-mixing linears
# ----------------------------------------------------------------------------------------
def linear(X, W):
    """OUT[n, m, :] = X[n, m, :] @ W[l(m)] / sqrt(K); X [N, 16, K], W [4, K, K'].
    cuda/src/linear_impl.cu:16-133 (path weight at :33)."""
    K = X.shape[-1]
    return torch.einsum("nmk,mkj->nmj", X, W[L_OF_M]) / math.sqrt(K)


def elemental_linear(X, W, one_hot):
    """As linear() with the weight block of the node's element: W [ne, 4, K, K'], element of
    node n = the column where one_hot[n] == 1 (jit_wrappers/src/linear_wrapper.cpp:137-145,
    cuda/src/linear_impl.cu:134-255).  Rows with no such column give zeros."""
    K = X.shape[-1]
    has = (one_hot == 1).any(dim=1)
    elem = (one_hot == 1).to(torch.int8).argmax(dim=1)
    Wn = W[elem][:, L_OF_M]  # [N, 16, K, K']
    out = torch.einsum("nmk,nmkj->nmj", X, Wn) / math.sqrt(K)
    return out * has[:, None, None].to(X.dtype)


# ----------------------------------------------------------------------------------------
# symmetric contraction (correlation 3, scalar output)
# ----------------------------------------------------------------------------------------
def unpack_u_tables(U3_num, U3_idx, U3_val, U2_num, U2_idx, U2_val, n_paths3: int, n_paths2: int):
    """Dense U3 [16,16,16,P3] and U2 [16,16,P2] from the packed tables built by
    ops/symmetric_contraction.py:91-187 (index word: bits 0-7 weight path, bits 8-15 k)."""
    U3 = torch.zeros(16, 16, 16, n_paths3, dtype=torch.float64)
    U2 = torch.zeros(16, 16, n_paths2, dtype=torch.float64)
    for i in range(16):
        for j in range(16):
            for t in range(int(U3_num[i, j])):
                word = int(U3_idx[t, i, j])
                U3[i, j, (word >> 8) & 0xFF, word & 0xFF] = float(U3_val[t, i, j])
            if int(U2_num[i, j]) > 0:
                U2[i, j, int(U2_idx[i, j])] = float(U2_val[i, j])
    return U3, U2


def symmetric_contraction(X, atom_types, U3, U2, W3, W2, W1):
    """out[n, c] = sum_ijk,p U3[i,j,k,p] W3[e_n,p,c] x_i x_j x_k
                 + sum_ij,p  U2[i,j,p]   W2[e_n,p,c] x_i x_j
                 +           W1[e_n,0,c] x_0,             x_i = X[n, i, c].

    X [N, 16, C]; U3/U2 dense (see unpack_u_tables); W3 [ne, P3, C], W2 [ne, P2, C],
    W1 [ne, 1, C].  The forward value of cuda/src/symmetric_contraction_impl.cu:108-196.
    Its gradient with respect to X is taken by torch.autograd on this expression.
    """
    e = atom_types.long()
    U3 = U3.to(X.dtype)
    U2 = U2.to(X.dtype)
    c3 = torch.einsum("ijkp,npc->nijkc", U3, W3[e])
    out = torch.einsum("nijkc,nic,njc,nkc->nc", c3, X, X, X)
    c2 = torch.einsum("ijp,npc->nijc", U2, W2[e])
    out = out + torch.einsum("nijc,nic,njc->nc", c2, X, X)
    out = out + W1[e][:, 0, :] * X[:, 0, :]
    return out


# ----------------------------------------------------------------------------------------
# edge geometry
# ----------------------------------------------------------------------------------------
def edge_geometry(positions, row_a, row_b, shifts):
    """vectors = positions[row_b] - positions[row_a] + shifts and their lengths; the upstream helper the reference
    model calls at models/InvariantMACE.py:297-301.  Gradients by torch.autograd on this expression."""
    vec = positions[row_b.long()] - positions[row_a.long()] + shifts
    return vec, vec.norm(dim=-1)


# -----------------------------------------------------------------------------------------------
def neighbour_list(positions: np.ndarray, cell, pbc, cutoff: float):
    """All ordered pairs (i, j, S) with |r_j - r_i + S . cell| < cutoff and (j, S) != (i, 0), sorted by
    (i, j, Sx, Sy, Sz): what the upstream host-side neighbour search hands the reference's model
    (models/InvariantMACE.py:297-301 consumes edge_index / shifts; tests/test_utils.py:62-105 builds them through the
    upstream data loader).  Brute force over all atom pairs and all images that can reach; the accept test is
    evaluated term by term in fp64,
        v = (r_j - r_i) + ((Sx c0 + Sy c1) + Sz c2),   (v0 v0 + v1 v1) + v2 v2 < cutoff^2.
    Returns (edge_index int64 [2, E], unit_shifts int64 [E, 3])."""
    pos = np.asarray(positions, dtype=np.float64).reshape(-1, 3)
    n = pos.shape[0]
    pbc = np.array([bool(b) for b in pbc])
    c = np.zeros((3, 3)) if cell is None else np.asarray(cell, dtype=np.float64).reshape(3, 3)
    if pbc.any():
        inv = np.linalg.inv(c)
        heights = 1.0 / np.linalg.norm(inv, axis=0)
        reach = np.where(pbc, np.ceil(cutoff / heights).astype(np.int64) + 1, 0)
    else:
        inv = np.zeros((3, 3))
        reach = np.zeros(3, dtype=np.int64)
    rows = []
    rc2 = cutoff * cutoff
    offsets = np.array([(a, b, d) for a in range(-reach[0], reach[0] + 1) for b in range(-reach[1], reach[1] + 1)
                        for d in range(-reach[2], reach[2] + 1)], dtype=np.int64)
    for i in range(n):
        d = pos - pos[i]                                     # r_j - r_i, [n, 3]
        # image that brings the pair closest in fractional terms, then every image within reach of it
        S0 = np.where(pbc, -np.round(d @ inv), 0).astype(np.int64)          # [n, 3]
        S = S0[:, None, :] + offsets[None, :, :]                              # [n, n_img, 3]
        Sf = S.astype(np.float64)
        d2 = 0.0
        for k in range(3):
            shift = (Sf[..., 0] * c[0, k] + Sf[..., 1] * c[1, k]) + Sf[..., 2] * c[2, k]
            v = d[:, None, k] + shift
            d2 = v * v if k == 0 else d2 + v * v
        hit = d2 < rc2
        hit[i] &= ~np.all(S[i] == 0, axis=-1)
        j, img = np.nonzero(hit)
        for jj, im in zip(j, img):
            rows.append((i, jj, S[jj, im, 0], S[jj, im, 1], S[jj, im, 2]))
    if not rows:
        return np.zeros((2, 0), dtype=np.int64), np.zeros((0, 3), dtype=np.int64)
    arr = np.array(sorted(set(rows)), dtype=np.int64)
    assert arr.shape[0] == len(rows), "an image was visited twice"
    return arr[:, :2].T.copy(), arr[:, 2:].copy()


# -----------------------------------------------------------------------------------------------
def readout_energies(h1, h2, w1, W2a, w2b, act_cst: float, scale: float, shift: float):
    """Node energies of the two readouts the reference's model applies in fp64 to the per-layer node features
    (models/InvariantMACE.py:330-337: linear readout of layer 1, one-hidden-layer readout with a normalised silu gate
    of layer 2) followed by scale and shift (:343).  Weights come with their 1/sqrt(fan_in) folded in."""
    h1, h2 = h1.double(), h2.double()
    z = h2 @ W2a.double()
    return scale * (h1 @ w1.double() + (act_cst * torch.nn.functional.silu(z)) @ w2b.double()) + shift
