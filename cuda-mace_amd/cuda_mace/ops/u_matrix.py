"""Coupling tensors of the symmetric contraction for scalar (0e) output, l <= 3 inputs.

The reference obtains them from upstream `mace.tools.cg.U_matrix_real` (ops/symmetric_contraction.py:29-34),
which is not a dependency here.  For a scalar output each coupling path (l1, l2, l3) carries the
unique rotation-invariant 3-tensor of unit Frobenius norm.  Because l1 + l2 + l3 is even on every
such path, that tensor is proportional to the integral over the sphere of the product of the three
real spherical harmonics -- in exactly the component basis and axis convention the spherical-harmonics
kernel uses -- so it is computed here by an exact quadrature of those functions.

Conventions fixed here (upstream's cannot be checked offline; they only matter when weights trained
upstream are loaded): paths are ordered lexicographically in (l1, l2, l3); the sign of each path makes
its first non-zero entry (lexicographic in i, j, k) positive.
"""
from __future__ import annotations

import math
from functools import lru_cache
from typing import List, Tuple

import numpy as np
import torch


def real_sh_l3(xyz: np.ndarray) -> np.ndarray:
    """[P, 3] vectors -> [P, 16] component-normalised real harmonics with the kernels' axis
    convention (x, y, z) = (in[2], in[0], in[1])."""
    v = xyz / np.linalg.norm(xyz, axis=1, keepdims=True)
    x, y, z = v[:, 2], v[:, 0], v[:, 1]
    x2, y2, z2 = x * x, y * y, z * z
    s3, s5, s7, s15, s105 = math.sqrt(3), math.sqrt(5), math.sqrt(7), math.sqrt(15), math.sqrt(105)
    a, b = math.sqrt(35 / 8), math.sqrt(21 / 8)
    cols = [
        np.ones_like(x), s3 * y, s3 * z, s3 * x,
        s15 * x * y, s15 * y * z, 0.5 * s5 * (2 * z2 - x2 - y2), s15 * x * z, 0.5 * s15 * (x2 - y2),
        a * y * (3 * x2 - y2), s105 * x * y * z, b * y * (4 * z2 - x2 - y2),
        0.5 * s7 * z * (2 * z2 - 3 * x2 - 3 * y2), b * x * (4 * z2 - x2 - y2), 0.5 * s105 * z * (x2 - y2),
        a * x * (x2 - 3 * y2),
    ]
    return np.stack(cols, axis=1)


def _sphere_quadrature(n_theta: int = 16, n_phi: int = 32):
    """Nodes and weights (summing to 1) exact for polynomials of degree < 2*n_theta and < n_phi."""
    ct, wt = np.polynomial.legendre.leggauss(n_theta)
    phi = (np.arange(n_phi) + 0.5) * (2 * math.pi / n_phi)
    st = np.sqrt(1 - ct * ct)
    pts = np.stack(
        [np.outer(st, np.cos(phi)).ravel(), np.outer(st, np.sin(phi)).ravel(), np.outer(ct, np.ones(n_phi)).ravel()],
        axis=1,
    )
    w = np.outer(wt, np.full(n_phi, 1.0 / n_phi)).ravel() / 2.0
    return pts, w


def coupling_paths(lmax: int = 3) -> List[Tuple[int, int, int]]:
    """(l1, l2, l3) with |l1-l2| <= l3 <= l1+l2 and even sum, lexicographic: 23 paths for lmax = 3."""
    return [
        (l1, l2, l3)
        for l1 in range(lmax + 1)
        for l2 in range(lmax + 1)
        for l3 in range(lmax + 1)
        if abs(l1 - l2) <= l3 <= l1 + l2 and (l1 + l2 + l3) % 2 == 0
    ]


@lru_cache(maxsize=None)
def _u_tensors_np():
    pts, w = _sphere_quadrature()
    Y = real_sh_l3(pts)  # [P, 16]
    gaunt = np.einsum("p,pi,pj,pk->ijk", w, Y, Y, Y)
    paths = coupling_paths(3)
    U3 = np.zeros((16, 16, 16, len(paths)))
    for p, (l1, l2, l3) in enumerate(paths):
        blk = np.zeros((16, 16, 16))
        s1, s2, s3_ = slice(l1 * l1, (l1 + 1) ** 2), slice(l2 * l2, (l2 + 1) ** 2), slice(l3 * l3, (l3 + 1) ** 2)
        blk[s1, s2, s3_] = gaunt[s1, s2, s3_]
        blk[np.abs(blk) < 1e-12] = 0.0
        blk /= np.linalg.norm(blk)
        first = blk.ravel()[np.flatnonzero(blk.ravel())[0]]
        U3[..., p] = blk * (1.0 if first > 0 else -1.0)
    U2 = np.zeros((16, 16, 4))
    for l in range(4):
        for i in range(l * l, (l + 1) ** 2):
            U2[i, i, l] = 1.0 / math.sqrt(2 * l + 1)
    U1 = np.zeros((16, 1))
    U1[0, 0] = 1.0
    return U1, U2, U3


def U_matrix_real(irreps_in=None, irreps_out=None, correlation: int = 3, dtype=torch.float32):
    """Same call shape as upstream's function: returns a list whose last item is the coupling tensor of
    the requested correlation order, [16]*correlation + [num_paths].  Only 0e+1o+2e+3o inputs and a
    single 0e output are supported (the invariant model)."""
    if irreps_in is not None and int(getattr(irreps_in, "lmax", 3)) != 3:
        raise NotImplementedError("coupling tensors are provided for l_max = 3 inputs only")
    if irreps_out is not None and str(irreps_out).replace("1x", "") != "0e":
        raise NotImplementedError("coupling tensors are provided for a scalar (0e) output only")
    if correlation not in (1, 2, 3):
        raise NotImplementedError("correlation must be 1, 2 or 3")
    U = _u_tensors_np()[correlation - 1]
    return [str(irreps_out) if irreps_out is not None else "0e", torch.from_numpy(U.copy()).to(dtype)]
