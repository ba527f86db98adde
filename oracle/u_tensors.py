"""Coupling tensors of the scalar-output symmetric contraction from Wigner 3j symbols.
TEST INFRASTRUCTURE ONLY.

Independent derivation of what the reference takes from upstream `mace.tools.cg.U_matrix_real`
(ops/symmetric_contraction.py:29-34): sympy's complex-basis Wigner 3j symbols are rotated into the real
spherical-harmonic basis (order m = -l..l, no Condon-Shortley sign in the real functions:
m > 0: sqrt2 (-1)^m Re Y_l^m, m < 0: sqrt2 (-1)^m Im Y_l^|m|), normalised to unit Frobenius norm per
path, and given the sign that makes the first non-zero entry positive.  Path order: lexicographic in
(l1, l2, l3).  The order and sign that upstream mace uses are PARITY UNPINNED (package unavailable
offline); they do not affect models with randomly initialised weights.
"""
from __future__ import annotations

import math
from functools import lru_cache

import numpy as np


def _real_from_complex(l: int) -> np.ndarray:
    """Q[m_real + l, m_complex + l] with Y^real_m = sum_m' Q[m, m'] Y_l^m'."""
    Q = np.zeros((2 * l + 1, 2 * l + 1), dtype=complex)
    Q[l, l] = 1.0
    for mu in range(1, l + 1):
        s = (-1.0) ** mu
        Q[l + mu, l + mu] = s / math.sqrt(2)
        Q[l + mu, l - mu] = 1 / math.sqrt(2)
        Q[l - mu, l + mu] = s / (math.sqrt(2) * 1j)
        Q[l - mu, l - mu] = -1 / (math.sqrt(2) * 1j)
    return Q


def _real_w3j(l1: int, l2: int, l3: int) -> np.ndarray:
    from sympy.physics.wigner import wigner_3j

    w = np.zeros((2 * l1 + 1, 2 * l2 + 1, 2 * l3 + 1))
    for m1 in range(-l1, l1 + 1):
        for m2 in range(-l2, l2 + 1):
            m3 = -m1 - m2
            if abs(m3) <= l3:
                w[m1 + l1, m2 + l2, m3 + l3] = float(wigner_3j(l1, l2, l3, m1, m2, m3))
    Q1, Q2, Q3 = (np.conj(_real_from_complex(l)) for l in (l1, l2, l3))
    t = np.einsum("abc,ia,jb,kc->ijk", w, Q1, Q2, Q3)
    # even l1+l2+l3: the real-basis tensor is real
    assert np.abs(t.imag).max() < 1e-12
    return t.real


def coupling_paths(lmax: int = 3):
    return [
        (l1, l2, l3)
        for l1 in range(lmax + 1)
        for l2 in range(lmax + 1)
        for l3 in range(lmax + 1)
        if abs(l1 - l2) <= l3 <= l1 + l2 and (l1 + l2 + l3) % 2 == 0
    ]


@lru_cache(maxsize=None)
def u_tensors():
    """(U1 [16,1], U2 [16,16,4], U3 [16,16,16,23]) as float64 numpy arrays."""
    paths = coupling_paths(3)
    U3 = np.zeros((16, 16, 16, len(paths)))
    for p, (l1, l2, l3) in enumerate(paths):
        t = _real_w3j(l1, l2, l3)
        t[np.abs(t) < 1e-12] = 0.0
        t /= np.linalg.norm(t)
        first = t.ravel()[np.flatnonzero(t.ravel())[0]]
        t *= 1.0 if first > 0 else -1.0
        U3[l1 * l1:(l1 + 1) ** 2, l2 * l2:(l2 + 1) ** 2, l3 * l3:(l3 + 1) ** 2, p] = t
    U2 = np.zeros((16, 16, 4))
    for l in range(4):
        # unit-norm invariant of l x l -> 0: delta_ij / sqrt(2l+1)
        for i in range(l * l, (l + 1) ** 2):
            U2[i, i, l] = 1.0 / math.sqrt(2 * l + 1)
    U1 = np.zeros((16, 1))
    U1[0, 0] = 1.0
    return U1, U2, U3
