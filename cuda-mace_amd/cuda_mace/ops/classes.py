"""Stateless op objects with the method schemas of the reference's TorchScript custom classes.

The reference registers six classes through TORCH_LIBRARY and reaches them as
`torch.classes.<namespace>.<Class>()` (src/invariant_message_passing.cpp:73-90,
src/spherical_harmonics.cpp:52-69, src/cubic_spline.cpp:54-68, src/linear.cpp:105-137,
src/symmetric_contraction.cpp:124-158).  The objects below keep namespace, class and argument
names (including the reference's spelling `raidal`) and the empty pickle state; each `forward` is one
autograd function whose forward and backward call the C ABI.
"""
from __future__ import annotations

from types import SimpleNamespace

import torch

from . import _autograd as A


class _Stateless:
    def __getstate__(self):
        return {}

    def __setstate__(self, state):
        return


class InvariantMessagePassingTP(_Stateless):
    def forward(self, X, Y, raidal, sender_list, receiver_list, nnodes):
        return A.InvariantMessagePassingTPAutograd.apply(X, Y, raidal, sender_list, receiver_list, int(nnodes))


class SphericalHarmonics(_Stateless):
    def forward(self, xyz):
        return A.SphericalHarmonicsAutograd.apply(xyz)


class CubicSpline(_Stateless):
    def forward(self, r, r_knots, coeffs, r_width, r_max):
        return A.CubicSplineAutograd.apply(r, r_knots, coeffs, float(r_width), float(r_max))


class Linear(_Stateless):
    def forward(self, X, W, W_T):
        return A.LinearAutograd.apply(X, W, W_T)


class ElementalLinear(_Stateless):
    def forward(self, X, W, W_T, one_hot_encoding):
        return A.ElementalLinearAutograd.apply(X, W, W_T, one_hot_encoding)


class SymmetricContraction(_Stateless):
    def forward(self, X, atom_types, U3_max_nonsparse, U3_num_nonzero, U3_indices, U3_values, U2_num_nonzero,
                U2_indices, U2_values, U1_num_nonzero, U1_index, W3, W2, W1, W3_size, W2_size, W1_size):
        return A.SymmetricContractionAutograd.apply(
            X, atom_types, int(U3_max_nonsparse), U3_num_nonzero, U3_indices, U3_values, U2_num_nonzero, U2_indices,
            U2_values, U1_num_nonzero, U1_index, W3, W2, W1, int(W3_size), int(W2_size), int(W1_size))


inv_message_passing = SimpleNamespace(InvariantMessagePassingTP=InvariantMessagePassingTP)
spherical_harmonics = SimpleNamespace(SphericalHarmonics=SphericalHarmonics)
cubic_spline = SimpleNamespace(CubicSpline=CubicSpline)
linear_wmma = SimpleNamespace(Linear=Linear, ElementalLinear=ElementalLinear)
symm_contract = SimpleNamespace(SymmetricContraction=SymmetricContraction)
