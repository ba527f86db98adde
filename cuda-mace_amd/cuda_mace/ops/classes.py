"""The TorchScript custom classes of the reference, served by lib/libcuda_mace.so.

The reference registers six classes through TORCH_LIBRARY and reaches them as
`torch.classes.<namespace>.<Class>()` (src/invariant_message_passing.cpp:73-90,
src/spherical_harmonics.cpp:52-69, src/cubic_spline.cpp:54-68, src/linear.cpp:105-137,
src/symmetric_contraction.cpp:124-158).  Here the same namespaces, class names, method schemas (including the
reference's spelling `raidal`) and empty pickle state are registered by csrc/torch_classes.cpp, whose forward and
backward call the C ABI of the HIP kernel library.  This module loads that library the way the reference does
(`torch.classes.load_library`, ops/__init__.py:7-15) and re-exports the namespaces for convenience:

    classes.inv_message_passing.InvariantMessagePassingTP()   is   torch.classes.inv_message_passing.InvariantMessagePassingTP()
"""
from __future__ import annotations

import os

import torch

_HERE = os.path.realpath(os.path.dirname(__file__))


def _lib_path() -> str:
    path = os.path.join(_HERE, "..", "lib", "libcuda_mace.so")
    if os.path.isfile(path):
        return path
    raise ImportError("Could not find libcuda_mace shared library at " + path + "; build it with `python cuda-mace_amd/build.py`")


torch.classes.load_library(_lib_path())

inv_message_passing = torch.classes.inv_message_passing
spherical_harmonics = torch.classes.spherical_harmonics
cubic_spline = torch.classes.cubic_spline
linear_wmma = torch.classes.linear_wmma
symm_contract = torch.classes.symm_contract
