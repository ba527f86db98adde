"""Op wrappers with the reference's module names and call signatures.

Importing this package loads the HIP kernel library (the counterpart of the reference's
`torch.classes.load_library(lib/libcuda_mace.so)` in ops/__init__.py:7-15) and fails loudly if it
has not been built.
"""
from .. import _cabi  # noqa: F401  (raises ImportError when the library is missing)
from . import classes  # noqa: F401
from .cubic_spline import CubicSpline  # noqa: F401
from .invariant_message_passing import InvariantMessagePassingTP  # noqa: F401
from .linear import ElementalLinear, Linear  # noqa: F401
from .symmetric_contraction import SymmetricContraction  # noqa: F401
