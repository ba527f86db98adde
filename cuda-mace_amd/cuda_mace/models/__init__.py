from .InvariantMACE import OptimizedInvariantMACE  # noqa: F401
from .upstream_like import SyntheticInvariantMACE  # noqa: F401
