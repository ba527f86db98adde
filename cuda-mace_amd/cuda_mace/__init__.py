"""cuda_mace: the invariant-MACE hot path on AMD MI355X (gfx950).

Same import paths as the reference package (`cuda_mace.ops.*`, `cuda_mace.models.OptimizedInvariantMACE`);
the compute goes to hand-written HIP kernels in lib/libcuda_mace_hip.so.
"""
__version__ = "0.1.0"
