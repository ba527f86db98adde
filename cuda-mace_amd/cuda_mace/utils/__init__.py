from .irreps import Instruction, Irrep, Irreps  # noqa: F401
