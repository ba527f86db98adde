from .ase_calculator import MACECalculator  # noqa: F401
from .device_calculator import DeviceCalculator  # noqa: F401
from .lammps_mace import LAMMPS_MACE  # noqa: F401
