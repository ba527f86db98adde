"""ASE-protocol calculator over the optimised model.

The reference ships no calculator: its tool hands a test batch to `OptimizedInvariantMACE.forward` directly
(tools/model_surgery.py:145-234), and users of upstream MACE drive the model through an ASE calculator that builds
the neighbour list on the host for every call.  `MACECalculator` offers that calling convention on top of
`DeviceCalculator` (neighbour list, Verlet skin and HIP graph on the GPU): `atoms.calc = MACECalculator(model)`, then
`atoms.get_potential_energy()`, `atoms.get_forces()`, `atoms.get_stress()` work as with any ASE calculator.

ASE itself is not imported: the class speaks the calculator protocol (`calculate`, `get_potential_energy`,
`get_forces`, `get_stress`, `get_property`, `results`, `implemented_properties`) and reads the structure through the
`Atoms` accessors (`get_positions`, `get_atomic_numbers`, `get_cell`, `get_pbc`), so it accepts `ase.Atoms` where ASE
is installed and any object with those four methods elsewhere.  Units as in ASE: eV, eV/Angstrom, stress in
eV/Angstrom^3 as the six Voigt components (xx, yy, zz, yz, xz, xy).
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence

import numpy as np
import torch

from .device_calculator import DeviceCalculator


class MACECalculator:
    implemented_properties = ["energy", "free_energy", "forces", "stress"]

    def __init__(self, model: torch.nn.Module, device: str = "cuda", skin: float = 0.5, use_graph: Optional[bool] = None):
        self.model = model
        self.device = torch.device(device)
        self.skin = float(skin)
        self.use_graph = use_graph
        self.z_table = [int(z) for z in model.atomic_numbers.tolist()]
        self.results: Dict[str, np.ndarray] = {}
        self.atoms = None
        self._key = None          # (atomic numbers, cell, pbc, stress wanted) the device calculator was built for
        self._last = None         # positions of the last evaluation
        self._device_calc: Optional[DeviceCalculator] = None

    # -- structure -> device ---------------------------------------------------------------------------
    def _node_attrs(self, numbers: np.ndarray) -> torch.Tensor:
        index = np.full(int(max(self.z_table)) + 1, -1, dtype=np.int64)
        index[self.z_table] = np.arange(len(self.z_table))
        if numbers.max(initial=0) >= index.shape[0] or (index[numbers] < 0).any():
            unknown = sorted(set(int(z) for z in numbers) - set(self.z_table))
            raise ValueError("atomic numbers %s are not covered by the model (it knows %s)" % (unknown, self.z_table))
        one_hot = torch.zeros(numbers.shape[0], len(self.z_table), dtype=torch.float64)
        one_hot[torch.arange(numbers.shape[0]), torch.from_numpy(index[numbers])] = 1.0
        return one_hot.to(self.device)

    def _prepare(self, atoms, want_stress: bool) -> DeviceCalculator:
        numbers = np.asarray(atoms.get_atomic_numbers(), dtype=np.int64)
        cell = np.asarray(atoms.get_cell(), dtype=np.float64).reshape(3, 3)
        pbc = tuple(bool(b) for b in np.broadcast_to(np.asarray(atoms.get_pbc()), (3,)))
        key = (numbers.tobytes(), cell.tobytes(), pbc, want_stress)
        if key != self._key:
            if want_stress and not all(pbc):
                raise ValueError("stress needs a structure that is periodic along all three cell vectors")
            self._device_calc = DeviceCalculator(
                self.model, self._node_attrs(numbers), skin=self.skin, pbc=pbc,
                cell=torch.from_numpy(cell).to(self.device) if any(pbc) else None, use_graph=self.use_graph,
                compute_stress=want_stress)
            self._key = key
        return self._device_calc

    # -- calculator protocol ---------------------------------------------------------------------------
    def calculate(self, atoms=None, properties: Sequence[str] = ("energy",), system_changes=None) -> None:
        if atoms is None:
            atoms = self.atoms
        if atoms is None:
            raise ValueError("MACECalculator.calculate needs an atoms object")
        unknown = [p for p in properties if p not in self.implemented_properties]
        if unknown:
            raise NotImplementedError("properties %s are not implemented (available: %s)" % (unknown, self.implemented_properties))
        want_stress = "stress" in properties
        calc = self._prepare(atoms, want_stress or (self._key is not None and self._key[3]))
        positions = np.asarray(atoms.get_positions(), dtype=np.float64)
        out = calc.compute(torch.from_numpy(positions).to(self.device))
        energy = float(out["energy"].double().sum().cpu())
        self.results = {"energy": energy, "free_energy": energy, "forces": out["forces"].double().cpu().numpy()}
        if calc.compute_stress:
            s = out["stress"].double().reshape(3, 3).cpu().numpy()
            self.results["stress"] = np.array([s[0, 0], s[1, 1], s[2, 2], s[1, 2], s[0, 2], s[0, 1]])
        self.atoms = atoms
        self._last = (positions.copy(), self._key)

    def _fresh(self, atoms, name: str) -> bool:
        if self._last is None or name not in self.results:
            return False
        numbers = np.asarray(atoms.get_atomic_numbers(), dtype=np.int64)
        cell = np.asarray(atoms.get_cell(), dtype=np.float64).reshape(3, 3)
        pbc = tuple(bool(b) for b in np.broadcast_to(np.asarray(atoms.get_pbc()), (3,)))
        return (self._last[1][:3] == (numbers.tobytes(), cell.tobytes(), pbc)
                and np.array_equal(self._last[0], np.asarray(atoms.get_positions(), dtype=np.float64)))

    def get_property(self, name: str, atoms=None, allow_calculation: bool = True):
        atoms = self.atoms if atoms is None else atoms
        if name not in self.implemented_properties:
            raise NotImplementedError("property %r is not implemented" % name)
        if atoms is None or not self._fresh(atoms, name):
            if not allow_calculation:
                return None
            self.calculate(atoms, [name])
        value = self.results[name]
        return value.copy() if isinstance(value, np.ndarray) else value

    def get_potential_energy(self, atoms=None, force_consistent: bool = False) -> float:
        return self.get_property("free_energy" if force_consistent else "energy", atoms)

    def get_forces(self, atoms=None) -> np.ndarray:
        return self.get_property("forces", atoms)

    def get_stress(self, atoms=None) -> np.ndarray:
        return self.get_property("stress", atoms)

    def calculation_required(self, atoms, properties: Sequence[str]) -> bool:
        return any(not self._fresh(atoms, p) for p in properties)

    def reset(self) -> None:
        self.results = {}
        self._last = None
