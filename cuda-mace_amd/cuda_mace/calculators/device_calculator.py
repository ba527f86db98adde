"""Energy and forces for a molecular-dynamics driver, everything on the GPU.

The reference stops at the model: its users get `edge_index` / `shifts` from upstream's host-side neighbour search
(tests/test_utils.py:62-105) and call `OptimizedInvariantMACE.forward` (tools/model_surgery.py:217-229 times exactly
that).  This class strings the device-side pieces together the way an MD code does:

  * a Verlet list: neighbours within cutoff + skin, rebuilt on the GPU only when some atom has moved more than
    skin / 2 since the last build (one scalar leaves the GPU per step for that test).  Pairs between cutoff and
    cutoff + skin contribute exact zeros (the radial spline vanishes beyond r_max), so results do not depend on
    the skin;
  * between rebuilds the step runs as one HIP graph (utils/graph.py), re-captured after every rebuild.
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence

import torch

from cuda_mace.utils.graph import GraphedStep
from cuda_mace.utils.neighbour_list import get_neighborhood


class DeviceCalculator:
    def __init__(self, model: torch.nn.Module, node_attrs: torch.Tensor, cutoff: Optional[float] = None, skin: float = 0.5,
                 pbc: Sequence[bool] = (False, False, False), cell: Optional[torch.Tensor] = None,
                 use_graph: Optional[bool] = None, compute_stress: bool = False):
        """use_graph: replay the step as one HIP graph between list rebuilds.  None decides by size: up to 8192 atoms the
        step is bound by host launches and the graph pays for its re-capture after a rebuild; larger systems are bound
        by the GPU and run eagerly."""
        self.model = model
        self.node_attrs = node_attrs
        self.cutoff = float(model.r_max) if cutoff is None else float(cutoff)
        self.skin = float(skin)
        self.pbc = tuple(bool(b) for b in pbc)
        self.cell = None if cell is None else cell.detach().double().reshape(3, 3).contiguous()
        if use_graph is None:
            use_graph = node_attrs.shape[0] <= 8192
        self.use_graph = bool(use_graph) and not compute_stress  # the strain path re-derives shifts from the cell
        self.compute_stress = bool(compute_stress)
        self.builds = 0
        self.steps = 0
        self._ref_positions: Optional[torch.Tensor] = None
        self._data: Optional[Dict[str, torch.Tensor]] = None
        self._graph: Optional[GraphedStep] = None

    # -- Verlet list ---------------------------------------------------------------------------------------
    def _needs_rebuild(self, positions: torch.Tensor) -> bool:
        if self._ref_positions is None or self._ref_positions.shape != positions.shape:
            return True
        moved2 = ((positions - self._ref_positions) ** 2).sum(dim=1).max()
        return bool(moved2 > (0.5 * self.skin) ** 2)

    def _rebuild(self, positions: torch.Tensor) -> None:
        pos = positions.detach().double().contiguous()
        edge_index, shifts, unit_shifts, cell = get_neighborhood(pos, self.cutoff + self.skin, self.pbc, self.cell)
        n = pos.shape[0]
        dev = pos.device
        self._data = {
            "positions": pos.clone(), "node_attrs": self.node_attrs, "edge_index": edge_index, "shifts": shifts,
            "unit_shifts": unit_shifts, "cell": cell, "batch": torch.zeros(n, dtype=torch.int64, device=dev),
            "ptr": torch.tensor([0, n], dtype=torch.int64, device=dev),
        }
        self._ref_positions = pos.clone()
        self._graph = GraphedStep(self.model, self._data, warmup=1) if self.use_graph else None
        self.builds += 1

    # -- evaluation ----------------------------------------------------------------------------------------
    def compute(self, positions: torch.Tensor) -> Dict[str, torch.Tensor]:
        """energy [1], forces [N, 3] (and virials / stress when asked for) at `positions` (fp64, on the GPU)."""
        positions = positions.detach().double()
        if self._needs_rebuild(positions):
            self._rebuild(positions)
        self.steps += 1
        if self._graph is not None:
            return self._graph(positions)
        data = dict(self._data)
        data["positions"] = positions.clone()
        out = self.model(data, compute_virials=self.compute_stress, compute_stress=self.compute_stress)
        return {k: v.detach() for k, v in out.items() if isinstance(v, torch.Tensor)}
