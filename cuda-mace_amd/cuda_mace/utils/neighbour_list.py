"""Neighbour list on the GPU, in the format the model's `data` dictionary takes.

Upstream builds the list on the host (`get_neighborhood(positions, cutoff, pbc, cell)` inside its data pipeline; the
reference reaches it through the data loader, tests/test_utils.py:62-105).  Here the same quantities come from the
device kernels behind `cm_neighbour_list_count / _fill`:

    edge_index   int64 [2, E]   row 0 = centre atom i (non-decreasing), row 1 = neighbour j,
                                sorted lexicographically by (i, j, Sx, Sy, Sz)
    unit_shifts  fp64  [E, 3]   integer image S of the neighbour
    shifts       fp64  [E, 3]   S . cell, so that  vector = positions[j] - positions[i] + shifts

Every pair with |vector| < cutoff is listed, including periodic images of an atom with itself when the cell is
smaller than the cutoff; (i, i, S = 0) is not.
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence, Tuple

import torch

from cuda_mace import _cabi as cabi


def _cell_and_pbc(cell, pbc, device) -> Tuple[Optional[torch.Tensor], Tuple[bool, bool, bool]]:
    if pbc is None:
        pbc = (False, False, False)
    if isinstance(pbc, bool):
        pbc = (pbc, pbc, pbc)
    pbc = tuple(bool(b) for b in pbc)
    if len(pbc) != 3:
        raise ValueError("pbc must hold three flags")
    if cell is None:
        if any(pbc):
            raise ValueError("a periodic axis needs a cell")
        return None, pbc
    cell = torch.as_tensor(cell, dtype=torch.float64, device=device).reshape(3, 3).contiguous()
    return cell, pbc


def shifts_from_unit_shifts(unit_shifts: torch.Tensor, cell: Optional[torch.Tensor]) -> torch.Tensor:
    """S . cell evaluated term by term in the order the neighbour search itself uses (no matrix-multiply kernel,
    whose summation order is unspecified)."""
    S = unit_shifts.double()
    if cell is None:
        return torch.zeros_like(S)
    return (S[:, 0:1] * cell[0] + S[:, 1:2] * cell[1]) + S[:, 2:3] * cell[2]


def get_neighborhood(positions: torch.Tensor, cutoff: float, pbc: Optional[Sequence[bool]] = None, cell=None,
                     max_cells: int = 0):
    """(edge_index, shifts, unit_shifts, cell) like upstream's helper of the same name, computed on the GPU that
    holds `positions`."""
    if not positions.is_cuda:
        raise cabi.CudaMaceError("get_neighborhood: positions must live on the GPU")
    pos = positions.detach().double().contiguous()
    cell_t, pbc = _cell_and_pbc(cell, pbc, pos.device)
    row_i, row_j, S = cabi.neighbour_list(pos, cell_t, pbc, float(cutoff), max_cells)
    edge_index = torch.stack([row_i, row_j]).long()
    # the model derives int32 rows from edge_index once per list; hand it the ones that already exist
    edge_index.__dict__["_cm_int32_rows"] = ((edge_index._version, edge_index.data_ptr(), None), (row_i, row_j))
    unit_shifts = S.double()
    shifts = shifts_from_unit_shifts(S, cell_t)
    if cell_t is None:
        cell_t = torch.zeros(3, 3, dtype=torch.float64, device=pos.device)
    return edge_index, shifts, unit_shifts, cell_t


def neighbour_data(positions: torch.Tensor, node_attrs: torch.Tensor, cutoff: float, pbc=None, cell=None) -> Dict[str, torch.Tensor]:
    """The `data` dictionary of a single graph for OptimizedInvariantMACE.forward, neighbour list included."""
    edge_index, shifts, unit_shifts, cell_t = get_neighborhood(positions, cutoff, pbc, cell)
    n = positions.shape[0]
    dev = positions.device
    return {
        "positions": positions, "node_attrs": node_attrs, "batch": torch.zeros(n, dtype=torch.int64, device=dev),
        "ptr": torch.tensor([0, n], dtype=torch.int64, device=dev), "edge_index": edge_index, "unit_shifts": unit_shifts,
        "shifts": shifts, "cell": cell_t,
    }
