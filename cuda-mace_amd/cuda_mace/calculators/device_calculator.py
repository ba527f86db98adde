"""Energy and forces for a molecular-dynamics driver, everything on the GPU.

The reference stops at the model: its users get `edge_index` / `shifts` from upstream's host-side neighbour search
(tests/test_utils.py:62-105) and call `OptimizedInvariantMACE.forward` (tools/model_surgery.py:217-229 times exactly
that).  This class strings the device-side pieces together the way an MD code does:

  * a Verlet list: neighbours within cutoff + skin, rebuilt on the GPU only when some atom has moved more than
    skin / 2 since the last build.  Pairs between cutoff and cutoff + skin contribute exact zeros (the radial spline
    vanishes beyond r_max), so results do not depend on the skin;
  * the test for that (one kernel, `cm_max_displacement`, one scalar copied to pinned host memory) does not drain
    the GPU: while the largest displacement seen at the previous step leaves room for twice the largest growth seen
    per step, the step is enqueued on the old list before the host reads the scalar, so the GPU always has the next
    step queued; should the scalar then say that the list was stale after all, the step is enqueued again on a fresh
    list and the first result is dropped.  Close to the limit the host reads the scalar first, as a plain Verlet
    list does;
  * between rebuilds the step can run as one HIP graph (utils/graph.py), re-captured after every rebuild; by default
    only models that go through the Python autograd functions do (see use_graph).
"""
from __future__ import annotations

import math
from typing import Dict, Optional, Sequence

import torch

from cuda_mace import _cabi
from cuda_mace.utils.graph import GraphedStep
from cuda_mace.utils.neighbour_list import get_neighborhood


class DeviceCalculator:
    def __init__(self, model: torch.nn.Module, node_attrs: torch.Tensor, cutoff: Optional[float] = None, skin: float = 0.5,
                 pbc: Sequence[bool] = (False, False, False), cell: Optional[torch.Tensor] = None,
                 use_graph: Optional[bool] = None, compute_stress: bool = False, run_ahead: bool = True):
        """use_graph: replay the step as one HIP graph between list rebuilds.  None decides: a model that takes the
        library's one-call step runs eagerly at every size (one call enqueues the step's kernels back to back, a replay
        of the same kernels is a few per cent slower and every rebuild costs a capture: 0.24 against 0.29 ms per MD step
        at 300 atoms, 1.01 against 1.13 at 8 000); a model that goes through the Python autograd functions is bound by
        host launches up to about 8192 atoms and is replayed as a graph there.  run_ahead=False reads the displacement
        test before every step."""
        self.model = model
        self.node_attrs = node_attrs
        self.cutoff = float(model.r_max) if cutoff is None else float(cutoff)
        self.skin = float(skin)
        self.pbc = tuple(bool(b) for b in pbc)
        self.cell = None if cell is None else cell.detach().double().reshape(3, 3).contiguous()
        self.compute_stress = bool(compute_stress)
        # Stress comes out of the library's one-call step without a strain tensor and replays like the forces; only the
        # autograd path (a model that cannot take the one-call step) re-derives the shifts from a strained cell.
        one_call = bool(getattr(model, "native_step", False)) and getattr(model, "_native_step_of", lambda: None)() is not None
        if use_graph is None:
            use_graph = (not one_call) and node_attrs.shape[0] <= 8192
        self.use_graph = bool(use_graph) and (one_call or not self.compute_stress)
        self.run_ahead = bool(run_ahead)
        # an MD step reads energy, forces and stress only: a model that can skip the per-node feature output is told to
        self._forward_kwargs = {"compute_node_feats": False} if one_call else {}
        self.builds = 0
        self.steps = 0
        self.dropped = 0  # steps enqueued on a list that turned out stale, and enqueued again
        self._ref_positions: Optional[torch.Tensor] = None
        self._data: Optional[Dict[str, torch.Tensor]] = None
        self._graph: Optional[GraphedStep] = None
        self._moved_sq = torch.empty(1, dtype=torch.float64, device=node_attrs.device)
        self._moved_sq_host = torch.empty(1, dtype=torch.float64, pin_memory=True)
        self._arrived = torch.cuda.Event()
        self._moved = 0.0           # largest displacement since the build, as of the last test
        self._growth = math.inf     # largest growth of that between two tests (decays slowly); unknown at first

    # -- Verlet list ---------------------------------------------------------------------------------------
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
        self._graph = None
        if self.use_graph:
            self._graph = GraphedStep(self.model, self._data, warmup=1, compute_virials=self.compute_stress,
                                      compute_stress=self.compute_stress, **self._forward_kwargs)
        self._moved = 0.0
        self.builds += 1

    # -- evaluation ----------------------------------------------------------------------------------------
    def _run(self, positions: torch.Tensor) -> Dict[str, torch.Tensor]:
        if self._graph is not None:
            return self._graph(positions)
        data = dict(self._data)
        data["positions"] = positions.detach()  # an alias: the model marks its own handle as differentiable, not the caller's
        out = self.model(data, compute_virials=self.compute_stress, compute_stress=self.compute_stress, **self._forward_kwargs)
        return {k: v.detach() for k, v in out.items() if isinstance(v, torch.Tensor)}

    def compute(self, positions: torch.Tensor) -> Dict[str, torch.Tensor]:
        """energy [1], forces [N, 3] (and virials / stress when asked for) at `positions` (fp64, on the GPU)."""
        positions = positions.detach().double().contiguous()
        self.steps += 1
        if self._ref_positions is None or self._ref_positions.shape != positions.shape:
            self._rebuild(positions)
            return self._run(positions)
        _cabi.max_displacement(positions, self._ref_positions, out=self._moved_sq)
        self._moved_sq_host.copy_(self._moved_sq, non_blocking=True)
        self._arrived.record()
        limit = 0.5 * self.skin
        ahead = self.run_ahead and self._moved + 2.0 * self._growth <= limit
        out = self._run(positions) if ahead else None
        self._arrived.synchronize()  # the scalar, not the step: the step's kernels come after it on the stream
        moved = math.sqrt(float(self._moved_sq_host[0]))
        if not moved <= limit:
            self.dropped += int(ahead)
            self._rebuild(positions)
            return self._run(positions)
        self._growth = max(moved - self._moved, 0.95 * self._growth if math.isfinite(self._growth) else 0.0)
        self._moved = moved
        return out if ahead else self._run(positions)
