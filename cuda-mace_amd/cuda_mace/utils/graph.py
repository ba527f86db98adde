"""Whole energy+forces step as one HIP graph.

An MD driver evaluates the same model on the same neighbour list many times with new positions.  `GraphedStep`
captures one such evaluation (forward, and the backward that gives the forces) into a HIP graph and replays it: the
~100 kernel launches of a step become one graph launch, which removes the host launch cost (decisive for small
systems) and most of the idle time between kernels on large ones.  The captured step reads positions from a static
buffer and leaves its results in static output tensors; `GraphedStep.__call__` copies the new positions in, replays,
and returns those tensors (valid until the next call).

The neighbour list and the species are part of the capture: build a new `GraphedStep` when the list is rebuilt.
Everything the step derives from them (int32 edge rows, CSR offsets, sender-sorted view, element groups,
species-only features) is computed in the eager warm-up runs before the capture, so the graph holds no sort and no
host synchronisation.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch


class GraphedStep:
    def __init__(self, model: torch.nn.Module, data: Dict[str, torch.Tensor], warmup: int = 2, **forward_kwargs):
        if not data["positions"].is_cuda:
            raise RuntimeError("GraphedStep: the data must live on the GPU")
        self.model = model
        self.kwargs = dict(forward_kwargs)
        # static inputs: the step always reads these very tensors
        self.data = {k: (v.detach().clone() if k == "positions" else v) for k, v in data.items()}
        self.positions = self.data["positions"]
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(max(1, warmup)):  # builds every cached index structure and warms the allocator
                self._eager()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            out = self._eager()
        self.outputs = {k: v for k, v in out.items() if isinstance(v, torch.Tensor)}

    def _eager(self) -> Dict[str, Optional[torch.Tensor]]:
        self.positions.grad = None
        out = self.model(dict(self.data), **self.kwargs)
        return {k: (v.detach() if isinstance(v, torch.Tensor) else v) for k, v in out.items()}

    def __call__(self, positions: Optional[torch.Tensor] = None) -> Dict[str, torch.Tensor]:
        """Evaluates the captured step for `positions` (same shape as at capture; None = keep the current ones)."""
        if positions is not None:
            with torch.no_grad():
                self.positions.copy_(positions)
        self.graph.replay()
        return self.outputs
