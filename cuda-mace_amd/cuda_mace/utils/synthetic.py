"""Seeded synthetic atomic systems and neighbour lists for tests and benchmarks (host side, numpy).

Periodic boxes: N atoms uniform in a cube of density `density` atoms/A^3 with a minimum-image distance of
at least `min_dist` between any two (sequential rejection), species uniform over `num_elements`.
Neighbour list: all ordered pairs (i, j, S) with |r_j - r_i + S L| < cutoff, sorted lexicographically by
(i, j, S); `edge_index[0]` is therefore non-decreasing, which is what the message-passing op needs for the
row it treats as receivers.
"""
from __future__ import annotations

from typing import Dict, Optional

import numpy as np
import torch


def _rejection_positions(n: int, box: float, min_dist: float, rng: np.random.Generator, periodic: bool) -> np.ndarray:
    ncell = max(int(box / min_dist), 1)
    w = box / ncell
    grid: Dict[tuple, list] = {}
    pos = np.empty((n, 3))
    count = 0
    md2 = min_dist * min_dist
    offsets = [(a, b, c) for a in (-1, 0, 1) for b in (-1, 0, 1) for c in (-1, 0, 1)]
    while count < n:
        cand = rng.random((max(n - count, 64) * 2, 3)) * box
        for p in cand:
            c = tuple(np.minimum((p / w).astype(int), ncell - 1))
            ok = True
            for o in offsets:
                key = (c[0] + o[0], c[1] + o[1], c[2] + o[2])
                if periodic:
                    key = (key[0] % ncell, key[1] % ncell, key[2] % ncell)
                for q in grid.get(key, ()):
                    d = p - pos[q]
                    if periodic:
                        d -= box * np.round(d / box)
                    if d @ d < md2:
                        ok = False
                        break
                if not ok:
                    break
            if ok:
                pos[count] = p
                grid.setdefault(c, []).append(count)
                count += 1
                if count == n:
                    break
    return pos


def neighbour_list(positions: np.ndarray, cutoff: float, box: Optional[float] = None):
    """(edge_index int64 [2, E], unit_shifts float64 [E, 3]) sorted by (i, j, S).  `box` = cubic cell edge for a
    periodic system (must exceed 2 * cutoff, so that at most one image of a pair is inside the cutoff)."""
    from scipy.spatial import cKDTree

    if box is not None:
        assert box > 2 * cutoff, "minimum-image neighbour list needs box > 2 * cutoff"
        tree = cKDTree(np.mod(positions, box), boxsize=box)
    else:
        tree = cKDTree(positions)
    pairs = tree.query_pairs(cutoff, output_type="ndarray")  # i < j
    i = np.concatenate([pairs[:, 0], pairs[:, 1]])
    j = np.concatenate([pairs[:, 1], pairs[:, 0]])
    if box is not None:
        d = positions[j] - positions[i]
        S = -np.round(d / box)
    else:
        S = np.zeros((i.shape[0], 3))
    order = np.lexsort((S[:, 2], S[:, 1], S[:, 0], j, i))
    edge_index = np.stack([i[order], j[order]]).astype(np.int64)
    return edge_index, S[order]


def make_system(n_atoms: int, num_elements: int, seed: int = 0, density: Optional[float] = 0.1, cutoff: float = 5.0,
                min_dist: float = 0.9, cluster_box: Optional[float] = None, dtype=torch.float64) -> Dict[str, torch.Tensor]:
    """The `data` dictionary the model's forward consumes.  density=None with cluster_box=L gives a
    non-periodic cluster in an L^3 cube."""
    rng = np.random.default_rng(seed)
    periodic = cluster_box is None
    box = (n_atoms / density) ** (1.0 / 3.0) if periodic else float(cluster_box)
    pos = _rejection_positions(n_atoms, box, min_dist, rng, periodic)
    species = rng.integers(0, num_elements, n_atoms)
    edge_index, S = neighbour_list(pos, cutoff, box if periodic else None)
    cell = np.eye(3) * box if periodic else np.zeros((3, 3))
    node_attrs = np.zeros((n_atoms, num_elements))
    node_attrs[np.arange(n_atoms), species] = 1.0
    return {
        "positions": torch.tensor(pos, dtype=dtype),
        "node_attrs": torch.tensor(node_attrs, dtype=dtype),
        "batch": torch.zeros(n_atoms, dtype=torch.int64),
        "ptr": torch.tensor([0, n_atoms], dtype=torch.int64),
        "edge_index": torch.from_numpy(edge_index),
        "unit_shifts": torch.tensor(S, dtype=dtype),
        "shifts": torch.tensor(S @ cell, dtype=dtype),
        "cell": torch.tensor(cell, dtype=dtype),
    }


def collate(systems) -> Dict[str, torch.Tensor]:
    """Several single-graph `data` dictionaries as one batch: nodes concatenated, edge indices offset, `batch` / `ptr`
    naming the graph of every node, one 3x3 cell per graph stacked row-wise ([3 * graphs, 3], as upstream batches it)."""
    counts = [int(d["positions"].shape[0]) for d in systems]
    starts = np.concatenate([[0], np.cumsum(counts)])
    out = {k: torch.cat([d[k] for d in systems], dim=0) for k in ("positions", "node_attrs", "unit_shifts", "shifts", "cell")}
    out["edge_index"] = torch.cat([d["edge_index"] + int(o) for d, o in zip(systems, starts[:-1])], dim=1)
    out["batch"] = torch.cat([torch.full((c,), g, dtype=torch.int64) for g, c in enumerate(counts)])
    out["ptr"] = torch.tensor(starts, dtype=torch.int64)
    return out


def to_device(data: Dict[str, torch.Tensor], device) -> Dict[str, torch.Tensor]:
    return {k: v.to(device) for k, v in data.items()}


def make_large_system(n_atoms: int, num_elements: int, seed: int = 0, density: float = 0.1, cutoff: float = 5.0,
                      device="cuda") -> Dict[str, torch.Tensor]:
    """A periodic box of `n_atoms` at `density` atoms / A^3 for sizes at which `make_system`'s rejection sampling and
    host-side neighbour search take minutes: atoms on randomly chosen sites of a cubic lattice, each moved by up to 0.3
    lattice spacings per axis (no close pairs), the neighbour list from the device search (utils/neighbour_list.py)."""
    from .neighbour_list import neighbour_data

    g = torch.Generator().manual_seed(seed)
    box = (n_atoms / density) ** (1.0 / 3.0)
    m = int(round(n_atoms ** (1.0 / 3.0))) + 1
    site = torch.randperm(m ** 3, generator=g)[:n_atoms]
    grid = torch.stack([site // (m * m), (site // m) % m, site % m], dim=1).double()
    positions = (grid + 0.5 + 0.6 * (torch.rand(n_atoms, 3, generator=g, dtype=torch.float64) - 0.5)) * (box / m)
    species = torch.randint(0, num_elements, (n_atoms,), generator=g)
    node_attrs = torch.nn.functional.one_hot(species, num_elements).double()
    cell = torch.eye(3, dtype=torch.float64) * box
    return neighbour_data(positions.to(device), node_attrs.to(device), cutoff=cutoff, pbc=(True, True, True), cell=cell.to(device))

