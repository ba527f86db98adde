"""Pins of the fp64 reference model (oracle/mace_model.py) by what physics fixes: invariances of the
energy, equivariance of the forces, F = -dE/dx by central differences, sum of forces = 0, smooth cutoff."""
import math

import numpy as np
import pytest
import torch

from cuda_mace.models import SyntheticInvariantMACE
from cuda_mace.utils.synthetic import make_system, neighbour_list
from oracle import mace_model as M


@pytest.fixture(scope="module")
def setup():
    model = SyntheticInvariantMACE(channels=32, atomic_numbers=(1, 6, 7, 8), avg_num_neighbors=9.0, seed=0)
    params = model.export_params()
    data = make_system(21, 4, seed=0, density=None, cluster_box=8.0)
    return params, data


def _rebuild(data, pos):
    ei, S = neighbour_list(pos.numpy(), 5.0, None)
    out = dict(data)
    out["positions"] = pos
    out["edge_index"] = torch.from_numpy(ei)
    out["shifts"] = torch.zeros(ei.shape[1], 3, dtype=torch.float64)
    return out


def _random_rotation(seed):
    q, r = np.linalg.qr(np.random.default_rng(seed).normal(size=(3, 3)))
    q = q * np.sign(np.diag(r))
    if np.linalg.det(q) < 0:
        q[:, 0] = -q[:, 0]
    return torch.tensor(q)


def test_energy_is_finite_and_nontrivial(setup):
    params, data = setup
    out = M.energy_and_forces(params, data)
    assert torch.isfinite(out["energy"]).all() and torch.isfinite(out["forces"]).all()
    assert float(out["forces"].abs().max()) > 1e-3
    assert data["edge_index"].shape[1] > 100


def test_rotation_translation_invariance(setup):
    params, data = setup
    base = M.energy_and_forces(params, data)
    Rm = _random_rotation(1)
    pos2 = data["positions"] @ Rm.t() + torch.tensor([0.3, -1.2, 2.0])
    out = M.energy_and_forces(params, _rebuild(data, pos2))
    torch.testing.assert_close(out["energy"], base["energy"], rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(out["forces"], base["forces"] @ Rm.t(), rtol=1e-8, atol=1e-9)
    # improper rotation (inversion): parity of every coupling path is even
    out = M.energy_and_forces(params, _rebuild(data, -data["positions"]))
    torch.testing.assert_close(out["energy"], base["energy"], rtol=1e-10, atol=1e-10)


def test_permutation_invariance(setup):
    params, data = setup
    base = M.energy_and_forces(params, data)
    perm = torch.from_numpy(np.random.default_rng(2).permutation(21))
    d2 = _rebuild(data, data["positions"][perm])
    d2["node_attrs"] = data["node_attrs"][perm]
    out = M.energy_and_forces(params, d2)
    torch.testing.assert_close(out["energy"], base["energy"], rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(out["forces"], base["forces"][perm], rtol=1e-8, atol=1e-9)


def test_forces_are_minus_gradient_and_sum_to_zero(setup):
    params, data = setup
    base = M.energy_and_forces(params, data)
    torch.testing.assert_close(base["forces"].sum(0), torch.zeros(3, dtype=torch.float64), atol=1e-9, rtol=0)
    h = 1e-5
    for atom, k in [(0, 0), (5, 1), (20, 2)]:
        e = []
        for s in (+1, -1):
            pos = data["positions"].clone()
            pos[atom, k] += s * h
            d = dict(data)
            d["positions"] = pos
            e.append(float(M.energy_and_forces(params, d, compute_forces=False)["interaction_energy"]))
        fd = -(e[0] - e[1]) / (2 * h)
        assert abs(fd - float(base["forces"][atom, k])) < 1e-6 * max(1.0, abs(fd))


def test_edge_direction_convention_does_not_matter(setup):
    """Swapping the roles of edge_index rows (the reference's choice, models/InvariantMACE.py:99-100) flips the sign
    of odd-l message components and leaves the energy unchanged."""
    params, data = setup
    base = M.energy_and_forces(params, data)
    d2 = dict(data)
    d2["edge_index"] = data["edge_index"].flip(0)
    out = M.energy_and_forces(params, d2)  # vectors now point receiver -> sender
    torch.testing.assert_close(out["energy"], base["energy"], rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(out["forces"], base["forces"], rtol=1e-8, atol=1e-9)


def test_periodic_images_are_equivalent():
    model = SyntheticInvariantMACE(channels=32, atomic_numbers=(1, 8), avg_num_neighbors=40.0, seed=1)
    params = model.export_params()
    data = make_system(60, 2, seed=3, density=0.05)  # box 10.6 A > 2 * cutoff
    base = M.energy_and_forces(params, data)
    box = float(data["cell"][0, 0])
    # move a few atoms by lattice vectors: same crystal, shifts change
    pos = data["positions"].clone()
    pos[::7] += torch.tensor([box, -box, 2 * box], dtype=torch.float64)
    ei, S = neighbour_list(pos.numpy(), 5.0, box)
    d2 = dict(data)
    d2["positions"], d2["edge_index"] = pos, torch.from_numpy(ei)
    d2["shifts"] = torch.tensor(S) * box
    out = M.energy_and_forces(params, d2)
    torch.testing.assert_close(out["energy"], base["energy"], rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(out["forces"], base["forces"], rtol=1e-8, atol=1e-9)
