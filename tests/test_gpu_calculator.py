"""DeviceCalculator: Verlet list on the GPU + graph replays reproduce the model on an exact, freshly built list."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("use_graph", [True, False], ids=["graph", "eager"])
def test_md_like_walk(cabi, use_graph):
    from cuda_mace.calculators import DeviceCalculator
    from cuda_mace.models import OptimizedInvariantMACE, SyntheticInvariantMACE
    from cuda_mace.utils.neighbour_list import neighbour_data
    from cuda_mace.utils.synthetic import make_system, to_device

    n = 400
    data = to_device(make_system(n, 10, seed=11, density=0.1), "cuda")
    avg = data["edge_index"].shape[1] / n
    model = OptimizedInvariantMACE(SyntheticInvariantMACE(channels=64, atomic_numbers=tuple(range(1, 11)),
                                                          avg_num_neighbors=avg, seed=12), device="cuda",
                                   spatial_order_min_atoms=0 if use_graph else None)  # one of the two with relabelling
    calc = DeviceCalculator(model, data["node_attrs"], cutoff=5.0, skin=0.4, pbc=(True, True, True), cell=data["cell"],
                            use_graph=use_graph)
    g = torch.Generator(device="cuda").manual_seed(1)
    pos = data["positions"].clone()
    for it in range(25):
        pos = pos + 0.03 * torch.randn(pos.shape, device="cuda", dtype=pos.dtype, generator=g)
        got = calc.compute(pos)
        exact = model(neighbour_data(pos.clone(), data["node_attrs"], 5.0, (True, True, True), data["cell"]))
        scale = float(exact["forces"].abs().max())
        torch.testing.assert_close(got["energy"], exact["energy"].detach(), rtol=1e-7, atol=1e-7)
        torch.testing.assert_close(got["forces"], exact["forces"].detach(), rtol=0, atol=2e-6 * scale)
    assert 1 < calc.builds < 25 and calc.steps == 25


class _Atoms:
    """The four accessors of ase.Atoms that a calculator reads."""

    def __init__(self, positions, numbers, cell, pbc):
        self.positions, self.numbers, self.cell, self.pbc = positions, numbers, cell, pbc
        self.calc = None

    def get_positions(self):
        return self.positions.copy()

    def get_atomic_numbers(self):
        return self.numbers.copy()

    def get_cell(self):
        return self.cell.copy()

    def get_pbc(self):
        return self.pbc


def test_ase_protocol_calculator(cabi):
    """Energy, forces and Voigt stress through the ASE calculator protocol equal the model on a freshly built list."""
    import numpy as np

    from cuda_mace.calculators import MACECalculator
    from cuda_mace.models import OptimizedInvariantMACE, SyntheticInvariantMACE
    from cuda_mace.utils.neighbour_list import neighbour_data
    from cuda_mace.utils.synthetic import make_system, to_device

    n = 300
    zs = (1, 6, 7, 8)
    data = to_device(make_system(n, len(zs), seed=21, density=0.1), "cuda")
    avg = data["edge_index"].shape[1] / n
    model = OptimizedInvariantMACE(SyntheticInvariantMACE(channels=32, atomic_numbers=zs, avg_num_neighbors=avg, seed=22),
                                   device="cuda")
    numbers = np.asarray(zs)[data["node_attrs"].argmax(1).cpu().numpy()]
    atoms = _Atoms(data["positions"].cpu().numpy(), numbers, data["cell"].reshape(3, 3).cpu().numpy(), (True, True, True))
    calc = MACECalculator(model)
    atoms.calc = calc

    def exact(positions):
        d = neighbour_data(torch.from_numpy(positions).cuda(), data["node_attrs"], 5.0, (True, True, True), data["cell"])
        return model(d, compute_virials=True, compute_stress=True)

    ref = exact(atoms.positions)
    e = calc.get_potential_energy(atoms)
    f = calc.get_forces(atoms)
    assert not calc.calculation_required(atoms, ["energy", "forces"])
    scale = float(ref["forces"].abs().max())
    assert abs(e - float(ref["energy"].sum())) <= 1e-7 * max(1.0, abs(e))
    np.testing.assert_allclose(f, ref["forces"].detach().cpu().numpy(), rtol=0, atol=2e-6 * scale)
    s = calc.get_stress(atoms)
    full = ref["stress"].detach().reshape(3, 3).cpu().numpy()
    voigt = np.array([full[0, 0], full[1, 1], full[2, 2], full[1, 2], full[0, 2], full[0, 1]])
    np.testing.assert_allclose(s, voigt, rtol=0, atol=2e-6 * float(np.abs(voigt).max()))

    # moved atoms: results are recomputed; an unknown species is refused
    atoms.positions = atoms.positions + 0.02 * np.random.default_rng(0).normal(size=atoms.positions.shape)
    assert calc.calculation_required(atoms, ["forces"])
    ref2 = exact(atoms.positions)
    np.testing.assert_allclose(calc.get_forces(atoms), ref2["forces"].detach().cpu().numpy(), rtol=0, atol=2e-6 * scale)
    assert abs(calc.get_potential_energy(atoms) - float(ref2["energy"].sum())) <= 1e-7 * max(1.0, abs(e))
    atoms.numbers = atoms.numbers.copy()
    atoms.numbers[0] = 79
    with pytest.raises(ValueError, match="not covered"):
        calc.get_forces(atoms)
