"""DeviceCalculator / MACECalculator: Verlet list on the GPU + graph replays against the fp64 reference model evaluated
on a host-built exact list (energy within 1e-5 relative, forces within 1e-4 eV/A, stress against a strain finite
difference of the reference energy), and against the model itself on a freshly built device list."""
import pytest
import torch

from tests.util import reference_on_fresh_list

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
    upstream = SyntheticInvariantMACE(channels=64, atomic_numbers=tuple(range(1, 11)), avg_num_neighbors=avg, seed=12)
    params = upstream.export_params()
    box = float(data["cell"][0, 0])
    model = OptimizedInvariantMACE(upstream, device="cuda",
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
        if it % 6 == 0 or it == 24:  # the fp64 reference on a host-built exact list for the same positions
            ref = reference_on_fresh_list(params, pos.cpu().numpy(), data["node_attrs"], box)
            e, e_ref = float(got["energy"].double().sum()), float(ref["energy"])
            assert abs(e - e_ref) <= 1e-5 * abs(e_ref), (it, e, e_ref)
            assert float((got["forces"].double().cpu() - ref["forces"]).abs().max()) <= 1e-4
    assert 1 < calc.builds < 25 and calc.steps == 25


def test_running_ahead_of_the_displacement_test(cabi):
    """The step is enqueued before the host has read how far the atoms have moved; a step that ran on a list which turns
    out stale is enqueued again on a fresh one.  Small moves first (the calculator learns how fast the largest
    displacement grows and starts to run ahead), then one atom jumps further than half the skin: the result of that
    step equals the model's on an exact list, and one step was dropped.  With run_ahead=False nothing is dropped and the
    results are the same."""
    from cuda_mace.calculators import DeviceCalculator
    from cuda_mace.models import OptimizedInvariantMACE, SyntheticInvariantMACE
    from cuda_mace.utils.neighbour_list import neighbour_data
    from cuda_mace.utils.synthetic import make_system, to_device

    n = 300
    data = to_device(make_system(n, 4, seed=5, density=0.1), "cuda")
    upstream = SyntheticInvariantMACE(channels=32, atomic_numbers=(1, 6, 7, 8), avg_num_neighbors=data["edge_index"].shape[1] / n,
                                      seed=6)
    model = OptimizedInvariantMACE(upstream, device="cuda")
    pbc = (True, True, True)
    results = {}
    for run_ahead in (True, False):
        calc = DeviceCalculator(model, data["node_attrs"], cutoff=5.0, skin=0.4, pbc=pbc, cell=data["cell"], use_graph=False,
                                run_ahead=run_ahead)
        g = torch.Generator(device="cuda").manual_seed(3)
        pos = data["positions"].clone()
        outs = []
        for it in range(6):
            step = 1e-3 * torch.randn(pos.shape, device="cuda", dtype=pos.dtype, generator=g)
            if it == 4:
                step[17, 0] += 0.3  # further than skin / 2 in one step
            pos = pos + step
            got = calc.compute(pos)
            exact = model(neighbour_data(pos.clone(), data["node_attrs"], 5.0, pbc, data["cell"]))
            scale = float(exact["forces"].abs().max())
            torch.testing.assert_close(got["energy"], exact["energy"].detach(), rtol=1e-7, atol=1e-7)
            torch.testing.assert_close(got["forces"], exact["forces"].detach(), rtol=0, atol=2e-6 * scale)
            outs.append((got["energy"].clone(), got["forces"].clone()))
        assert calc.builds == 2 and calc.steps == 6
        assert calc.dropped == (1 if run_ahead else 0)
        results[run_ahead] = outs
    for (ea, fa), (eb, fb) in zip(results[True], results[False]):
        assert torch.equal(ea, eb) and torch.equal(fa, fb)


def test_stress_replays_with_the_forces(cabi):
    """With stress asked for, the calculator still replays the step as one HIP graph (the one-call step forms the virials
    from the per-edge gradients, no strain tensor in the way): energy, forces and stress of every step of a short walk
    equal the model's on an exact list."""
    from cuda_mace.calculators import DeviceCalculator
    from cuda_mace.models import OptimizedInvariantMACE, SyntheticInvariantMACE
    from cuda_mace.utils.neighbour_list import neighbour_data
    from cuda_mace.utils.synthetic import make_system, to_device

    n = 350
    data = to_device(make_system(n, 4, seed=41, density=0.1), "cuda")
    upstream = SyntheticInvariantMACE(channels=64, atomic_numbers=(1, 6, 7, 8), avg_num_neighbors=data["edge_index"].shape[1] / n,
                                      seed=42)
    model = OptimizedInvariantMACE(upstream, device="cuda")
    pbc = (True, True, True)
    calc = DeviceCalculator(model, data["node_attrs"], cutoff=5.0, skin=0.4, pbc=pbc, cell=data["cell"], use_graph=True,
                            compute_stress=True)
    assert calc.use_graph
    g = torch.Generator(device="cuda").manual_seed(2)
    pos = data["positions"].clone()
    for _ in range(8):
        pos = pos + 0.04 * torch.randn(pos.shape, device="cuda", dtype=pos.dtype, generator=g)
        got = calc.compute(pos)
        assert calc._graph is not None
        exact = model(neighbour_data(pos.clone(), data["node_attrs"], 5.0, pbc, data["cell"]), compute_stress=True)
        torch.testing.assert_close(got["energy"], exact["energy"].detach(), rtol=1e-7, atol=1e-7)
        torch.testing.assert_close(got["forces"], exact["forces"].detach(), rtol=0, atol=2e-6 * float(exact["forces"].abs().max()))
        torch.testing.assert_close(got["stress"], exact["stress"].detach(), rtol=0, atol=2e-6 * float(exact["stress"].abs().max()))
    assert calc.builds >= 2


@pytest.mark.parametrize("relabel", [False, True], ids=["as_given", "relabelled"])
def test_lammps_style_wrapper(cabi, relabel):
    """LAMMPS_MACE (upstream's interface for a domain-decomposed MD code): the energy of the rank's own atoms and minus
    its gradient with respect to every atom, ghosts included, against the fp64 reference model seeded with the same
    mask; with every atom local it equals the model's own energy, forces and virials."""
    from oracle import mace_model as M

    from cuda_mace.calculators import LAMMPS_MACE
    from cuda_mace.models import OptimizedInvariantMACE, SyntheticInvariantMACE
    from cuda_mace.utils.synthetic import make_system, to_device

    n = 320
    data = make_system(n, 4, seed=31, density=0.1)
    upstream = SyntheticInvariantMACE(channels=32, atomic_numbers=(1, 6, 7, 8), avg_num_neighbors=data["edge_index"].shape[1] / n,
                                      seed=32, atomic_energies=torch.linspace(-2.0, -1.0, 4, dtype=torch.float64))
    params = upstream.export_params()
    model = OptimizedInvariantMACE(upstream, device="cuda", spatial_order_min_atoms=0 if relabel else None)
    wrapper = LAMMPS_MACE(model)
    dev = to_device(data, "cuda")
    local = (torch.rand(n, generator=torch.Generator().manual_seed(33)) < 0.6).double()
    got = wrapper(dict(dev), local.cuda())
    assert model._native not in (None, False)  # the mask went into the library's one-call step as node weights
    # the route for models that know nothing of node weights (upstream's own): node energies out, autograd in the wrapper
    got_v = wrapper(dict(dev), local.cuda(), compute_virials=True)  # virials of the masked energy, from the same call
    model.supports_node_weights = False
    try:
        generic = wrapper(dict(dev), local.cuda())
        generic_v = wrapper(dict(dev), local.cuda(), compute_virials=True)  # by autograd through the strain
    finally:
        del model.supports_node_weights
    assert torch.equal(got_v["forces"], got["forces"])
    torch.testing.assert_close(got_v["virials"], generic_v["virials"], rtol=0, atol=2e-6 * float(generic_v["virials"].abs().max()))
    torch.testing.assert_close(generic["total_energy_local"], got["total_energy_local"], rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(generic["forces"], got["forces"], rtol=0, atol=5e-7 * float(got["forces"].abs().max()))
    # all-ones weights are the unweighted step bit for bit
    ones = dict(dev, node_weights=torch.ones(n, dtype=torch.float64, device="cuda"))
    a, b = model(ones), model(dict(dev))
    assert torch.equal(a["forces"], b["forces"]) and torch.equal(a["energy"], b["energy"])
    ref = M.energy_and_forces(params, data, node_weights=local)
    e_ref = float((ref["node_energy"] * local).sum())
    assert abs(float(got["total_energy_local"].sum()) - e_ref) <= 1e-5 * abs(e_ref)
    assert float((got["forces"].double().cpu() - ref["forces"]).abs().max()) <= 1e-4
    assert float((got["node_energy"].double().cpu() - ref["node_energy"]).abs().max()) <= 1e-5 * float(ref["node_energy"].abs().max())
    # the masked forces are not the forces of the whole system (the mask matters) ...
    whole = M.energy_and_forces(params, data)
    assert float((ref["forces"] - whole["forces"]).abs().max()) > 1e-2
    # ... and with every atom local the wrapper reproduces the model's own outputs
    every = wrapper(dict(dev), torch.ones(n, device="cuda"), compute_virials=True)
    own = model(dict(dev), compute_virials=True)
    scale = float(own["forces"].abs().max())
    torch.testing.assert_close(every["total_energy_local"], own["energy"].detach(), rtol=1e-9, atol=1e-9)
    torch.testing.assert_close(every["forces"], own["forces"].detach(), rtol=0, atol=2e-6 * scale)
    torch.testing.assert_close(every["virials"], own["virials"].detach(), rtol=0, atol=2e-6 * float(own["virials"].abs().max()))
    assert got["virials"] is None and every["virials"].shape == (1, 3, 3)


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
    """Energy and forces through the ASE calculator protocol against the fp64 reference model, the Voigt stress against
    a central strain difference of the reference energy; all three also against the model on a freshly built list."""
    import numpy as np

    from cuda_mace.calculators import MACECalculator
    from cuda_mace.models import OptimizedInvariantMACE, SyntheticInvariantMACE
    from cuda_mace.utils.neighbour_list import neighbour_data
    from cuda_mace.utils.synthetic import make_system, to_device

    n = 300
    zs = (1, 6, 7, 8)
    data = to_device(make_system(n, len(zs), seed=21, density=0.1), "cuda")
    avg = data["edge_index"].shape[1] / n
    upstream = SyntheticInvariantMACE(channels=32, atomic_numbers=zs, avg_num_neighbors=avg, seed=22)
    params = upstream.export_params()
    box = float(data["cell"][0, 0])
    model = OptimizedInvariantMACE(upstream, device="cuda")
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
    assert abs(e - float(ref["energy"].detach().sum())) <= 1e-7 * max(1.0, abs(e))
    np.testing.assert_allclose(f, ref["forces"].detach().cpu().numpy(), rtol=0, atol=2e-6 * scale)
    s = calc.get_stress(atoms)
    full = ref["stress"].detach().reshape(3, 3).cpu().numpy()
    voigt = np.array([full[0, 0], full[1, 1], full[2, 2], full[1, 2], full[0, 2], full[0, 1]])
    np.testing.assert_allclose(s, voigt, rtol=0, atol=2e-6 * float(np.abs(voigt).max()))

    # the fp64 reference: energy, forces, and stress = (1/V) dE/d(strain) by central differences
    oracle = reference_on_fresh_list(params, atoms.positions, data["node_attrs"], box)
    assert abs(e - float(oracle["energy"])) <= 1e-5 * abs(float(oracle["energy"]))
    assert float(np.abs(f - oracle["forces"].numpy()).max()) <= 1e-4
    h, vol = 1e-5, box ** 3
    for comp, (a, b) in enumerate([(0, 0), (1, 1), (2, 2), (1, 2), (0, 2), (0, 1)]):
        if comp in (1, 2, 4):
            continue  # three of the six components pin the convention (diagonal, two off-diagonal orders)
        es = []
        for sign in (+1, -1):
            eps = np.zeros((3, 3))
            eps[a, b] += sign * h / 2
            eps[b, a] += sign * h / 2
            es.append(float(reference_on_fresh_list(params, atoms.positions, data["node_attrs"], box, strain=eps,
                                                    compute_forces=False)["interaction_energy"]))
        fd = (es[0] - es[1]) / (2 * h) / vol
        assert abs(fd - s[comp]) <= 2e-3 * float(np.abs(s).max()), (comp, fd, s[comp])

    # moved atoms: results are recomputed; an unknown species is refused
    atoms.positions = atoms.positions + 0.02 * np.random.default_rng(0).normal(size=atoms.positions.shape)
    assert calc.calculation_required(atoms, ["forces"])
    ref2 = exact(atoms.positions)
    np.testing.assert_allclose(calc.get_forces(atoms), ref2["forces"].detach().cpu().numpy(), rtol=0, atol=2e-6 * scale)
    oracle2 = reference_on_fresh_list(params, atoms.positions, data["node_attrs"], box)
    assert float(np.abs(calc.get_forces(atoms) - oracle2["forces"].numpy()).max()) <= 1e-4
    assert abs(calc.get_potential_energy(atoms) - float(oracle2["energy"])) <= 1e-5 * abs(float(oracle2["energy"]))
    assert abs(calc.get_potential_energy(atoms) - float(ref2["energy"].detach().sum())) <= 1e-7 * max(1.0, abs(e))
    atoms.numbers = atoms.numbers.copy()
    atoms.numbers[0] = 79
    with pytest.raises(ValueError, match="not covered"):
        calc.get_forces(atoms)
