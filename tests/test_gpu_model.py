"""End-to-end parity on the GPU: OptimizedInvariantMACE (fp32 HIP kernels, splined radial functions) against
the fp64 CPU reference model on the same seeded weights and structures.

Bar: energy within 1e-5 relative, forces within 1e-4 eV/A max-abs.
"""
import numpy as np
import pytest
import torch

from cuda_mace.utils.synthetic import make_system, to_device
from oracle import mace_model as M
from tests.util import carve_cluster as _carve

pytestmark = pytest.mark.gpu

E_RTOL = 1e-5
F_ATOL = 1e-4


def _say(*a):
    print(*a, flush=True)


def _build(channels, numbers, data, seed, fused=True, fused_readout=True, fused_contraction=True):
    from cuda_mace.models import OptimizedInvariantMACE, SyntheticInvariantMACE

    avg = data["edge_index"].shape[1] / data["positions"].shape[0]
    up = SyntheticInvariantMACE(channels=channels, atomic_numbers=numbers, avg_num_neighbors=avg, seed=seed)
    model = OptimizedInvariantMACE(up, device="cuda", fused_radial=fused, fused_readout=fused_readout,
                                   fused_contraction=fused_contraction)
    assert model.fused_readout == fused_readout
    return up.export_params(), model


def _compare(params, model, data):
    ref = M.energy_and_forces(params, data)
    out = model(to_device(data, "cuda"))
    e, e_ref = float(out["interaction_energy"].detach().cpu()), float(ref["interaction_energy"])
    f_err = float((out["forces"].double().cpu() - ref["forces"]).abs().max())
    _say("  E %.10g ref %.10g rel %.2e | max|dF| %.2e (max|F| %.3g)" % (e, e_ref, abs(e - e_ref) / abs(e_ref), f_err,
                                                                       float(ref["forces"].abs().max())))
    assert abs(e - e_ref) <= E_RTOL * abs(e_ref)
    assert f_err <= F_ATOL
    nf = out["node_feats"].double().cpu()
    torch.testing.assert_close(nf, ref["node_feats"], rtol=1e-4, atol=1e-5 * float(ref["node_feats"].abs().max()))
    return out, ref


def test_cluster_config1(cabi):
    """Benchmark configuration 1: 21-atom non-periodic cluster in an 8 A cube, {H, C, N, O}, 64 channels."""
    _say("model c1: 21-atom cluster, C=64")
    data = make_system(21, 4, seed=0, density=None, cluster_box=8.0)
    params, model = _build(64, (1, 6, 7, 8), data, seed=0)
    out, ref = _compare(params, model, data)
    _, unfused = _build(64, (1, 6, 7, 8), data, seed=0, fused=False)
    _compare(params, unfused, data)
    _, module_readouts = _build(64, (1, 6, 7, 8), data, seed=0, fused_readout=False)  # the readout modules themselves
    _compare(params, module_readouts, data)
    _, separate_ops = _build(64, (1, 6, 7, 8), data, seed=0, fused_contraction=False)  # Linear -> SymmetricContraction ops
    _compare(params, separate_ops, data)
    assert out["energy"].shape == (1,) and out["forces"].shape == (21, 3)
    assert set(out) == {"energy", "node_energy", "interaction_energy", "forces", "virials", "stress", "hessian",
                        "displacement", "node_feats", "edge_forces"}


@pytest.mark.parametrize("fused", [True, False], ids=["fused_radial", "tabulated_radial"])
@pytest.mark.parametrize("natoms,channels,seed", [(300, 96, 1), (400, 128, 2), (250, 192, 3)])
def test_periodic_box(cabi, natoms, channels, seed, fused):
    """Periodic boxes at the benchmark density (0.1 atoms/A^3, about 52 neighbours), 10 elements; with the radial
    spline evaluated inside the message-passing kernels and with the reference's separate spline step."""
    _say("model periodic: N=%d C=%d seed=%d fused=%s" % (natoms, channels, seed, fused))
    data = make_system(natoms, 10, seed=seed, density=0.1)
    params, model = _build(channels, tuple(range(1, 11)), data, seed=seed, fused=fused, fused_contraction=fused)
    _compare(params, model, data)


def test_forces_sum_to_zero_and_repeatable(cabi):
    data = make_system(500, 10, seed=5, density=0.1)
    params, model = _build(128, tuple(range(1, 11)), data, seed=5)
    d = to_device(data, "cuda")
    a = model(dict(d))
    b = model(dict(d))
    assert torch.equal(a["forces"], b["forces"]) and torch.equal(a["energy"], b["energy"])
    assert float(a["forces"].sum(0).abs().max()) < 1e-3 * float(a["forces"].abs().max()) + 1e-5


def test_virials_match_strain_derivative(cabi):
    """virials = -dE/d(strain): compared with a central difference of the fp64 reference energy under a
    symmetric strain of positions and cell."""
    data = make_system(200, 4, seed=7, density=0.1)
    params, model = _build(64, (1, 6, 7, 8), data, seed=7)
    out = model(to_device(data, "cuda"), compute_virials=True, compute_stress=True)
    vir = out["virials"].double().cpu()[0]
    h = 1e-5
    for (a, b) in [(0, 0), (0, 1), (2, 1)]:
        es = []
        for s in (+1, -1):
            eps = torch.zeros(3, 3, dtype=torch.float64)
            eps[a, b] += s * h / 2
            eps[b, a] += s * h / 2
            d2 = dict(data)
            d2["positions"] = data["positions"] + data["positions"] @ eps
            cell = data["cell"] + data["cell"] @ eps
            d2["shifts"] = data["unit_shifts"] @ cell
            es.append(float(M.energy_and_forces(params, d2, compute_forces=False)["interaction_energy"]))
        fd = -(es[0] - es[1]) / (2 * h)
        assert abs(fd - float(vir[a, b])) < 2e-3 * max(1.0, float(vir.abs().max()))
    vol = float(torch.det(data["cell"]))
    torch.testing.assert_close(out["stress"].double().cpu()[0], -vir / vol, rtol=1e-5, atol=1e-8)


def test_batch_of_graphs(cabi):
    """Three different periodic boxes as one batch: per-graph energies, forces, virials and stress equal those of the
    graphs evaluated one by one (GPU) and the fp64 reference."""
    from cuda_mace.models import OptimizedInvariantMACE, SyntheticInvariantMACE
    from cuda_mace.utils.synthetic import collate

    systems = [make_system(n, 4, seed=20 + k, density=0.1) for k, n in enumerate((150, 230, 120))]
    deg = sum(int(d["edge_index"].shape[1]) for d in systems) / sum(int(d["positions"].shape[0]) for d in systems)
    upstream = SyntheticInvariantMACE(channels=64, atomic_numbers=(1, 6, 7, 8), avg_num_neighbors=deg, seed=9)
    params = upstream.export_params()
    model = OptimizedInvariantMACE(upstream, device="cuda")
    batch = model(to_device(collate(systems), "cuda"), compute_virials=True, compute_stress=True)
    assert batch["energy"].shape == (3,) and batch["virials"].shape == (3, 3, 3) and batch["stress"].shape == (3, 3, 3)
    start = 0
    for g, d in enumerate(systems):
        n = d["positions"].shape[0]
        single = model(to_device(d, "cuda"), compute_virials=True, compute_stress=True)
        ref = M.energy_and_forces(params, d)
        scale = float(ref["forces"].abs().max())
        assert abs(float(batch["energy"][g].detach()) - float(ref["energy"])) <= 1e-5 * abs(float(ref["energy"])) + 1e-6
        assert float((batch["forces"][start:start + n].double().cpu() - ref["forces"]).abs().max()) <= 1e-4
        torch.testing.assert_close(batch["energy"][g].detach(), single["energy"][0].detach(), rtol=1e-6, atol=1e-7)
        torch.testing.assert_close(batch["forces"][start:start + n], single["forces"], rtol=0, atol=1e-6 * scale + 1e-7)
        torch.testing.assert_close(batch["virials"][g], single["virials"][0], rtol=1e-5, atol=1e-5 * float(single["virials"].abs().max()))
        torch.testing.assert_close(batch["stress"][g], single["stress"][0], rtol=1e-5, atol=1e-5 * float(single["stress"].abs().max()))
        start += n


def test_config3_full_size_against_reference(cabi):
    """Benchmark configuration 3 at its real size (5 000 atoms, 96 channels, 10 elements): energy and forces against the fp64
    reference evaluated in edge chunks."""
    _say("model c3: 5000-atom periodic box, C=96")
    data = make_system(5000, 10, seed=0, density=0.1)
    params, model = _build(96, tuple(range(1, 11)), data, seed=0)
    ref = M.energy_and_forces(params, data, edge_chunk=65536)
    out = model(to_device(data, "cuda"))
    e, e_ref = float(out["interaction_energy"].detach().cpu()), float(ref["interaction_energy"])
    f_err = float((out["forces"].double().cpu() - ref["forces"]).abs().max())
    _say("  E %.10g ref %.10g rel %.2e | max|dF| %.2e" % (e, e_ref, abs(e - e_ref) / abs(e_ref), f_err))
    assert abs(e - e_ref) <= E_RTOL * abs(e_ref)
    assert f_err <= F_ATOL


def test_config4_full_size_properties(cabi):
    """Benchmark configuration 4 at its real size (25 000 atoms, 128 channels), where the fp64 reference is out of reach: forces
    sum to zero, two evaluations agree bit for bit, and rotating the whole periodic system (positions, cell, shifts)
    leaves the energy unchanged and rotates the forces."""
    _say("model c4: 25000-atom periodic box, C=128")
    data = make_system(25000, 10, seed=0, density=0.1)
    _, model = _build(128, tuple(range(1, 11)), data, seed=0)
    dev = to_device(data, "cuda")
    a = model(dict(dev))
    b = model(dict(dev))
    assert torch.equal(a["energy"], b["energy"]) and torch.equal(a["forces"], b["forces"])
    fmax = float(a["forces"].abs().max())
    assert float(a["forces"].sum(0).abs().max()) < 1e-4 * 25000 ** 0.5 * max(fmax, 1.0) * 1e-1

    # a proper rotation from a QR decomposition
    g = torch.Generator().manual_seed(3)
    Q, _ = torch.linalg.qr(torch.randn(3, 3, generator=g, dtype=torch.float64))
    if torch.det(Q) < 0:
        Q[:, 0] = -Q[:, 0]
    Q = Q.to("cuda")
    rot = dict(dev)
    rot["positions"] = dev["positions"].detach() @ Q
    rot["cell"] = dev["cell"] @ Q
    rot["shifts"] = dev["shifts"] @ Q
    c = model(rot)
    e0, e1 = float(a["interaction_energy"].detach()), float(c["interaction_energy"].detach())
    _say("  E %.10g rotated %.10g rel %.2e" % (e0, e1, abs(e0 - e1) / abs(e0)))
    assert abs(e0 - e1) <= 2e-6 * abs(e0)
    f_rot = a["forces"].detach() @ Q
    assert float((c["forces"].detach() - f_rot).abs().max()) <= 2e-5 * max(fmax, 1.0)


def test_spatial_relabelling_is_transparent(cabi):
    """The model on its internally relabelled graph (atoms sorted by spatial bin, edges re-sorted) returns, in the caller's
    order, what it returns without the relabelling: a batch of two boxes with virials, against the plain path and the
    fp64 reference; the relabelled run repeats bit for bit."""
    from cuda_mace.models import OptimizedInvariantMACE, SyntheticInvariantMACE
    from cuda_mace.utils.synthetic import collate

    systems = [make_system(n, 4, seed=40 + k, density=0.1) for k, n in enumerate((260, 190))]
    deg = sum(int(d["edge_index"].shape[1]) for d in systems) / sum(int(d["positions"].shape[0]) for d in systems)
    upstream = SyntheticInvariantMACE(channels=64, atomic_numbers=(1, 6, 7, 8), avg_num_neighbors=deg, seed=13)
    params = upstream.export_params()
    plain = OptimizedInvariantMACE(upstream, device="cuda", spatial_order_min_atoms=None)
    ordered = OptimizedInvariantMACE(upstream, device="cuda", spatial_order_min_atoms=0)
    data = to_device(collate(systems), "cuda")
    a = plain(dict(data), compute_virials=True, compute_stress=True)
    b = ordered(dict(data), compute_virials=True, compute_stress=True)
    perm = data["edge_index"]._cm_spatial_order[1][0]
    assert not torch.equal(perm, torch.arange(perm.numel(), device="cuda"))  # the relabelling did something
    scale = float(a["forces"].abs().max())
    torch.testing.assert_close(b["energy"].detach(), a["energy"].detach(), rtol=1e-7, atol=1e-7)
    torch.testing.assert_close(b["forces"], a["forces"], rtol=0, atol=2e-6 * scale)
    torch.testing.assert_close(b["node_energy"].detach(), a["node_energy"].detach(), rtol=1e-6, atol=1e-7)
    torch.testing.assert_close(b["node_feats"].detach(), a["node_feats"].detach(), rtol=1e-5, atol=1e-6 * float(a["node_feats"].abs().max()))
    torch.testing.assert_close(b["virials"], a["virials"], rtol=1e-5, atol=1e-5 * float(a["virials"].abs().max()))
    torch.testing.assert_close(b["stress"], a["stress"], rtol=1e-5, atol=1e-5 * float(a["stress"].abs().max()))
    again = ordered(dict(data), compute_virials=True, compute_stress=True)
    assert torch.equal(again["forces"], b["forces"]) and torch.equal(again["energy"], b["energy"])
    start = 0
    for g, d in enumerate(systems):
        n = d["positions"].shape[0]
        ref = M.energy_and_forces(params, d)
        assert abs(float(b["energy"][g].detach()) - float(ref["energy"])) <= 1e-5 * abs(float(ref["energy"])) + 1e-6
        assert float((b["forces"][start:start + n].double().cpu() - ref["forces"]).abs().max()) <= 1e-4
        start += n


def test_config5_full_size_properties(cabi):
    """Benchmark configuration 5 at its real size (100 000 atoms, 192 channels, 5.2 M edges; three channels per lane in the
    message-passing kernels): forces sum to zero, two evaluations agree bit for bit, and moving every atom by the same
    vector (the edge vectors change only by rounding) leaves energy and forces unchanged."""
    _say("model c5: 100000-atom periodic box, C=192")
    data = make_system(100000, 10, seed=0, density=0.1)
    _, model = _build(192, tuple(range(1, 11)), data, seed=0)
    dev = to_device(data, "cuda")
    a = model(dict(dev))
    b = model(dict(dev))
    assert torch.equal(a["energy"], b["energy"]) and torch.equal(a["forces"], b["forces"])
    assert bool(torch.isfinite(a["forces"]).all())
    fmax = float(a["forces"].abs().max())
    assert float(a["forces"].sum(0).abs().max()) < 1e-5 * 100000 ** 0.5 * max(fmax, 1.0)
    moved = dict(dev)
    moved["positions"] = dev["positions"].detach() + torch.tensor([0.37, -1.21, 2.05], dtype=torch.float64, device="cuda")
    c = model(moved)
    e0, e1 = float(a["interaction_energy"].detach()), float(c["interaction_energy"].detach())
    _say("  E %.10g translated %.10g rel %.2e" % (e0, e1, abs(e0 - e1) / abs(e0)))
    assert abs(e0 - e1) <= 2e-6 * abs(e0)
    assert float((c["forces"].detach() - a["forces"].detach()).abs().max()) <= 2e-5 * max(fmax, 1.0)


def test_large_box_400k_atoms_properties(cabi):
    """Sixteen times the headline size on one GPU (400 000 atoms, 20.9 M pairs, 128 channels, 29 GB): the list comes from
    the device neighbour search, the step from the same single library call.  Size-independent properties: forces sum
    to zero, two evaluations agree bit for bit, a rigid translation changes nothing beyond rounding, and the per-atom
    throughput stays that of the headline size (the indexing holds beyond 2^31 feature elements)."""
    from cuda_mace.models import OptimizedInvariantMACE, SyntheticInvariantMACE
    from cuda_mace.utils.synthetic import make_large_system

    n = 400000
    _say("model: 400000-atom periodic box from the device neighbour list, C=128")
    data = make_large_system(n, 10, seed=0, density=0.1)
    pairs = data["edge_index"].shape[1]
    assert 50.0 < pairs / n < 55.0  # 4/3 pi 5^3 x 0.1 = 52.4 neighbours per atom
    assert 16 * n * 128 > 2 ** 29 and pairs * 128 > 2 ** 31  # the [N,16,C] and [E,C] buffers, in elements
    up = SyntheticInvariantMACE(channels=128, atomic_numbers=tuple(range(1, 11)), avg_num_neighbors=pairs / n, seed=0)
    model = OptimizedInvariantMACE(up, device="cuda")
    a = model(dict(data))
    b = model(dict(data))
    assert torch.equal(a["energy"], b["energy"]) and torch.equal(a["forces"], b["forces"])
    assert bool(torch.isfinite(a["forces"]).all()) and bool(torch.isfinite(a["node_energy"]).all())
    fmax = float(a["forces"].abs().max())
    assert fmax > 1e-4  # the forces are not trivially zero
    assert float(a["forces"].sum(0).abs().max()) < 1e-5 * n ** 0.5 * max(fmax, 1.0)
    moved = dict(data)
    moved["positions"] = data["positions"].detach() + torch.tensor([0.37, -1.21, 2.05], dtype=torch.float64, device="cuda")
    c = model(moved)
    e0, e1 = float(a["interaction_energy"].detach()), float(c["interaction_energy"].detach())
    _say("  E %.10g translated %.10g rel %.2e, max|F| %.3g" % (e0, e1, abs(e0 - e1) / abs(e0), fmax))
    assert abs(e0 - e1) <= 2e-6 * abs(e0)
    assert float((c["forces"].detach() - a["forces"].detach()).abs().max()) <= 2e-5 * max(fmax, 1.0)
    del a, b, c, model
    torch.cuda.empty_cache()


# ---- oracle parity at the full sizes of configurations 4 and 5 ------------------------------------------------------
def _check_against_carved_clusters(params, data, out, centres, cutoff=5.0):
    node_e = out["node_energy"].detach().double().cpu()
    forces = out["forces"].detach().double().cpu()
    worst_e, worst_f, checked = 0.0, 0.0, 0
    for centre in centres:
        cluster, keep, cdist = _carve(data, int(centre), 4 * cutoff, 3 * cutoff, cutoff)
        ref = M.energy_and_forces(params, cluster)
        inner = np.flatnonzero(cdist < 2 * cutoff - 1e-9)  # nodes whose energy is exact in the cluster
        e_ref = ref["node_energy"][inner]
        e_got = node_e[keep[inner]]
        scale = float(e_ref.abs().max())
        err_e = float((e_got - e_ref).abs().max()) / scale
        me = int(np.flatnonzero(keep == centre)[0])
        err_f = float((forces[centre] - ref["forces"][me]).abs().max())
        _say("  atom %6d: cluster of %d atoms, %d edges; %d node energies max err %.2e of max |E_n| = %.3g; |dF| %.2e (|F| %.3g)"
             % (centre, keep.size, cluster["edge_index"].shape[1], inner.size, err_e, scale, err_f,
                float(ref["forces"][me].abs().max())))
        assert err_e <= E_RTOL, (centre, err_e)
        assert err_f <= F_ATOL, (centre, err_f)
        worst_e, worst_f, checked = max(worst_e, err_e), max(worst_f, err_f), checked + inner.size
    return worst_e, worst_f, checked


def test_config4_full_size_against_reference_clusters(cabi):
    """Benchmark configuration 4 at its real size (25 000 atoms, 128 channels, 1.3 M edges): node energies of about 400
    atoms around each of several centres and the force on every centre against the fp64 reference evaluated on the
    carved neighbourhoods.  Centres include the first and last atom and atoms at both ends of the box."""
    _say("model c4 vs reference clusters")
    data = make_system(25000, 10, seed=0, density=0.1)
    params, model = _build(128, tuple(range(1, 11)), data, seed=0)
    out = model(to_device(data, "cuda"))
    centres = [0, 24999] + np.random.default_rng(1).integers(0, 25000, 3).tolist()
    worst_e, worst_f, checked = _check_against_carved_clusters(params, data, out, centres)
    _say("  c4: %d node energies within %.2e, %d forces within %.2e" % (checked, worst_e, len(centres), worst_f))


def test_config5_full_size_against_reference_clusters(cabi):
    """Benchmark configuration 5 at its real size (100 000 atoms, 192 channels, 5.2 M edges), as above."""
    _say("model c5 vs reference clusters")
    data = make_system(100000, 10, seed=0, density=0.1)
    params, model = _build(192, tuple(range(1, 11)), data, seed=0)
    out = model(to_device(data, "cuda"))
    centres = [0, 99999] + np.random.default_rng(2).integers(0, 100000, 2).tolist()
    worst_e, worst_f, checked = _check_against_carved_clusters(params, data, out, centres)
    _say("  c5: %d node energies within %.2e, %d forces within %.2e" % (checked, worst_e, len(centres), worst_f))


def test_model_in_a_foreign_coupling_basis(cabi):
    """A source model whose contraction modules carry their own coupling tensors (upstream's U_matrix buffers) in a
    permuted, sign-flipped path basis: the converted model follows that basis, and matches the fp64 reference fed the
    same tensors, in the fused and in the separate-op contraction."""
    from cuda_mace.models import OptimizedInvariantMACE, SyntheticInvariantMACE

    data = make_system(300, 4, seed=8, density=0.1)
    avg = data["edge_index"].shape[1] / 300
    up = SyntheticInvariantMACE(channels=64, atomic_numbers=(1, 6, 7, 8), avg_num_neighbors=avg, seed=6, coupling_basis_seed=5)
    params = up.export_params()
    assert "U3" in params["layers"][0]
    for fused_contraction in (True, False):
        model = OptimizedInvariantMACE(up, device="cuda", fused_contraction=fused_contraction)
        _compare(params, model, data)
    # the same weights read in the package's own basis give another model: the buffers matter
    own = SyntheticInvariantMACE(channels=64, atomic_numbers=(1, 6, 7, 8), avg_num_neighbors=avg, seed=6)
    ref_own = M.energy_and_forces(own.export_params(), data)
    ref = M.energy_and_forces(params, data)
    assert abs(float(ref_own["interaction_energy"]) - float(ref["interaction_energy"])) > 1e-3 * abs(float(ref["interaction_energy"]))


@pytest.mark.parametrize("case", ["cluster", "periodic96", "periodic192", "batch_relabelled", "isolated_atoms", "single_atom"])
def test_native_step_equals_autograd_path(cabi, case):
    """The step enqueued by the library in one call (cm_mace_step) against the same kernels driven from Python through
    autograd: identical node energies and features (same kernels in the same order), energies equal up to the order of
    the final sum, forces equal up to single-precision rounding of the gradient sums (the library adds the three
    contributions to the gradient of the first layer's features in the linear kernels' epilogues, autograd in separate
    additions)."""
    from cuda_mace.models import OptimizedInvariantMACE, SyntheticInvariantMACE
    from cuda_mace.utils.synthetic import collate

    kwargs = {}
    if case == "cluster":
        data, C, numbers = make_system(21, 4, seed=0, density=None, cluster_box=8.0), 64, (1, 6, 7, 8)
    elif case == "periodic96":
        data, C, numbers = make_system(300, 10, seed=1, density=0.1), 96, tuple(range(1, 11))
    elif case == "periodic192":
        data, C, numbers = make_system(250, 10, seed=3, density=0.1), 192, tuple(range(1, 11))
    elif case == "batch_relabelled":
        data = collate([make_system(n, 4, seed=30 + k, density=0.1) for k, n in enumerate((150, 230, 120))])
        C, numbers, kwargs = 64, (1, 6, 7, 8), dict(spatial_order_min_atoms=0)
    elif case == "single_atom":  # no edge at all: the energy is E0 + shift, the force zero
        data, C, numbers = make_system(1, 4, seed=2, density=None, cluster_box=4.0), 32, (1, 6, 7, 8)
        assert data["edge_index"].shape[1] == 0
    else:  # a sparse cluster: most atoms have no neighbour at all
        data, C, numbers = make_system(12, 4, seed=2, density=None, cluster_box=40.0, min_dist=3.0), 32, (1, 6, 7, 8)
    N = data["positions"].shape[0]
    up = SyntheticInvariantMACE(channels=C, atomic_numbers=numbers, avg_num_neighbors=max(data["edge_index"].shape[1] / N, 1.0),
                                seed=4, atomic_energies=torch.linspace(-3.0, -1.0, len(numbers), dtype=torch.float64), shift=0.1)
    native = OptimizedInvariantMACE(up, device="cuda", native_step=True, **kwargs)
    eager = OptimizedInvariantMACE(up, device="cuda", native_step=False, **kwargs)
    dev = to_device(data, "cuda")
    a, b = native(dict(dev)), eager(dict(dev))
    assert native._native not in (None, False) and eager._native is None  # the fast path ran / stayed off
    assert a["forces"].grad_fn is None and a["energy"].grad_fn is None
    _say("  %s: E native %.12g autograd %.12g" % (case, float(a["energy"].sum()), float(b["energy"].sum())))
    torch.testing.assert_close(a["energy"], b["energy"].detach(), rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(a["interaction_energy"], b["interaction_energy"].detach(), rtol=1e-12, atol=1e-12)
    assert torch.equal(a["node_energy"], b["node_energy"].detach())
    fscale = float(b["forces"].abs().max())
    torch.testing.assert_close(a["forces"], b["forces"].detach(), rtol=0, atol=5e-7 * fscale)
    assert torch.equal(a["node_feats"], b["node_feats"].detach())
    assert a["virials"] is None and a["stress"] is None and a["displacement"].shape == b["displacement"].shape
    again = native(dict(dev))
    assert torch.equal(again["forces"], a["forces"]) and torch.equal(again["energy"], a["energy"])
    # virials and stress come out of the same call (from the per-edge gradients, no strain tensor): the forces are the
    # same bits, the virials equal the strain derivative that the autograd path takes
    if case in ("periodic96", "batch_relabelled", "cluster"):
        c = native(dict(dev), compute_virials=True, compute_stress=True)
        d = eager(dict(dev), compute_virials=True, compute_stress=True)
        assert torch.equal(c["forces"], a["forces"]) and torch.equal(c["energy"], a["energy"])
        vscale = float(d["virials"].abs().max())
        torch.testing.assert_close(c["virials"], d["virials"].detach(), rtol=0, atol=2e-6 * vscale)
        torch.testing.assert_close(c["virials"], c["virials"].transpose(-1, -2), rtol=0, atol=0)
        torch.testing.assert_close(d["forces"].detach(), a["forces"], rtol=0, atol=5e-7 * fscale)
        if d["stress"] is None:
            assert c["stress"] is None
        else:
            torch.testing.assert_close(c["stress"], d["stress"].detach(), rtol=0, atol=2e-6 * float(d["stress"].abs().max()))
        # what the fast path does not cover still works on the same model: the strain tensor itself goes through autograd
        e = native(dict(dev), compute_displacement=True)
        assert e["displacement"].requires_grad and e["displacement"].shape == c["virials"].shape
    ref = M.energy_and_forces(up.export_params(), data)
    assert abs(float(a["energy"].sum()) - float(ref["energy"])) <= E_RTOL * abs(float(ref["energy"]))
    assert float((a["forces"].cpu() - ref["forces"]).abs().max()) <= F_ATOL


@pytest.mark.parametrize("relabel", [True, False], ids=["shell_last", "shell_in_place"])
def test_native_step_on_a_list_with_a_skin(cabi, relabel):
    """A neighbour list built out to cutoff + skin, at a size where the forward runs the LDS-table kernel: the step walks
    each receiver's edges only up to its last pair inside the cutoff (with relabelling the shell pairs sit at the end of
    every segment, without it they stay where the list has them).  Features and node energies equal the autograd path's on
    the same list bit for bit (a pair beyond the cutoff adds an exact zero there), energy and forces equal the exact
    list's up to the order of the sums."""
    from cuda_mace.models import OptimizedInvariantMACE, SyntheticInvariantMACE
    from cuda_mace.utils.neighbour_list import neighbour_data

    n, C = 2600, 64
    base = to_device(make_system(n, 4, seed=21, density=0.1), "cuda")
    avg = base["edge_index"].shape[1] / n
    up = SyntheticInvariantMACE(channels=C, atomic_numbers=(1, 6, 7, 8), avg_num_neighbors=avg, seed=9)
    kwargs = dict(spatial_order_min_atoms=0) if relabel else dict(spatial_order_min_atoms=None)
    native = OptimizedInvariantMACE(up, device="cuda", native_step=True, **kwargs)
    eager = OptimizedInvariantMACE(up, device="cuda", native_step=False, **kwargs)
    pbc = (True, True, True)
    wide = neighbour_data(base["positions"].clone(), base["node_attrs"], 5.6, pbc, base["cell"])
    exact = neighbour_data(base["positions"].clone(), base["node_attrs"], 5.0, pbc, base["cell"])
    assert wide["edge_index"].shape[1] > 1.3 * exact["edge_index"].shape[1]
    a, b, c = native(dict(wide)), eager(dict(wide)), native(dict(exact))
    assert native._native not in (None, False) and eager._native is None
    _say("  skin list (%s): E %.12g, exact list %.12g" % ("relabelled" if relabel else "as built", float(a["energy"].sum()),
                                                         float(c["energy"].sum())))
    assert torch.equal(a["node_feats"], b["node_feats"].detach()) and torch.equal(a["node_energy"], b["node_energy"].detach())
    fscale = float(c["forces"].abs().max())
    torch.testing.assert_close(a["forces"], b["forces"].detach(), rtol=0, atol=5e-7 * fscale)
    torch.testing.assert_close(a["energy"], c["energy"], rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(a["forces"], c["forces"], rtol=0, atol=2e-6 * fscale)


@pytest.mark.parametrize("natoms,channels", [(60, 64), (700, 128), (3000, 96)])
def test_step_with_chained_node_kernels_equals_the_separate_launches(cabi, natoms, channels, monkeypatch):
    """Up to 128 channels the one-call step runs the three [N,C] products between the layers, and their transposes, as one
    chained launch per direction (on 32-node tiles for few nodes, 128-node tiles otherwise) and sums the energies in that
    launch; the library's switch for the separate launches (CM_STEP_GLUE=-1, read per call) gives the same step as the
    same kernels beyond 128 channels run it.  Same operand split, piece order and rounding points: node energies, node
    features and forces agree bit for bit; the graph energy is a sum in another (fixed) order."""
    if natoms < 130:  # too few for a periodic box of twice the cutoff: a cluster
        data = make_system(natoms, 4, seed=5, density=None, cluster_box=10.0)
    else:
        data = make_system(natoms, 4, seed=5, density=0.1)
    _, model = _build(channels, (1, 6, 7, 8), data, seed=6)
    dev = to_device(data, "cuda")
    monkeypatch.delenv("CM_STEP_GLUE", raising=False)
    a = model(dict(dev))
    monkeypatch.setenv("CM_STEP_GLUE", "-1")
    b = model(dict(dev))
    monkeypatch.delenv("CM_STEP_GLUE")
    assert model._native not in (None, False)
    assert torch.equal(a["node_energy"], b["node_energy"]) and torch.equal(a["node_feats"], b["node_feats"])
    assert torch.equal(a["forces"], b["forces"])
    torch.testing.assert_close(a["energy"], b["energy"], rtol=1e-13, atol=1e-13)


@pytest.mark.parametrize("channels", [32, 64, 96, 128, 160, 192, 224, 256])
def test_repeated_evaluations_agree_bit_for_bit_at_every_width(cabi, channels):
    """Every kernel sums in a fixed order and reads nothing it (or an earlier kernel of the same step) has not written:
    the same input gives the same bits again, also after an evaluation of another size has left other values in the
    shared workspace.  Two sizes per width: with one wave per node and with a node's edges cut into parts (few nodes).
    (A kernel whose hand-issued loads were read before they had landed once passed every tolerance test and failed
    only this kind.)"""
    from cuda_mace.models import OptimizedInvariantMACE, SyntheticInvariantMACE

    boxes = {"large": to_device(make_system(2100, 4, seed=12, density=0.1), "cuda"),
             "small": to_device(make_system(260, 4, seed=11, density=0.1), "cuda")}
    up = SyntheticInvariantMACE(channels=channels, atomic_numbers=(1, 6, 7, 8), avg_num_neighbors=52.0, seed=13)
    model = OptimizedInvariantMACE(up, device="cuda")  # one model: both boxes share its workspace
    first = {k: model(dict(d)) for k, d in boxes.items()}
    assert model._native not in (None, False)
    for _ in range(2):
        for k, d in boxes.items():  # the other size ran in between: the workspace holds its leftovers
            again = model(dict(d))
            for key in ("energy", "node_energy", "forces", "node_feats"):
                assert torch.equal(again[key], first[k][key]), "%s of the %s box differs between evaluations at C=%d" % (key, k, channels)


def test_step_total_energies_through_the_library_call(cabi):
    """cm_mace_step's total_energy / total_node_energy: the interaction parts plus the constants handed over in the graph
    struct (graph_e0 per graph, node_e0 per atom in list order), the per-atom total written to the caller's rows; without
    the constants the totals are the interaction parts; an empty system returns the constants alone."""
    import ctypes

    from cuda_mace.models import OptimizedInvariantMACE, SyntheticInvariantMACE
    from cuda_mace.ops._autograd import groups_of, groups_of_one_hot
    from cuda_mace.ops.native_step import NativeStep
    from cuda_mace.utils.synthetic import collate

    data = to_device(collate([make_system(n, 4, seed=40 + k, density=0.1) for k, n in enumerate((140, 170))]), "cuda")
    n = data["positions"].shape[0]
    up = SyntheticInvariantMACE(channels=64, atomic_numbers=(1, 6, 7, 8), avg_num_neighbors=data["edge_index"].shape[1] / n, seed=41)
    model = OptimizedInvariantMACE(up, device="cuda", spatial_order_min_atoms=None)
    model(dict(data))  # builds the model's own step object and the caches on the tensors
    step = model._native
    assert isinstance(step, NativeStep)
    recv, send = data["edge_index"][0].int().contiguous(), data["edge_index"][1].int().contiguous()
    attrs32, types = data["node_attrs"].float(), data["node_attrs"].argmax(dim=-1).int()
    with torch.no_grad():
        X1 = model.interactions[0].linear_up(model.node_embedding(data["node_attrs"].double()).float())
    g = torch.Generator().manual_seed(42)
    rows = torch.randperm(n, generator=g).int().cuda()  # atom k of the lists is row rows[k] of the caller
    pos_rows = torch.empty_like(data["positions"])
    pos_rows[rows.long()] = data["positions"]
    node_e0 = torch.randn(n, generator=g, dtype=torch.float64).cuda()
    graph_e0 = torch.tensor([3.25, -1.5], dtype=torch.float64, device="cuda")
    plain = step.graph(data["edge_index"], recv, send, attrs32, types, data["ptr"], X1, rows)
    full = step.graph(data["edge_index"], recv, send, attrs32, types, data["ptr"], X1, rows, node_e0, graph_e0)
    a = step(plain, pos_rows, data["shifts"])
    b = step(full, pos_rows, data["shifts"])
    assert torch.equal(a["forces"], b["forces"]) and torch.equal(a["interaction_energy"], b["interaction_energy"])
    assert torch.equal(a["energy"], a["interaction_energy"])
    assert torch.equal(b["energy"], b["interaction_energy"] + graph_e0)
    expect = torch.empty(n, dtype=torch.float64, device="cuda")
    expect[rows.long()] = a["interaction_node_energy"]
    assert torch.equal(a["node_energy"], expect)
    expect[rows.long()] = b["interaction_node_energy"] + node_e0
    assert torch.equal(b["node_energy"], expect)
    # no atoms: zeros, or the constants
    lib = cabi.lib
    empty = ctypes.create_string_buffer(bytes(full.struct))
    from cuda_mace.ops.native_step import _Graph

    g0 = _Graph.from_buffer(empty)
    g0.nnodes, g0.nedges = 0, 0
    out_i = torch.full((2,), 7.0, dtype=torch.float64, device="cuda")
    out_t = torch.full((2,), 7.0, dtype=torch.float64, device="cuda")
    cabi._check(lib.cm_mace_step(ctypes.addressof(step.weights), ctypes.addressof(g0), None, None, None, 0, out_i.data_ptr(), None, None,
                                 None, None, out_t.data_ptr(), None, cabi._stream()))
    assert torch.equal(out_i, torch.zeros_like(out_i)) and torch.equal(out_t, graph_e0)


def test_step_without_the_feature_output(cabi):
    """compute_node_feats=False (what the MD calculators pass): the step skips the [N, 2C] fp64 output and nothing else
    changes."""
    data = make_system(500, 4, seed=7, density=0.1)
    _, model = _build(64, (1, 6, 7, 8), data, seed=8)
    dev = to_device(data, "cuda")
    a = model(dict(dev))
    b = model(dict(dev), compute_node_feats=False)
    assert model._native not in (None, False)
    assert a["node_feats"] is not None and b["node_feats"] is None
    for key in ("energy", "node_energy", "forces", "interaction_energy"):
        assert torch.equal(a[key], b[key])


def test_a_second_model_on_the_same_tensors_gets_its_own_graph_handle(cabi):
    """Model A evaluated on a batch and deleted, model B (other weights) built and evaluated on the very same tensors,
    several times over so that B's cache token can land on A's freed address: B's one-call step must use B's own first-layer
    features, i.e. agree with B's autograd path, and differ from A's result."""
    import gc

    from cuda_mace.models import OptimizedInvariantMACE, SyntheticInvariantMACE

    data = make_system(120, 4, seed=8, density=0.1)
    dev = to_device(data, "cuda")
    avg = data["edge_index"].shape[1] / 120
    last = None
    for seed in range(6):
        up = SyntheticInvariantMACE(channels=32, atomic_numbers=(1, 6, 7, 8), avg_num_neighbors=avg, seed=seed)
        model = OptimizedInvariantMACE(up, device="cuda", native_step=True)
        out = model(dict(dev))
        assert model._native not in (None, False)
        check = OptimizedInvariantMACE(up, device="cuda", native_step=False)(dict(dev))
        assert torch.equal(out["node_energy"], check["node_energy"].detach()), "seed %d ran on another model's handle" % seed
        if last is not None:
            assert not torch.equal(out["node_energy"], last)
        last = out["node_energy"].clone()
        del model, out, check, up
        gc.collect()


def test_captured_step_survives_a_larger_eager_evaluation(cabi):
    """A step captured as a HIP graph keeps its own workspace: evaluating the same model eagerly on a larger structure
    afterwards (which replaces the buffer eager calls share) must not disturb the replays."""
    from cuda_mace.models import OptimizedInvariantMACE, SyntheticInvariantMACE
    from cuda_mace.utils.graph import GraphedStep

    small, large = make_system(130, 4, seed=3, density=0.1), make_system(700, 4, seed=4, density=0.1)
    up = SyntheticInvariantMACE(channels=64, atomic_numbers=(1, 6, 7, 8), avg_num_neighbors=50.0, seed=2)
    model = OptimizedInvariantMACE(up, device="cuda")
    dev_small, dev_large = to_device(small, "cuda"), to_device(large, "cuda")
    step = GraphedStep(model, dev_small)
    first = {k: v.clone() for k, v in step().items() if k in ("energy", "forces", "node_energy")}
    big = model(dict(dev_large))
    torch.cuda.synchronize()
    big2 = model(dict(dev_large))
    # the eager buffer was replaced and is in use by other work; the replay still reads and writes its own
    for _ in range(3):
        again = step()
        torch.cuda.synchronize()
        for k, v in first.items():
            assert torch.equal(again[k], v), k
        junk = torch.randn(1 << 22, device="cuda")  # allocator traffic between replays
        del junk
    fresh = model(dict(dev_small))
    for k, v in first.items():
        assert torch.equal(fresh[k].detach(), v), k
    assert torch.equal(big["forces"], big2["forces"])
