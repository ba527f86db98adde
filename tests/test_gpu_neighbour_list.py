"""Device neighbour list (cm_neighbour_list_count / _fill) against the brute-force oracle: identical integer output."""
import numpy as np
import pytest
import torch

from oracle import ops as O

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _device_list(pos, cell, pbc, cutoff, max_cells=0):
    from cuda_mace import _cabi as cabi

    p = torch.tensor(pos, dtype=torch.float64, device=DEV).reshape(-1, 3)
    c = None if cell is None else torch.tensor(cell, dtype=torch.float64, device=DEV)
    ri, rj, S = cabi.neighbour_list(p, c, pbc, cutoff, max_cells)
    return np.stack([ri.cpu().numpy(), rj.cpu().numpy()]).astype(np.int64), S.cpu().numpy().astype(np.int64)


def _check(pos, cell, pbc, cutoff, max_cells=0):
    ei, S = _device_list(pos, cell, pbc, cutoff, max_cells)
    ei_ref, S_ref = O.neighbour_list(pos, cell, pbc, cutoff)
    assert ei.shape == ei_ref.shape, (ei.shape, ei_ref.shape)
    assert np.array_equal(ei, ei_ref)
    assert np.array_equal(S, S_ref)
    return ei, S


CASES = {
    "cluster": dict(n=60, lo=0.0, hi=9.0, cell=None, pbc=(0, 0, 0), cutoff=5.0),
    "cluster_with_unused_cell": dict(n=40, lo=-4.0, hi=7.0, cell=np.eye(3) * 30.0, pbc=(0, 0, 0), cutoff=4.0),
    "cubic": dict(n=300, lo=0.0, hi=14.0, cell=np.eye(3) * 14.0, pbc=(1, 1, 1), cutoff=5.0),
    "cubic_unwrapped": dict(n=200, lo=-40.0, hi=55.0, cell=np.eye(3) * 13.0, pbc=(1, 1, 1), cutoff=5.0),
    "orthorhombic_slab": dict(n=150, lo=0.0, hi=11.0, cell=np.diag([11.0, 16.0, 40.0]), pbc=(1, 1, 0), cutoff=5.0),
    "triclinic": dict(n=120, lo=-2.0, hi=15.0, cell=np.array([[12.0, 0, 0], [3.0, 11.0, 0], [-2.0, 4.0, 13.0]]),
                      pbc=(1, 1, 1), cutoff=5.0),
    "small_cell_many_images": dict(n=7, lo=-3.0, hi=8.0, cell=np.array([[4.0, 0, 0], [1.0, 3.5, 0], [0.5, 0.7, 4.2]]),
                                   pbc=(1, 1, 1), cutoff=5.0),
    "wire": dict(n=25, lo=0.0, hi=6.0, cell=np.array([[0.0, 0, 3.1], [7.0, 0.0, 0], [0.0, 9.0, 0.0]]), pbc=(1, 0, 0),
                 cutoff=4.5),
    "left_handed_cell": dict(n=50, lo=0.0, hi=12.0, cell=np.array([[0, 12.0, 0], [12.5, 0, 0], [0, 0, 13.0]]),
                             pbc=(1, 1, 1), cutoff=5.0),
}


@pytest.mark.parametrize("name", sorted(CASES))
def test_neighbour_list_matches_brute_force(cabi, name):
    k = CASES[name]
    rng = np.random.default_rng(sorted(CASES).index(name))
    pos = rng.uniform(k["lo"], k["hi"], (k["n"], 3))
    ei, S = _check(pos, k["cell"], k["pbc"], k["cutoff"])
    assert ei.shape[1] > 0
    assert np.all(np.diff(ei[0]) >= 0)
    # every pair appears with its reverse
    fwd = {tuple(r) for r in np.concatenate([ei.T, S], axis=1)}
    assert fwd == {(j, i, -a, -b, -c) for (i, j, a, b, c) in fwd}


def test_bin_cap_does_not_change_the_list(cabi):
    rng = np.random.default_rng(5)
    pos = rng.uniform(0, 30.0, (400, 3))
    cell = np.eye(3) * 30.0
    base = _device_list(pos, cell, (1, 1, 1), 4.0)
    for cap in (1, 2, 7, 50):
        got = _device_list(pos, cell, (1, 1, 1), 4.0, max_cells=cap)
        assert np.array_equal(got[0], base[0]) and np.array_equal(got[1], base[1])
    ref = O.neighbour_list(pos, cell, (1, 1, 1), 4.0)
    assert np.array_equal(base[0], ref[0]) and np.array_equal(base[1], ref[1])


def test_degenerate_inputs(cabi):
    from cuda_mace import _cabi as cabi_mod

    # no atoms, one atom without and with self-images, two atoms out of range, coincident coordinates along an axis
    ei, S = _device_list(np.zeros((0, 3)), None, (0, 0, 0), 5.0)
    assert ei.shape == (2, 0) and S.shape == (0, 3)
    ei, S = _device_list(np.array([[1.0, 2.0, 3.0]]), None, (0, 0, 0), 5.0)
    assert ei.shape == (2, 0)
    _check(np.array([[1.0, 2.0, 3.0]]), np.eye(3) * 3.0, (1, 1, 1), 5.0)
    ei, _ = _device_list(np.array([[0.0, 0, 0], [9.0, 0, 0]]), None, (0, 0, 0), 5.0)
    assert ei.shape == (2, 0)
    planar = np.random.default_rng(3).uniform(0, 8.0, (30, 3))
    planar[:, 2] = 1.25
    _check(planar, None, (0, 0, 0), 3.0)
    with pytest.raises(cabi_mod.CudaMaceError, match="singular"):
        _device_list(planar, np.zeros((3, 3)), (1, 1, 1), 3.0)
    with pytest.raises(cabi_mod.CudaMaceError):
        _device_list(planar, None, (0, 0, 0), -1.0)


def test_full_size_box_equals_host_list_and_feeds_the_model(cabi):
    """25 000 atoms: the device list equals the host list of the benchmark generator entry for entry, and the model gives
    bit-identical energy and forces from either."""
    from cuda_mace.models import OptimizedInvariantMACE, SyntheticInvariantMACE
    from cuda_mace.utils.neighbour_list import get_neighborhood
    from cuda_mace.utils.synthetic import make_system, to_device

    data = make_system(25000, 10, seed=0)
    dev = to_device(data, DEV)
    edge_index, shifts, unit_shifts, cell = get_neighborhood(dev["positions"], 5.0, (True, True, True), dev["cell"])
    assert torch.equal(edge_index.cpu(), data["edge_index"])
    assert torch.equal(unit_shifts.cpu(), data["unit_shifts"])
    assert torch.allclose(shifts.cpu(), data["shifts"], rtol=0, atol=1e-12)
    avg = data["edge_index"].shape[1] / 25000
    model = OptimizedInvariantMACE(SyntheticInvariantMACE(channels=32, atomic_numbers=tuple(range(1, 11)), avg_num_neighbors=avg,
                                                          seed=1), device=DEV)
    out_host = model(dict(dev))
    dev2 = dict(to_device(data, DEV))
    dev2.update(edge_index=edge_index, shifts=shifts, unit_shifts=unit_shifts)
    out_dev = model(dev2)
    assert torch.equal(out_host["energy"], out_dev["energy"])
    assert torch.equal(out_host["forces"], out_dev["forces"])


@pytest.mark.parametrize("n", [0, 1, 63, 1000, 300_001])
def test_max_displacement(cabi, n):
    """cm_max_displacement against the same maximum taken by torch in fp64 (bit-exact: squares and sums of three terms,
    left to right without fused multiply-adds, then a maximum); a NaN coordinate gives +inf."""
    g = torch.Generator(device="cuda").manual_seed(n)
    ref = 20.0 * torch.rand(n, 3, device="cuda", dtype=torch.float64, generator=g)
    pos = ref + 0.1 * torch.randn(n, 3, device="cuda", dtype=torch.float64, generator=g)
    got = cabi.max_displacement(pos, ref)
    d = pos - ref
    want = (d[:, 0] * d[:, 0] + d[:, 1] * d[:, 1] + d[:, 2] * d[:, 2]).max() if n else torch.zeros((), dtype=torch.float64)
    assert got.shape == (1,) and float(got[0]) == float(want)
    if n:
        pos[n // 2, 1] = float("nan")
        assert float(cabi.max_displacement(pos, ref, out=got)[0]) == float("inf")


@pytest.mark.parametrize("case", ["periodic_skin", "batch", "exact_list", "cluster", "no_edges", "headline"])
def test_graph_prepare_matches_the_host_restatement(cabi, case):
    """cm_graph_prepare (relabelled atoms, re-sorted pairs with the skin shell last, CSR offsets, sender-sorted view) entry
    for entry against a numpy restatement with library sorts, and its derived structures against the index oracles."""
    from cuda_mace.utils.synthetic import collate, make_system
    from oracle import ops as O
    from tests.util import spatial_order_reference

    r_max = 5.0
    if case == "periodic_skin":
        data = make_system(400, 4, seed=5, density=0.1, cutoff=5.6)
    elif case == "batch":
        data = collate([make_system(n, 4, seed=20 + k, density=0.1, cutoff=5.2) for k, n in enumerate((150, 230, 120))])
    elif case == "exact_list":
        data = make_system(300, 4, seed=6, density=0.1)
    elif case == "cluster":
        data = make_system(21, 4, seed=0, density=None, cluster_box=8.0)
    elif case == "no_edges":
        data = make_system(12, 4, seed=2, density=None, cluster_box=60.0, min_dist=8.0)
        assert data["edge_index"].shape[1] == 0
    else:
        data = make_system(25000, 10, seed=0, density=0.1, cutoff=5.5)
    N, E = data["positions"].shape[0], data["edge_index"].shape[1]
    ngraphs = int(data["ptr"].numel()) - 1
    print("graph_prepare", case, N, E, ngraphs, flush=True)
    dev = lambda t: t.to("cuda").contiguous()  # noqa: E731
    bins = 64 if ngraphs == 1 else 16
    got = cabi.graph_prepare(dev(data["positions"].double()), dev(data["edge_index"][0].int()), dev(data["edge_index"][1].int()),
                             dev(data["shifts"].double()), None if ngraphs == 1 else dev(data["batch"].int()), ngraphs, r_max, bins)
    perm, inverse, rcv, snd, order = spatial_order_reference(data["positions"], data["batch"], data["edge_index"], data["shifts"],
                                                             r_max, bins)
    eq = lambda name, want: np.testing.assert_array_equal(got[name].cpu().numpy(), want, err_msg=name)  # noqa: E731
    eq("node_perm", perm)
    eq("node_inverse", inverse)
    eq("receiver", rcv)
    eq("sender", snd)
    eq("edge_perm", order)
    assert torch.equal(got["shifts"].cpu(), data["shifts"].double()[torch.from_numpy(order)])
    assert torch.equal(got["first_occ"].cpu(), O.first_occurences(torch.from_numpy(rcv).int(), N))
    sperm, soff = O.stable_key_sort(torch.from_numpy(snd).int(), N)
    assert torch.equal(got["sender_perm"].cpu(), sperm) and torch.equal(got["sender_offsets"].cpu(), soff)
    if E:
        # every receiver's pairs beyond the cutoff come last
        v = data["positions"][data["edge_index"][1]] - data["positions"][data["edge_index"][0]] + data["shifts"]
        beyond = (v.norm(dim=1) > r_max)[torch.from_numpy(order)]
        fo = got["first_occ"].cpu()
        for n in (0, N // 2, N - 1):
            seg = beyond[fo[n]:fo[N + n]]
            assert bool((seg[1:] >= seg[:-1]).all())
