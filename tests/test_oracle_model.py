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


# ---- pins of the model-level helpers: each fails when the constant it names is off by 1 % ------------------------
def test_bessel_basis_is_orthonormal_under_r2_dr():
    """int_0^rmax b_n(r) b_m(r) r^2 dr = delta_nm fixes the prefactor sqrt(2 / r_max) and the frequencies n pi / r_max."""
    r_max, nb = 5.0, 8
    x, w = np.polynomial.legendre.leggauss(400)
    r = torch.tensor(0.5 * r_max * (x + 1.0))
    w = torch.tensor(0.5 * r_max * w)
    b = M.bessel_basis(r, r_max, nb)
    gram = torch.einsum("e,en,em->nm", w * r * r, b, b)
    torch.testing.assert_close(gram, torch.eye(nb, dtype=torch.float64), atol=1e-12, rtol=0)
    # first zero of every b_n at r_max / n (sin(n pi r / r_max) = 0), and b_n -> sqrt(2 / r_max) n pi / r_max at r -> 0
    n = torch.arange(1, nb + 1, dtype=torch.float64)
    b0 = M.bessel_basis(torch.tensor([1e-9], dtype=torch.float64), r_max, nb)[0]
    torch.testing.assert_close(b0, math.sqrt(2.0 / r_max) * n * math.pi / r_max, rtol=1e-9, atol=0)


@pytest.mark.parametrize("p", [5, 6])
def test_polynomial_cutoff_boundary_conditions(p):
    """f(0) = 1, f(1) = f'(1) = f''(1) = 0 determine the three coefficients of 1 - a x^p + b x^(p+1) - c x^(p+2)."""
    x = torch.tensor([1.0 - 1e-300], dtype=torch.float64, requires_grad=True)  # just inside the cutoff
    f = M.polynomial_cutoff(x, p)
    (d1,) = torch.autograd.grad(f.sum(), x, create_graph=True)
    (d2,) = torch.autograd.grad(d1.sum(), x)
    assert abs(float(f)) < 1e-12 and abs(float(d1)) < 1e-11 and abs(float(d2)) < 1e-10
    z = torch.tensor([0.0, 1.0, 1.5], dtype=torch.float64)
    torch.testing.assert_close(M.polynomial_cutoff(z, p), torch.tensor([1.0, 0.0, 0.0], dtype=torch.float64))
    # independent solve of the 3 x 3 system for (a, b, c)
    A = np.array([[1.0, 1.0, 1.0], [p, p + 1, p + 2], [p * (p - 1), (p + 1) * p, (p + 2) * (p + 1)]])
    a, b, c = np.linalg.solve(A, np.array([-1.0, 0.0, 0.0]))
    xs = torch.linspace(0.05, 0.95, 7, dtype=torch.float64)
    want = 1.0 + a * xs ** p + b * xs ** (p + 1) + c * xs ** (p + 2)
    torch.testing.assert_close(M.polynomial_cutoff(xs, p), want, rtol=1e-10, atol=1e-12)


def _silu_second_moment():
    x, w = np.polynomial.hermite_e.hermegauss(200)
    silu = x / (1.0 + np.exp(-x))
    return float((w * silu ** 2).sum() / math.sqrt(2.0 * math.pi))


def test_activation_constant_normalises_the_second_moment():
    """SILU_2MOM^2 E_{z ~ N(0,1)}[silu(z)^2] = 1 (the normalize2mom convention).  Upstream's constant is a Monte-Carlo
    estimate over 10^6 seeded fp64 normals, which this recipe reproduces to the last digit; it lies 0.16 % from the
    exact value 1.67653 that Gauss-Hermite quadrature gives."""
    z = torch.randn(1_000_000, generator=torch.Generator().manual_seed(0), dtype=torch.float64)
    mc = 1.0 / math.sqrt(float((torch.nn.functional.silu(z) ** 2).mean()))
    assert abs(mc - M.SILU_2MOM) < 1e-14
    assert abs(M.SILU_2MOM ** 2 * _silu_second_moment() - 1.0) < 5e-3


def test_radial_mlp_keeps_unit_second_moment():
    """Unit-variance weights and inputs of unit second moment give outputs of second moment SILU_2MOM^2 E[silu^2]
    (= 1.003) and zero mean: fixes the 1/sqrt(fan_in) of every layer (1 % off moves the result by 4 %), the activation
    constant (2 %) and that the last layer is linear (a gated output would have mean 0.35).  Wide layers keep the
    finite-width bias and the sampling noise at 0.3 % each."""
    g = torch.Generator().manual_seed(0)
    widths = [1024, 1024, 4096]
    x = torch.randn(2000, widths[0], generator=g, dtype=torch.float64)
    x = x / x.norm(dim=1, keepdim=True) * math.sqrt(widths[0])
    Ws = [torch.randn(a, b, generator=g, dtype=torch.float64) for a, b in zip(widths[:-1], widths[1:])]
    out = M.radial_mlp(x, Ws)
    want = M.SILU_2MOM ** 2 * _silu_second_moment()
    assert abs(float((out ** 2).mean()) - want) < 0.01, float((out ** 2).mean())
    assert abs(float(out.mean())) < 0.03
    # a single layer is a plain scaled product: second moment |x|^2 / fan_in exactly in expectation
    one = M.radial_mlp(x[:50], [Ws[1]])
    assert abs(float((one ** 2).mean()) - 1.0) < 0.01


def test_nested_contraction_equals_dense_definition():
    """contraction_nested (the form the model evaluates) against oracle.ops.symmetric_contraction, which
    tests/test_oracle_pins.py pins by python-loop brute force."""
    from oracle import ops as O
    from oracle.u_tensors import u_tensors

    g = torch.Generator().manual_seed(3)
    N, C, ne = 13, 5, 3
    U1, U2, U3 = (torch.from_numpy(u) for u in u_tensors())
    X = torch.randn(N, 16, C, generator=g, dtype=torch.float64)
    elem = torch.randint(0, ne, (N,), generator=g)
    W3 = torch.randn(ne, U3.shape[-1], C, generator=g, dtype=torch.float64)
    W2 = torch.randn(ne, U2.shape[-1], C, generator=g, dtype=torch.float64)
    W1 = torch.randn(ne, 1, C, generator=g, dtype=torch.float64)
    got = M.contraction_nested(X, elem, W3, W2, W1, U3, U2)
    want = O.symmetric_contraction(X, elem, U3, U2, W3, W2, W1)
    torch.testing.assert_close(got, want, rtol=1e-11, atol=1e-11)


def test_message_has_unit_path_weight(setup):
    """The per-edge product carries no factor besides u[sender] Y R (path weight 1 of the uvu tensor product, as in the
    reference's own check, tests/invariant_message_passing.py:93-120): for one edge, one channel and R = 1 the
    aggregated message on the receiver is exactly u * Y(r), with Y_00 = 1 and sum_m Y_1m^2 = 3."""
    from oracle import ops as O

    vec = torch.tensor([[0.3, -1.1, 0.7]], dtype=torch.float64)
    Y = O.spherical_harmonics(vec)  # [16, 1]
    u = torch.tensor([[2.0], [0.0]], dtype=torch.float64)
    A = O.mp_forward(u, Y, torch.ones(1, 4, 1, dtype=torch.float64), torch.tensor([0]), torch.tensor([1]), 2)
    torch.testing.assert_close(A[1, :, 0], 2.0 * Y[:, 0])
    assert float(A[0].abs().max()) == 0.0
    assert abs(float(Y[0, 0]) - 1.0) < 1e-14 and abs(float((Y[1:4, 0] ** 2).sum()) - 3.0) < 1e-13


def test_single_atom_energy_is_closed_form():
    """An isolated atom receives no messages: A = 0, so B = 0 (every contraction term is at least linear in A), h1 = 0,
    the layer-2 skip connection (a function of h1) is 0 and h2 = 0; silu(0) = 0, so both readouts vanish and the energy
    is E0[element] + shift exactly, whatever the weights and the scale."""
    e0 = torch.tensor([-13.6, -1029.0, -1485.0, -2042.0], dtype=torch.float64)
    model = SyntheticInvariantMACE(channels=32, atomic_numbers=(1, 6, 7, 8), avg_num_neighbors=9.0, seed=0,
                                   atomic_energies=e0, scale=0.7, shift=0.25)
    p = model.export_params()
    for e in (0, 2):
        attrs = torch.zeros(1, 4, dtype=torch.float64)
        attrs[0, e] = 1.0
        data = dict(positions=torch.zeros(1, 3, dtype=torch.float64), node_attrs=attrs,
                    edge_index=torch.zeros(2, 0, dtype=torch.long), shifts=torch.zeros(0, 3, dtype=torch.float64))
        out = M.energy_and_forces(p, data, compute_forces=False)
        assert abs(float(out["energy"]) - (float(e0[e]) + 0.25)) < 1e-12
        assert abs(float(out["interaction_energy"]) - 0.25) < 1e-15


def test_two_atom_energy_is_closed_form():
    """Two atoms at distance d along z, one channel per l that matters: with Y(z-axis) known in closed form (Y_l0 =
    sqrt(2l+1), every other component 0) both layers are a hand-computable scalar chain.  Checks the chain
    radial basis -> MLP -> message -> 1/avg_num_neighbors -> linear -> per-element linear (on the message in layer 1,
    as skip connection in layer 2) -> contraction -> product linear -> both readouts -> scale, shift, E0, with
    independent arithmetic (numpy, explicit loops over the 16 components, the hidden units and the channels)."""
    scale, shift = 1.7, -0.4
    model = SyntheticInvariantMACE(channels=32, atomic_numbers=(1, 6), avg_num_neighbors=3.0, seed=5, scale=scale,
                                   shift=shift, atomic_energies=torch.tensor([-1.25, 3.5]))
    p = model.export_params()
    C, ne, d = 32, 2, 1.7
    attrs = torch.tensor([[1.0, 0.0], [0.0, 1.0]], dtype=torch.float64)
    pos = torch.tensor([[0.0, 0.0, 0.0], [0.0, 0.0, d]], dtype=torch.float64)
    data = dict(positions=pos, node_attrs=attrs, edge_index=torch.tensor([[0, 1], [1, 0]]),
                shifts=torch.zeros(2, 3, dtype=torch.float64))
    out = M.energy_and_forces(p, data, compute_forces=False)
    from oracle import ops as O
    from oracle.u_tensors import u_tensors

    U1, U2, U3 = u_tensors()
    r_max, nb, pw = float(p["r_max"]), int(p["num_bessel"]), int(p["p"])
    x = d / r_max
    env = 1 - (pw + 1) * (pw + 2) / 2 * x ** pw + pw * (pw + 2) * x ** (pw + 1) - pw * (pw + 1) / 2 * x ** (pw + 2)
    basis = np.array([math.sqrt(2 / r_max) * math.sin(n * math.pi * d / r_max) / d * env for n in range(1, nb + 1)])
    h0 = (attrs @ p["W_emb"].double() / math.sqrt(ne)).numpy()

    def layer_by_hand(t, h_in):
        lay = p["layers"][t]
        z = basis
        mlp = [W.double().numpy() for W in lay["mlp"]]
        for i, W in enumerate(mlp):
            z = z @ W / math.sqrt(W.shape[0])
            if i + 1 < len(mlp):
                z = M.SILU_2MOM * z / (1 + np.exp(-z))
        R = z.reshape(4, C)
        u = h_in @ lay["W_up"].double().numpy() / math.sqrt(C)
        h_out = np.zeros((2, C))
        W_lin, W_skip = lay["W_lin"].double().numpy(), lay["W_skip"].double().numpy()
        for rcv, snd, sign in ((1, 0, +1.0), (0, 1, -1.0)):  # edge vector = pos[rcv] - pos[snd] = +-d along the 3rd axis
            # harmonics of +-z in the oracle's component order, taken from the scipy-pinned routine
            Y = O.spherical_harmonics(torch.tensor([[0.0, 0.0, sign * d]], dtype=torch.float64))[:, 0].numpy()
            A = np.zeros((16, C))
            for m in range(16):
                l = int(math.isqrt(m))
                msg = u[snd] * Y[m] * R[l]
                A[m] = (msg @ W_lin[l]) / math.sqrt(C) / 3.0
                if t == 0:  # the first layer's per-element linear acts on the message; element of atom rcv is rcv
                    A[m] = (A[m] @ W_skip[l][:, rcv, :]) / math.sqrt(C * ne)
            e = rcv
            B = np.zeros(C)
            W3, W2, W1 = (lay[k].double().numpy()[e] for k in ("W3", "W2", "W1"))
            for c in range(C):
                a = A[:, c]
                B[c] = (np.einsum("ijkp,p,i,j,k->", U3, W3[:, c], a, a, a) + np.einsum("ijp,p,i,j->", U2, W2[:, c], a, a)
                        + W1[0, c] * a[0])
            h_out[rcv] = B @ lay["W_prod"].double().numpy() / math.sqrt(C)
            if t == 1:  # the second layer's per-element linear is the skip connection on the incoming scalars
                h_out[rcv] += h_in[rcv] @ W_skip[0][:, rcv, :] / math.sqrt(C * ne)
        return h_out

    h1 = layer_by_hand(0, h0)
    h2 = layer_by_hand(1, h1)
    np.testing.assert_allclose(out["node_feats"][:, :C].numpy(), h1, rtol=1e-10, atol=1e-13)
    np.testing.assert_allclose(out["node_feats"][:, C:].numpy(), h2, rtol=1e-9, atol=1e-13)
    # readouts, scale and shift with scalar arithmetic: linear readout of layer 1; layer 2 through 16 hidden units
    # with the normalised silu gate; every weight divided by the square root of its fan-in; E0 of the element
    w0 = p["w_read0"].double().numpy()[:, 0]
    Wa, wb = p["W_read1"].double().numpy(), p["w_read2"].double().numpy()[:, 0]
    hidden = Wa.shape[1]
    assert hidden == 16 and abs(scale - 1.0) > 0.1 and abs(shift) > 0.1
    e_node = np.zeros(2)
    for n in range(2):
        e1 = sum(h1[n, c] * w0[c] for c in range(C)) / math.sqrt(C)
        e2 = 0.0
        for k in range(hidden):
            zk = sum(h2[n, c] * Wa[c, k] for c in range(C)) / math.sqrt(C)
            e2 += wb[k] * M.SILU_2MOM * zk / (1 + math.exp(-zk))
        e2 /= math.sqrt(hidden)
        e_node[n] = float(p["E0"][n]) + scale * (e1 + e2) + shift
        assert abs(e1) > 1e-6 and abs(e2) > 1e-6
    np.testing.assert_allclose(out["node_energy"].numpy(), e_node, rtol=1e-10, atol=1e-13)
    assert abs(float(out["energy"]) - e_node.sum()) < 1e-12 * max(1.0, abs(e_node.sum()))
    # the comparison has teeth: a 1 % error in the gate constant or in 1/sqrt(hidden) is 1e6 tolerances away
    assert np.abs(out["node_energy"].numpy() - e_node).max() < 1e-3 * abs(scale * 0.01 * e2)


def test_carving_is_exact_on_the_reference_itself():
    """The locality argument behind the carved clusters, checked on the CPU in fp64: node energies within two cutoffs
    of the centre and the force on the centre, computed on the cluster, equal those of the whole periodic box."""
    from tests.util import carve_cluster

    cutoff = 1.8  # a short cutoff and a dense box keep 4 cutoffs inside half the box of a small system
    data = make_system(1000, 3, seed=11, density=0.3, cutoff=cutoff)
    up = SyntheticInvariantMACE(channels=32, atomic_numbers=(1, 6, 8), r_max=cutoff,
                                avg_num_neighbors=data["edge_index"].shape[1] / 1000, seed=4)
    params = up.export_params()
    full = M.energy_and_forces(params, data)
    teeth = 0.0
    for centre in (0, 350, 999):
        cluster, keep, cdist = carve_cluster(data, centre, 4 * cutoff, 3 * cutoff, cutoff)
        assert keep.size < 600
        ref = M.energy_and_forces(params, cluster)
        inner = np.flatnonzero(cdist < 2 * cutoff - 1e-9)
        assert inner.size >= 5
        torch.testing.assert_close(ref["node_energy"][inner], full["node_energy"][keep[inner]], rtol=1e-10, atol=1e-12)
        me = int(np.flatnonzero(keep == centre)[0])
        torch.testing.assert_close(ref["forces"][me], full["forces"][centre], rtol=1e-9, atol=1e-11)
        # a cluster that is too small fails the same comparison: the check has teeth
        small, keep_s, _ = carve_cluster(data, centre, 2 * cutoff, 1.5 * cutoff, cutoff)
        bad = M.energy_and_forces(params, small)
        teeth += float((bad["forces"][int(np.flatnonzero(keep_s == centre)[0])] - full["forces"][centre]).abs().max())
    assert teeth > 1e-5
