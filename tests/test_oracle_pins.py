"""Pins of the CPU oracle against closed forms, library routines and brute force (no GPU).

A wrong sign, index, transposed operand or dropped term in oracle/ops.py fails at least one of
these; none of them re-types the oracle's own formula.
"""
import math

import numpy as np
import pytest
import torch

from oracle import ops as O
from tests.util import mp_inputs, random_graph



@pytest.fixture(autouse=True)
def _fp64_default():
    old = torch.get_default_dtype()
    torch.set_default_dtype(torch.float64)
    yield
    torch.set_default_dtype(old)


# ---- index kernels -------------------------------------------------------------------------------
def test_first_occurences_brute_force():
    recv = torch.tensor([0, 0, 2, 2, 2, 5], dtype=torch.int32)
    fo = O.first_occurences(recv, 7)
    assert fo[:7].tolist() == [0, 2, 2, 5, 5, 5, 6]
    assert fo[7:].tolist() == [2, 2, 5, 5, 5, 6, 6]
    for n in range(7):  # python scan
        idx = [e for e in range(6) if recv[e] == n]
        if idx:
            assert fo[n] == idx[0] and fo[7 + n] == idx[-1] + 1
        else:
            assert fo[n] == fo[7 + n]
    assert O.first_occurences(torch.zeros(0, dtype=torch.int32), 3).tolist() == [0] * 6


def test_stable_key_sort_matches_torch_sort():
    keys = torch.from_numpy(np.random.default_rng(0).integers(0, 13, 500).astype(np.int32))
    perm, off = O.stable_key_sort(keys, 13)
    _, ref = torch.sort(keys.long(), stable=True)
    assert torch.equal(perm.long(), ref)
    assert off[0] == 0 and off[-1] == 500
    for k in range(13):
        assert int(off[k + 1] - off[k]) == int((keys == k).sum())


# ---- message passing ---------------------------------------------------------------------------------
def test_mp_forward_brute_force_loops():
    """Python loops over edges on a tiny non-symmetric multigraph with an isolated node."""
    N, C = 5, 3
    sender = torch.tensor([1, 1, 4, 0, 2, 2], dtype=torch.int32)  # duplicate edge 1->0
    receiver = torch.tensor([0, 0, 0, 2, 3, 3], dtype=torch.int32)  # node 1 and 4 receive nothing
    X, v, R, _ = mp_inputs(N, 6, C, 0)
    Y = torch.randn(16, 6)
    out = O.mp_forward(X, Y, R, sender, receiver, N)
    ref = torch.zeros(N, 16, C)
    for e in range(6):
        for m in range(16):
            l = int(math.floor(math.sqrt(m)))
            for c in range(C):
                ref[receiver[e], m, c] += X[sender[e], c] * Y[m, e] * R[e, l, c]
    torch.testing.assert_close(out, ref)
    assert float(out[1].abs().sum()) == 0.0 and float(out[4].abs().sum()) == 0.0


def test_mp_backward_is_autograd_of_forward():
    snd, rcv = random_graph(40, 5, 3, isolated_frac=0.2)
    X, v, R, G = mp_inputs(40, snd.numel(), 8, 3)
    Y = torch.randn(16, snd.numel())
    Xa, Ya, Ra = (t.clone().requires_grad_(True) for t in (X, Y, R))
    (O.mp_forward(Xa, Ya, Ra, snd, rcv, 40) * G).sum().backward()
    gX, gY, gR = O.mp_backward(X, Y, R, G, snd, rcv)
    torch.testing.assert_close(gX, Xa.grad)
    torch.testing.assert_close(gY, Ya.grad)
    torch.testing.assert_close(gR, Ra.grad)


def test_mp_per_component_weights_brute_force_and_autograd():
    """The variant with one radial weight per component, R [E, 16, C]: python loops for the forward, autograd of the
    forward for the three gradients; with R[e, m] = R4[e, l(m)] it reduces to the reference's op."""
    N, C = 5, 3
    sender = torch.tensor([1, 1, 4, 0, 2, 2], dtype=torch.int32)
    receiver = torch.tensor([0, 0, 0, 2, 3, 3], dtype=torch.int32)
    g = torch.Generator().manual_seed(5)
    X = torch.randn(N, C, generator=g, dtype=torch.float64)
    Y = torch.randn(16, 6, generator=g, dtype=torch.float64)
    R = torch.randn(6, 16, C, generator=g, dtype=torch.float64)
    G = torch.randn(N, 16, C, generator=g, dtype=torch.float64)
    out = O.mp_forward(X, Y, R, sender, receiver, N)
    ref = torch.zeros(N, 16, C, dtype=torch.float64)
    for e in range(6):
        for m in range(16):
            for c in range(C):
                ref[receiver[e], m, c] += X[sender[e], c] * Y[m, e] * R[e, m, c]
    torch.testing.assert_close(out, ref)
    Xa, Ya, Ra = (t.clone().requires_grad_(True) for t in (X, Y, R))
    (O.mp_forward(Xa, Ya, Ra, sender, receiver, N) * G).sum().backward()
    gX, gY, gR = O.mp_backward(X, Y, R, G, sender, receiver)
    torch.testing.assert_close(gX, Xa.grad)
    torch.testing.assert_close(gY, Ya.grad)
    torch.testing.assert_close(gR, Ra.grad)
    R4 = torch.randn(6, 4, C, generator=g, dtype=torch.float64)
    torch.testing.assert_close(O.mp_forward(X, Y, R4[:, O.L_OF_M, :], sender, receiver, N), O.mp_forward(X, Y, R4, sender, receiver, N))


# ---- spherical harmonics -------------------------------------------------------------------------------
def test_sh_against_scipy_closed_form():
    """sqrt(4 pi) x real harmonics built from scipy's complex ones, without Condon-Shortley sign:
    m=0: Re;  m>0: sqrt2 (-1)^m Re;  m<0: sqrt2 (-1)^m Im, on (x,y,z) = (in2, in0, in1)."""
    from scipy.special import sph_harm_y

    xyz = torch.randn(200, 3) * 3.0
    out = O.spherical_harmonics(xyz).numpy()
    v = (xyz / xyz.norm(dim=1, keepdim=True)).numpy()
    x, y, z = v[:, 2], v[:, 0], v[:, 1]
    theta, phi = np.arccos(np.clip(z, -1, 1)), np.arctan2(y, x)
    row = 0
    for l in range(4):
        for m in range(-l, l + 1):
            c = sph_harm_y(l, abs(m), theta, phi)
            if m == 0:
                val = c.real
            elif m > 0:
                val = math.sqrt(2) * (-1) ** m * c.real
            else:
                val = math.sqrt(2) * (-1) ** m * c.imag
            np.testing.assert_allclose(out[row], math.sqrt(4 * math.pi) * val, atol=1e-12)
            row += 1


def test_sh_sum_rule_and_l1():
    xyz = torch.randn(50, 3)
    Y = O.spherical_harmonics(xyz)
    for l in range(4):
        torch.testing.assert_close((Y[l * l:(l + 1) ** 2] ** 2).sum(0), torch.full((50,), 2.0 * l + 1))
    torch.testing.assert_close(Y[1:4].t(), math.sqrt(3) * xyz / xyz.norm(dim=1, keepdim=True))


def test_sh_parity_and_scale_invariance():
    xyz = torch.randn(20, 3)
    Y, Ym, Ys = O.spherical_harmonics(xyz), O.spherical_harmonics(-xyz), O.spherical_harmonics(3.7 * xyz)
    sign = torch.tensor([(-1.0) ** int(math.isqrt(m)) for m in range(16)])[:, None]
    torch.testing.assert_close(Ym, sign * Y)
    torch.testing.assert_close(Ys, Y)


def test_sh_backward_finite_differences_and_radial_null():
    xyz = torch.randn(10, 3) + 0.5
    g = torch.randn(16, 10)
    gx = O.spherical_harmonics_backward(xyz, g)
    h = 1e-6
    for k in range(3):
        d = torch.zeros(10, 3)
        d[:, k] = h
        fd = ((O.spherical_harmonics(xyz + d) - O.spherical_harmonics(xyz - d)) * g).sum(0) / (2 * h)
        torch.testing.assert_close(gx[:, k], fd, rtol=1e-6, atol=1e-7)
    # homogeneous of degree 0: the gradient has no radial component
    torch.testing.assert_close((gx * xyz).sum(1), torch.zeros(10), atol=1e-12, rtol=0)


# ---- spline ---------------------------------------------------------------------------------------------
def test_spline_against_scipy_and_boundary_conditions():
    from scipy.interpolate import CubicSpline

    knots_np, h = np.linspace(1e-12, 6.0, 256, retstep=True)
    knots = torch.from_numpy(knots_np)
    table = torch.stack([torch.sin(knots * 1.3), torch.exp(-knots), knots ** 2, torch.cos(3 * knots)], dim=1)
    co = O.spline_coefficients(knots, table)
    assert co.shape == (255, 4, 4)
    torch.testing.assert_close(co[:, 0], table[:-1])  # a_k = y_k
    torch.testing.assert_close(co[0, 2], torch.zeros(4), atol=1e-9, rtol=0)  # natural: c_0 = 0
    r = torch.rand(300) * 5.9
    val, der = O.spline_eval(r, knots, co, float(h), 5.0, deriv=True)
    cs = CubicSpline(knots_np, table.numpy(), bc_type="natural")
    inside = (r <= 5.0).numpy()
    np.testing.assert_allclose(val.numpy()[inside], cs(r.numpy())[inside], atol=1e-10)
    np.testing.assert_allclose(der.numpy()[inside], cs(r.numpy(), 1)[inside], atol=1e-9)
    assert float(val[~torch.from_numpy(inside)].abs().sum()) == 0.0
    # interpolates a smooth function to O(h^4)
    np.testing.assert_allclose(val[:, 0].numpy()[inside], np.sin(1.3 * r.numpy())[inside], atol=1e-6)
    torch.testing.assert_close(O.spline_backward(torch.ones(300, 4), der), der.sum(1))


# ---- linears ---------------------------------------------------------------------------------------------
def test_linear_loops():
    X = torch.randn(3, 16, 4)
    W = torch.randn(4, 4, 5)
    out = O.linear(X, W)
    for n in range(3):
        for m in range(16):
            l = math.isqrt(m)
            torch.testing.assert_close(out[n, m], X[n, m] @ W[l] / 2.0)
    Wel = torch.randn(3, 4, 4, 5)
    one_hot = torch.tensor([[0., 1, 0], [1, 0, 0], [0, 0, 0]])
    oe = O.elemental_linear(X, Wel, one_hot)
    torch.testing.assert_close(oe[0], O.linear(X[:1], Wel[1])[0])
    torch.testing.assert_close(oe[1], O.linear(X[1:2], Wel[0])[0])
    assert float(oe[2].abs().sum()) == 0.0


# ---- symmetric contraction ----------------------------------------------------------------------------
def test_symmetric_contraction_brute_force():
    N, C, ne = 3, 2, 2
    U3 = torch.zeros(16, 16, 16, 5)
    U2 = torch.zeros(16, 16, 3)
    rng = np.random.default_rng(0)
    for _ in range(30):
        i, j, k = rng.integers(0, 16, 3)
        U3[i, j, k, rng.integers(0, 5)] = rng.normal()
    for _ in range(10):
        i, j = rng.integers(0, 16, 2)
        U2[i, j, rng.integers(0, 3)] = rng.normal()
    X = torch.randn(N, 16, C)
    W3, W2, W1 = torch.randn(ne, 5, C), torch.randn(ne, 3, C), torch.randn(ne, 1, C)
    types = torch.tensor([1, 0, 1])
    out = O.symmetric_contraction(X, types, U3, U2, W3, W2, W1)
    ref = torch.zeros(N, C)
    nz3 = U3.nonzero().tolist()
    nz2 = U2.nonzero().tolist()
    for n in range(N):
        e = int(types[n])
        for c in range(C):
            s = W1[e, 0, c] * X[n, 0, c]
            for (i, j, k, p) in nz3:
                s += U3[i, j, k, p] * W3[e, p, c] * X[n, i, c] * X[n, j, c] * X[n, k, c]
            for (i, j, p) in nz2:
                s += U2[i, j, p] * W2[e, p, c] * X[n, i, c] * X[n, j, c]
            ref[n, c] = s
    torch.testing.assert_close(out, ref)


# ---- neighbour list ---------------------------------------------------------------------------------------
def test_neighbour_list_oracle_vs_kdtree_periodic():
    """Cubic box wider than two cutoffs: scipy's periodic cKDTree finds the same pairs; the image follows from the
    minimum-image convention."""
    from scipy.spatial import cKDTree

    rng = np.random.default_rng(0)
    box, rc = 12.0, 5.0
    pos = rng.uniform(-5.0, 20.0, (150, 3))  # atoms outside the cell too
    ei, S = O.neighbour_list(pos, np.eye(3) * box, (1, 1, 1), rc)
    pairs = cKDTree(np.mod(pos, box), boxsize=box).query_pairs(rc, output_type="ndarray")
    i = np.concatenate([pairs[:, 0], pairs[:, 1]])
    j = np.concatenate([pairs[:, 1], pairs[:, 0]])
    Sk = -np.round((pos[j] - pos[i]) / box).astype(np.int64)
    order = np.lexsort((Sk[:, 2], Sk[:, 1], Sk[:, 0], j, i))
    assert np.array_equal(ei, np.stack([i[order], j[order]]))
    assert np.array_equal(S, Sk[order])


def test_neighbour_list_oracle_vs_replicated_cluster():
    """Triclinic cell smaller than the cutoff, two periodic axes: replicate the atoms explicitly and search the
    resulting cluster without periodicity."""
    from scipy.spatial import cKDTree

    rng = np.random.default_rng(1)
    cell = np.array([[4.0, 0, 0], [1.0, 3.5, 0], [0.5, 0.7, 4.2]])
    pos = rng.uniform(-3, 8, (7, 3))
    rc, R = 5.0, 4
    ei, S = O.neighbour_list(pos, cell, (1, 1, 0), rc)
    imgs = [(a, b, 0) for a in range(-R, R + 1) for b in range(-R, R + 1)]
    allpos = np.concatenate([pos + np.array(im) @ cell for im in imgs])
    tree = cKDTree(allpos)
    rows = []
    for i in range(7):
        for k in tree.query_ball_point(pos[i], rc):
            im, j = imgs[k // 7], k % 7
            if (j == i and im == (0, 0, 0)) or not np.linalg.norm(allpos[k] - pos[i]) < rc:
                continue
            rows.append((i, j) + im)
    rows = np.array(sorted(rows))
    assert rows.shape[0] > 100
    assert np.array_equal(rows[:, :2].T, ei) and np.array_equal(rows[:, 2:], S)
    # reverse pairs carry the negated image
    fwd = {tuple(r) for r in np.concatenate([ei.T, S], axis=1)}
    assert fwd == {(j, i, -a, -b, -c) for (i, j, a, b, c) in fwd}


def test_neighbour_list_oracle_cluster_and_self_images():
    pos = np.array([[0.0, 0, 0], [1.0, 0, 0], [0, 4.0, 0], [10.0, 10, 10]])
    ei, S = O.neighbour_list(pos, None, (0, 0, 0), 4.5)
    assert ei.T.tolist() == [[0, 1], [0, 2], [1, 0], [1, 2], [2, 0], [2, 1]] and not S.any()
    # a single atom in a 3 A cubic cell with a 3.5 A cutoff sees its 6 nearest images only (next shell at 4.24 A)
    ei, S = O.neighbour_list(np.array([[0.3, 0.2, 0.1]]), np.eye(3) * 3.0, (1, 1, 1), 3.5)
    assert ei.shape[1] == 6 and sorted(map(tuple, S)) == sorted([(1, 0, 0), (-1, 0, 0), (0, 1, 0), (0, -1, 0), (0, 0, 1), (0, 0, -1)])


# ---- readouts, scale and shift --------------------------------------------------------------------
def _readout_case(seed, n=7, C=5, H=3):
    g = np.random.default_rng(seed)
    return (g.normal(size=(n, C)), g.normal(size=(n, C)), g.normal(size=C), g.normal(size=(C, H)),
            g.normal(size=H), 1.37, 0.8, -0.35)


def _readout_loops(h1, h2, w1, W2a, w2b, act, scale, shift):
    """Scalar arithmetic, one node and one hidden unit at a time: layer-1 energy is a dot product, layer-2 energy
    a sum over hidden units of weight * act * z / (1 + exp(-z)); the sum of the two is scaled, then shifted."""
    out = np.zeros(h1.shape[0])
    for n in range(h1.shape[0]):
        e = 0.0
        for c in range(h1.shape[1]):
            e += h1[n, c] * w1[c]
        for k in range(W2a.shape[1]):
            z = 0.0
            for c in range(h2.shape[1]):
                z += h2[n, c] * W2a[c, k]
            e += w2b[k] * act * z / (1.0 + math.exp(-z))
        out[n] = scale * e + shift
    return out


def test_readout_energies_explicit_loops():
    case = _readout_case(0)
    got = O.readout_energies(*(torch.from_numpy(a) if isinstance(a, np.ndarray) else a for a in case)).numpy()
    np.testing.assert_allclose(got, _readout_loops(*case), rtol=1e-13, atol=1e-14)


def test_readout_energies_special_cases():
    h1, h2, w1, W2a, w2b, act, scale, shift = _readout_case(1)
    t = torch.from_numpy
    # a dead hidden layer (silu(0) = 0) leaves the linear readout alone: scale * h1.w1 + shift
    got = O.readout_energies(t(h1), t(h2), t(w1), t(np.zeros_like(W2a)), t(w2b), act, scale, shift).numpy()
    np.testing.assert_allclose(got, scale * (h1 @ w1) + shift, rtol=1e-13)
    # no layer-1 features, one hidden unit: a scalar chain per node
    W1u, w2u = W2a[:, :1], w2b[:1]
    got = O.readout_energies(t(np.zeros_like(h1)), t(h2), t(w1), t(W1u), t(w2u), act, scale, shift).numpy()
    for n in range(h2.shape[0]):
        z = float(h2[n] @ W1u[:, 0])
        assert abs(got[n] - (scale * w2u[0] * act * z / (1 + math.exp(-z)) + shift)) < 1e-13
    # the shift is added after the scale, not scaled with it; the scale multiplies both readouts
    a = O.readout_energies(t(h1), t(h2), t(w1), t(W2a), t(w2b), act, 1.0, 0.0).numpy()
    b = O.readout_energies(t(h1), t(h2), t(w1), t(W2a), t(w2b), act, 3.0, 0.5).numpy()
    np.testing.assert_allclose(b, 3.0 * a + 0.5, rtol=1e-13)
    # large pre-activations: the gate is the identity times act for z >> 0 and 0 for z << 0
    big = O.readout_energies(t(np.zeros((2, 1))), t(np.array([[40.0], [-40.0]])), t(np.zeros(1)), t(np.ones((1, 1))),
                             t(np.ones(1)), act, 1.0, 0.0).numpy()
    np.testing.assert_allclose(big, [act * 40.0, 0.0], rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("which", ["act", "scale", "shift_scaled", "w2b", "w1"])
def test_readout_pin_has_teeth(which):
    """A 1 % error in the activation constant, the scale, either weight fold, or a shift that is scaled with the sum
    moves the loop value by far more than the tolerance of the comparison above."""
    h1, h2, w1, W2a, w2b, act, scale, shift = _readout_case(2)
    ref = _readout_loops(h1, h2, w1, W2a, w2b, act, scale, shift)
    if which == "act":
        bad = _readout_loops(h1, h2, w1, W2a, w2b, act * 1.01, scale, shift)
    elif which == "scale":
        bad = _readout_loops(h1, h2, w1, W2a, w2b, act, scale * 1.01, shift)
    elif which == "shift_scaled":
        bad = _readout_loops(h1, h2, w1, W2a, w2b, act, scale, shift * scale)
    elif which == "w2b":
        bad = _readout_loops(h1, h2, w1, W2a, w2b * 1.01, act, scale, shift)
    else:
        bad = _readout_loops(h1, h2, w1 * 1.01, W2a, w2b, act, scale, shift)
    assert np.abs(bad - ref).max() > 1e-4
