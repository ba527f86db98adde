"""Host-side logic of the package checked on the CPU against the oracle: spline coefficients, coupling tensors,
the packed sparse tables and their regrouping into monomials."""
import numpy as np
import pytest
import torch

from oracle import ops as O
from oracle.u_tensors import u_tensors


def test_spline_coefficients_match_scipy():
    from cuda_mace.ops.cubic_spline import CubicSpline

    knots_np, h = np.linspace(1e-12, 6.0, 256, retstep=True)
    knots = torch.from_numpy(knots_np)
    table = torch.stack([torch.sin(knots * 2.1), torch.exp(-0.5 * knots) * knots, torch.cos(knots) ** 2], dim=1)
    mine = CubicSpline.cubic_spline_coefficients(knots, table, float(h))
    ref = O.spline_coefficients(knots, table)
    torch.testing.assert_close(mine, ref, rtol=1e-9, atol=1e-9)


def test_coupling_tensors_two_derivations_agree():
    from cuda_mace.ops.u_matrix import U_matrix_real, coupling_paths

    U1, U2, U3 = u_tensors()
    assert len(coupling_paths(3)) == 23
    for nu, ref in ((1, U1), (2, U2), (3, U3)):
        mine = U_matrix_real(correlation=nu, dtype=torch.float64)[-1].numpy()
        np.testing.assert_allclose(mine, ref, atol=1e-12)
    # unit Frobenius norm per path, one path per non-zero (i, j, k), known sparsity
    np.testing.assert_allclose((U3 ** 2).sum((0, 1, 2)), np.ones(23), atol=1e-12)
    assert int((U3 != 0).sum(-1).max()) == 1 and int((U3 != 0).sum()) == 353


def test_coupling_tensors_are_rotation_invariant():
    """U3 contracted with three copies of the harmonics' rotation matrix is unchanged; the rotation matrix in the
    16-dimensional component basis is fitted from function values."""
    from cuda_mace.ops.u_matrix import U_matrix_real

    rng = np.random.default_rng(0)
    q, r = np.linalg.qr(rng.normal(size=(3, 3)))
    q = q * np.sign(np.diag(r))
    v = torch.from_numpy(rng.normal(size=(400, 3)))
    Y = O.spherical_harmonics(v).numpy()  # [16, P]
    Yr = O.spherical_harmonics(v @ torch.from_numpy(q).t()).numpy()
    D = Yr @ np.linalg.pinv(Y)  # Y(Rv) = D Y(v)
    np.testing.assert_allclose(D @ D.T, np.eye(16), atol=1e-9)
    U3 = U_matrix_real(correlation=3, dtype=torch.float64)[-1].numpy()
    rot = np.einsum("ai,bj,ck,ijkp->abcp", D, D, D, U3)
    np.testing.assert_allclose(rot, U3, atol=1e-9)


def _fake_contraction(ne=3, C=32, seed=0):
    from cuda_mace.models.upstream_like import _SymmetricContraction

    return _SymmetricContraction(C, ne, torch.Generator().manual_seed(seed))


def test_packed_tables_round_trip_and_monomials():
    from cuda_mace.ops._autograd import monomials_from_packed
    from cuda_mace.ops.symmetric_contraction import SymmetricContraction

    sc = SymmetricContraction(_fake_contraction(), device="cpu")
    U1, U2, U3 = u_tensors()
    U3d, U2d = O.unpack_u_tables(sc.U3_num_nonsparse, sc.U3_indices, sc.U3_values, sc.U2_num_nonsparse, sc.U2_indices,
                                 sc.U2_values, 23, 4)
    np.testing.assert_allclose(U3d.numpy(), U3.astype(np.float32), atol=0)
    np.testing.assert_allclose(U2d.numpy(), U2.astype(np.float32), atol=0)
    assert sc.u3_max_nonsparse == 3 and sc.weights_3.shape == (1, 3, 23, 32)
    # the derivative path indices in the packed word name the paths of the permuted index triples
    word = int(sc.U3_indices[0, 1, 5])
    k = (word >> 8) & 0xFF
    assert U3[5, 1, k, (word >> 24) & 0xFF] != 0 and U3[5, k, 1, (word >> 16) & 0xFF] != 0

    (m3, o3, p3, v3), (m2, o2, p2, v2) = monomials_from_packed(sc.U3_num_nonsparse, sc.U3_indices, sc.U3_values,
                                                               sc.U2_num_nonsparse, sc.U2_indices, sc.U2_values)
    assert m3.shape[0] == 77 and m2.shape[0] == 16 and o3[-1] <= 353  # entries sharing a path are merged
    # evaluating the monomial form on the CPU reproduces the dense contraction
    g = torch.Generator().manual_seed(1)
    X = torch.randn(5, 16, 32, generator=g, dtype=torch.float64)
    types = torch.tensor([0, 2, 1, 1, 0])
    W3, W2, W1 = (w[0].double() for w in (sc.weights_3, sc.weights_2, sc.weights_1))
    ref = O.symmetric_contraction(X, types, U3d, U2d, W3, W2, W1)
    out = W1[types][:, 0] * X[:, 0]
    for t in range(77):
        i, j, k = m3[t] & 255, (m3[t] >> 8) & 255, (m3[t] >> 16) & 255
        coef = sum(float(v3[q]) * W3[types][:, int(p3[q])] for q in range(o3[t], o3[t + 1]))
        out = out + coef * X[:, i] * X[:, j] * X[:, k]
    for t in range(16):
        i, j = m2[t] & 255, (m2[t] >> 8) & 255
        coef = sum(float(v2[q]) * W2[types][:, int(p2[q])] for q in range(o2[t], o2[t + 1]))
        out = out + coef * X[:, i] * X[:, j]
    torch.testing.assert_close(out, ref, rtol=1e-6, atol=1e-6)  # merged fp32 table values round once more


def test_linear_weight_layout():
    from cuda_mace.models.InvariantMACE import element_linear_to_cuda
    from cuda_mace.models.upstream_like import _LinearPerL, _SkipTP
    from cuda_mace.ops.linear import Linear

    g = torch.Generator().manual_seed(0)
    lin = _LinearPerL(32, g)
    mod = Linear(lin)
    assert mod.weights.shape == (4, 32, 32)
    torch.testing.assert_close(mod.weights.double(), lin.weight.detach().view(4, 32, 32), rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(mod.weights_transposed, mod.weights.transpose(-1, -2))
    tp = _SkipTP(32, 5, 3, g)
    el = element_linear_to_cuda(tp)
    assert el.weights.shape == (5, 4, 32, 32)
    W = tp.weight.detach().view(4, 32, 5, 32)
    torch.testing.assert_close(el.weights[3, 2].double(), W[2, :, 3, :] / 5 ** 0.5, rtol=1e-6, atol=1e-6)


def test_model_constructs_on_cpu_and_refuses_to_run_there():
    from cuda_mace.models import OptimizedInvariantMACE, SyntheticInvariantMACE
    from cuda_mace.utils.synthetic import make_system

    model = OptimizedInvariantMACE(SyntheticInvariantMACE(channels=32, seed=0), device="cpu")
    data = make_system(10, 4, seed=0, density=None, cluster_box=6.0)
    with pytest.raises(RuntimeError, match="GPU"):
        model(data)


def test_contraction_tables_follow_the_coupling_basis_of_the_source_module():
    """A contraction module that carries its own coupling tensors (upstream's `U_matrix_1/2/3` buffers) is packed in
    that basis: with a permuted, sign-flipped path basis the packed tables unpack to exactly those tensors and the
    monomial form reproduces the dense contraction evaluated with them -- and differs from the result in the
    package's own basis, which the same weights would give if the buffers were ignored."""
    from cuda_mace.models.upstream_like import _SymmetricContraction, permuted_coupling_basis
    from cuda_mace.ops._autograd import monomials_from_packed
    from cuda_mace.ops.symmetric_contraction import SymmetricContraction

    basis = permuted_coupling_basis(7)
    own = _SymmetricContraction(32, 3, torch.Generator().manual_seed(0))
    up = _SymmetricContraction(32, 3, torch.Generator().manual_seed(0), coupling=basis)
    assert hasattr(up.contractions[0], "U_matrix_3") and not hasattr(own.contractions[0], "U_matrix_3")
    sc, sc_own = SymmetricContraction(up, device="cpu"), SymmetricContraction(own, device="cpu")
    U3d, U2d = O.unpack_u_tables(sc.U3_num_nonsparse, sc.U3_indices, sc.U3_values, sc.U2_num_nonsparse, sc.U2_indices,
                                 sc.U2_values, 23, 4)
    np.testing.assert_allclose(U3d.numpy(), basis[2].numpy().astype(np.float32), atol=0)
    np.testing.assert_allclose(U2d.numpy(), basis[1].numpy().astype(np.float32), atol=0)
    assert not torch.equal(sc.U3_indices, sc_own.U3_indices)

    g = torch.Generator().manual_seed(1)
    X = torch.randn(6, 16, 32, generator=g, dtype=torch.float64)
    types = torch.tensor([0, 2, 1, 1, 0, 2])
    W3, W2, W1 = (w[0].double() for w in (sc.weights_3, sc.weights_2, sc.weights_1))
    ref = O.symmetric_contraction(X, types, basis[2], basis[1], W3, W2, W1)
    U1, U2, U3 = u_tensors()
    other = O.symmetric_contraction(X, types, torch.from_numpy(U3), torch.from_numpy(U2), W3, W2, W1)
    assert float((ref - other).abs().max()) > 1e-2

    def monomial_form(mod):
        (m3, o3, p3, v3), (m2, o2, p2, v2) = monomials_from_packed(mod.U3_num_nonsparse, mod.U3_indices, mod.U3_values,
                                                                   mod.U2_num_nonsparse, mod.U2_indices, mod.U2_values)
        out = W1[types][:, 0] * X[:, 0]
        for t in range(len(m3)):
            i, j, k = m3[t] & 255, (m3[t] >> 8) & 255, (m3[t] >> 16) & 255
            out = out + sum(float(v3[q]) * W3[types][:, int(p3[q])] for q in range(o3[t], o3[t + 1])) * X[:, i] * X[:, j] * X[:, k]
        for t in range(len(m2)):
            i, j = m2[t] & 255, (m2[t] >> 8) & 255
            out = out + sum(float(v2[q]) * W2[types][:, int(p2[q])] for q in range(o2[t], o2[t + 1])) * X[:, i] * X[:, j]
        return out

    torch.testing.assert_close(monomial_form(sc), ref, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(monomial_form(sc_own), other, rtol=1e-6, atol=1e-6)


def test_coupling_tensor_checks():
    from cuda_mace.models.upstream_like import _SymmetricContraction, permuted_coupling_basis
    from cuda_mace.ops.symmetric_contraction import SymmetricContraction, check_coupling_tensor, coupling_tensors_of

    U1, U2, U3 = permuted_coupling_basis(0)
    for nu, U, paths in ((1, U1, 1), (2, U2, 4), (3, U3, 23)):
        check_coupling_tensor(U, nu, paths)
    with pytest.raises(ValueError, match="unit Frobenius norm"):
        check_coupling_tensor(U3 * 1.01, 3, 23)
    with pytest.raises(ValueError, match="paths, the weights have"):
        check_coupling_tensor(U3[..., :22], 3, 23)
    two = U3.clone()
    two[..., 1] = two[..., 0]
    with pytest.raises(ValueError, match="several paths"):
        check_coupling_tensor(two, 3, 23)
    with pytest.raises(ValueError, match="order 1"):
        check_coupling_tensor(-U1, 1, 1)
    with pytest.raises(ValueError, match="shape"):
        check_coupling_tensor(U3[:9], 3, 23)
    # a leading axis of length one and rounding residue of a basis change are accepted when read from a module
    up = _SymmetricContraction(32, 2, torch.Generator().manual_seed(0), coupling=(U1, U2, U3))
    con = up.contractions[0]
    con.U_matrix_3 = (U3 + 1e-17)[None]
    got = coupling_tensors_of(up)
    assert torch.equal(got[3] != 0, U3 != 0) and torch.allclose(got[3], U3, atol=1e-15, rtol=0) and torch.equal(got[2], U2)
    del con.U_matrix_2
    with pytest.raises(ValueError, match="orders"):
        SymmetricContraction(up, device="cpu")


def test_per_model_cache_survives_a_recycled_token_id():
    """Entries kept on a tensor per model are keyed on the model's token object, weakly: when a model dies its entry
    goes with it, so a new model whose token lands on the same address (same id) never sees the old value; two live
    models keep one entry each; a pickle or a copy of the tensor starts without entries."""
    import copy
    import gc
    import io

    from cuda_mace.models.InvariantMACE import _WeightsToken
    from cuda_mace.ops._autograd import _cached_per

    owner, other = torch.arange(5), torch.zeros(3)
    builds = []

    def build_for(name):
        def build():
            builds.append(name)
            return name
        return build

    seen_ids, recycled = set(), False
    for round_ in range(200):  # CPython hands a freed object's address to the next object of that size
        tok = _WeightsToken()
        recycled |= id(tok) in seen_ids
        seen_ids.add(id(tok))
        name = "model %d" % round_
        assert _cached_per(owner, "_slot", tok, other, build_for(name)) == name
        assert _cached_per(owner, "_slot", tok, other, build_for("never built")) == name  # a hit while the model lives
        del tok
        gc.collect()
        assert len(owner.__dict__["_slot"]) == 0
    assert recycled and len(builds) == 200
    a, b = _WeightsToken(), _WeightsToken()
    assert _cached_per(owner, "_slot", a, other, build_for("A")) == "A"
    assert _cached_per(owner, "_slot", b, other, build_for("B")) == "B"
    assert _cached_per(owner, "_slot", a, other, build_for("A2")) == "A"  # B did not evict A
    other.add_(1)  # the tensor the value was derived from changed in place
    assert _cached_per(owner, "_slot", a, other, build_for("A3")) == "A3"
    buf = io.BytesIO()
    torch.save(owner, buf)
    buf.seek(0)
    loaded = torch.load(buf, weights_only=False)
    assert torch.equal(loaded, owner) and len(loaded.__dict__.get("_slot", {})) == 0
    assert len(copy.deepcopy(owner).__dict__["_slot"]) == 0
