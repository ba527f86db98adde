"""The fp64 instantiations of message passing, spherical harmonics, cubic spline and symmetric contraction (the ops the
reference dispatches on float and double) against the fp64 CPU oracle on the same seeded inputs, through the C ABI and
through the op modules' autograd, including torch.autograd.gradcheck on the double path.

Tolerance: both sides compute in double, only the order of the sums differs: relative 1e-12 with an absolute floor of
1e-13 of the largest expected magnitude.
"""
import numpy as np
import pytest
import torch

from oracle import ops as O
from oracle.u_tensors import u_tensors
from tests.util import close, mp_inputs, random_graph

pytestmark = pytest.mark.gpu

RTOL = 1e-12
ATOL = 1e-13
DEV = "cuda"
F64 = torch.float64


def _say(*a):
    print(*a, flush=True)


MP_CASES = [
    # nnodes, avg degree, channels, degree mode, isolated fraction, seed
    (64, 8, 32, "poisson", 0.2, 0),
    (200, 30, 64, "poisson", 0.0, 1),
    (150, 30, 96, "fixed", 0.0, 2),
    (300, 52, 128, "poisson", 0.05, 3),
    (60, 20, 160, "poisson", 0.1, 5),
    (50, 40, 192, "poisson", 0.0, 6),
    (40, 25, 256, "poisson", 0.3, 8),
    (3, 1, 128, "fixed", 0.0, 9),
]


def _mp_case(nnodes, avg, C, mode, iso, seed):
    snd, rcv = random_graph(nnodes, avg, seed, degree_mode=mode, isolated_frac=iso)
    E = snd.numel()
    X, v, R, G = mp_inputs(nnodes, E, C, seed)
    Y = O.spherical_harmonics(v) if E else torch.zeros(16, 0, dtype=F64)
    return snd, rcv, X, Y.contiguous(), R, G


@pytest.mark.parametrize("case", MP_CASES, ids=lambda c: "N%d_d%d_C%d_%s_s%d" % (c[0], c[1], c[2], c[3], c[5]))
def test_mp_f64(cabi, case):
    _say("mp f64", case)
    nnodes = case[0]
    snd, rcv, X, Y, R, G = _mp_case(*case)
    ref = O.mp_forward(X, Y, R, snd, rcv, nnodes)
    gX_ref, gY_ref, gR_ref = O.mp_backward(X, Y, R, G, snd, rcv)
    d = lambda t: t.to(DEV)
    fo = cabi.first_occurences(d(rcv), nnodes)
    perm, off = cabi.stable_key_sort(d(snd), nnodes)
    out = cabi.mp_forward(d(X), d(Y), d(R), d(snd), fo, nnodes)
    assert out.dtype == F64
    close(out, ref, RTOL, ATOL)
    gX, gY, gR = cabi.mp_backward(d(X), d(Y), d(R), d(G), d(snd), fo, perm, off, nnodes)
    close(gR, gR_ref, RTOL, ATOL)
    close(gY, gY_ref, RTOL, ATOL)
    close(gX, gX_ref, RTOL, ATOL)
    # subsets of the gradients equal the full computation bit for bit; repeats are bit-identical
    for mask in range(1, 7):
        need = dict(need_gX=bool(mask & 1), need_gY=bool(mask & 2), need_gR=bool(mask & 4))
        part = cabi.mp_backward(d(X), d(Y), d(R), d(G), d(snd), fo, perm, off, nnodes, **need)
        for got, want, on in zip(part, (gX, gY, gR), (need["need_gX"], need["need_gY"], need["need_gR"])):
            assert (got is None) if not on else torch.equal(got, want)
    assert torch.equal(out, cabi.mp_forward(d(X), d(Y), d(R), d(snd), fo, nnodes))


def test_mp_f64_agrees_with_f32(cabi):
    """The two precisions of the same op differ by fp32 rounding only."""
    case = (120, 30, 128, "poisson", 0.0, 11)
    nnodes = case[0]
    snd, rcv, X, Y, R, _ = _mp_case(*case)
    d = lambda t: t.to(DEV)
    fo = cabi.first_occurences(d(rcv), nnodes)
    hi = cabi.mp_forward(d(X), d(Y), d(R), d(snd), fo, nnodes)
    lo = cabi.mp_forward(d(X).float(), d(Y).float(), d(R).float(), d(snd), fo, nnodes)
    assert lo.dtype == torch.float32
    close(lo, hi.cpu(), 2e-5, 2e-6)


def test_mixed_precision_is_rejected(cabi):
    X = torch.zeros(4, 32, device=DEV, dtype=F64)
    Y = torch.zeros(16, 0, device=DEV)  # fp32 next to an fp64 X
    R = torch.zeros(0, 4, 32, device=DEV, dtype=F64)
    snd = torch.zeros(0, dtype=torch.int32, device=DEV)
    fo = torch.zeros(8, dtype=torch.int32, device=DEV)
    with pytest.raises(RuntimeError, match="float64"):
        cabi.mp_forward(X, Y, R, snd, fo, 4)


@pytest.mark.parametrize("E,seed", [(1, 0), (1000, 1), (100003, 2)])
def test_sh_f64(cabi, E, seed):
    _say("sh f64", E, seed)
    g = torch.Generator().manual_seed(seed)
    xyz = torch.randn(E, 3, generator=g, dtype=F64) * 2.5
    gY = torch.randn(16, E, generator=g, dtype=F64)
    Y = cabi.sh_forward(xyz.to(DEV))
    gx = cabi.sh_backward(xyz.to(DEV), gY.to(DEV))
    assert Y.dtype == F64 and gx.dtype == F64
    close(Y, O.spherical_harmonics(xyz), RTOL, ATOL)
    # the projected gradient cancels large terms for short vectors: floor relative to the largest entry
    close(gx, O.spherical_harmonics_backward(xyz, gY), 1e-10, 1e-13)


@pytest.mark.parametrize("E,J,seed", [(1, 128, 0), (777, 384, 1), (300, 30, 2)])
def test_spline_f64(cabi, E, J, seed):
    _say("spline f64", E, J, seed)
    g = torch.Generator().manual_seed(seed)
    r_max = 5.0
    knots_np, h = np.linspace(1e-12, r_max + 1.0, 256, retstep=True)
    knots = torch.from_numpy(knots_np)
    table = torch.sin(knots[:, None] * torch.linspace(0.3, 3.0, J, dtype=F64)[None, :]) * torch.randn(1, J, generator=g, dtype=F64)
    coeffs = O.spline_coefficients(knots, table)
    r = torch.rand(E, generator=g, dtype=F64) * 5.6 + 0.4  # some beyond r_max
    gR = torch.randn(E, J, generator=g, dtype=F64)
    val_ref, der_ref = O.spline_eval(r, knots, coeffs, float(h), r_max, deriv=True)
    gr_ref = O.spline_backward(gR, der_ref)
    d = lambda t: t.to(DEV)
    val, der = cabi.spline_forward(d(r), d(knots), d(coeffs), float(h), r_max, want_deriv=True)
    val_only = cabi.spline_forward(d(r), d(knots), d(coeffs), float(h), r_max)
    gr = cabi.spline_backward(d(r), d(knots), d(coeffs), d(gR), float(h), r_max)
    assert val.dtype == F64 and torch.equal(val, val_only)
    close(val, val_ref, RTOL, ATOL)
    close(der, der_ref, RTOL, ATOL)
    bound = 1e-14 * (gR.abs() * der_ref.abs()).sum(-1) + 1e-300
    assert bool(((gr.cpu() - gr_ref).abs() <= bound).all())
    assert float(val[(r > r_max).to(DEV)].abs().sum()) == 0.0


def _symcon_module(ne, C, seed):
    from cuda_mace.models.upstream_like import _SymmetricContraction
    from cuda_mace.ops.symmetric_contraction import SymmetricContraction

    up = _SymmetricContraction(C, ne, torch.Generator().manual_seed(seed))
    return up, SymmetricContraction(up, device=DEV, dtype=F64)


@pytest.mark.parametrize("N,C,ne,seed", [(1, 32, 1, 0), (100, 128, 10, 1), (40, 96, 4, 2), (9, 256, 2, 3)])
def test_symmetric_contraction_f64(cabi, N, C, ne, seed):
    """Op module in double (weights in double, U values as the module stores them) against the dense oracle with
    independently derived U tensors; then the table-driven kernel against the unrolled one."""
    _say("symcon f64", N, C, ne, seed)
    up, mod = _symcon_module(ne, C, seed)
    assert mod.weights_3.dtype == F64
    con = up.contractions[0]
    U1, U2, U3 = (torch.from_numpy(u) for u in u_tensors())
    g = torch.Generator().manual_seed(seed)
    X = torch.randn(N, 16, C, generator=g, dtype=F64)
    types = torch.randint(0, ne, (N,), generator=g).int()
    gout = torch.randn(N, C, generator=g, dtype=F64)
    Xa = X.clone().requires_grad_(True)
    W3, W2, W1 = (w.detach().float().double() for w in (con.weights_max, con.weights[0], con.weights[1]))
    ref = O.symmetric_contraction(Xa, types, U3, U2, W3, W2, W1)
    (ref * gout).sum().backward()
    Xg = X.to(DEV).requires_grad_(True)
    out = mod(Xg, types.to(DEV))
    assert out.shape == (N, 1, C) and out.dtype == F64
    (out.squeeze(1) * gout.to(DEV)).sum().backward()
    # the module keeps the coupling values in fp32 (as the reference does): that rounding bounds the agreement
    close(out.squeeze(1).detach(), ref.detach(), 1e-6, 1e-7)
    close(Xg.grad, Xa.grad, 1e-6, 1e-7)

    from cuda_mace.ops import _autograd as A

    (m3, o3, p3, v3), (m2, o2, p2, v2) = A.monomials_from_packed(mod.U3_num_nonsparse, mod.U3_indices, mod.U3_values,
                                                                 mod.U2_num_nonsparse, mod.U2_indices, mod.U2_values)
    t = lambda a: torch.from_numpy(a).to(DEV)
    tv = lambda a: torch.from_numpy(a).double().to(DEV)
    T3, T2, T1 = cabi.symcon_tables(t(o3), t(p3), tv(v3), t(o2), t(p2), tv(v2), mod.weights_3[0], mod.weights_2[0], mod.weights_1[0])
    assert T3.dtype == F64
    perm, off = cabi.stable_key_sort(types.to(DEV), ne)
    xa = X.to(DEV)
    out_b, grad_b = cabi.symcon_forward(xa, perm, off, t(m3), t(m2), T3, T2, T1, builtin=True)
    out_t, grad_t = cabi.symcon_forward(xa, perm, off, t(m3), t(m2), T3, T2, T1, builtin=False)
    # (monomials_from_packed rounds the per-monomial sums of coupling values to fp32; the module's own path keeps them in double)
    close(out_b, out.squeeze(1).detach().cpu(), 1e-6, 1e-7)
    close(out_t, out_b.cpu(), RTOL, ATOL)
    close(grad_t, grad_b.cpu(), RTOL, ATOL)
    gX = cabi.symcon_backward(grad_b, gout.to(DEV))
    close(gX, Xg.grad.cpu(), 1e-6, 1e-7)


def test_gradcheck_double_path(cabi):
    """Numerical differentiation of the double path of every op module (first derivatives, as the reference supports)."""
    from cuda_mace.ops import CubicSpline, InvariantMessagePassingTP
    from cuda_mace.ops.spherical_harmonics import SphericalHarmonics

    g = torch.Generator().manual_seed(5)
    nnodes, C = 6, 32
    snd, rcv = random_graph(nnodes, 3, 5, degree_mode="fixed")
    E = snd.numel()
    X, v, R, _ = mp_inputs(nnodes, E, C, 5)
    Y = O.spherical_harmonics(v).contiguous()
    leaf = lambda t: t.to(DEV).requires_grad_(True)
    tp = InvariantMessagePassingTP()
    s_dev, r_dev = snd.to(DEV), rcv.to(DEV)
    assert torch.autograd.gradcheck(lambda x, y, r: tp(x, y, r, s_dev, r_dev, nnodes), (leaf(X), leaf(Y), leaf(R)),
                                    eps=1e-6, atol=1e-7, rtol=1e-6, nondet_tol=0.0)

    sh = SphericalHarmonics()
    xyz = torch.randn(7, 3, generator=g, dtype=F64) * 2.0
    assert torch.autograd.gradcheck(sh, (leaf(xyz),), eps=1e-6, atol=1e-7, rtol=1e-6, nondet_tol=0.0)

    knots_np, h = np.linspace(1e-12, 6.0, 64, retstep=True)
    knots = torch.from_numpy(knots_np)
    table = torch.cos(knots[:, None] * torch.linspace(0.2, 2.0, 8, dtype=F64)[None, :])
    spline = CubicSpline(knots, table, float(h), 5.0).to(DEV)
    assert spline.coefficients.dtype == F64
    # radii away from the knots (the third derivative jumps there) and inside r_max
    r = (torch.arange(9, dtype=F64) + 0.37) * float(h) * 5.0
    assert torch.autograd.gradcheck(spline, (leaf(r),), eps=1e-6, atol=1e-7, rtol=1e-6, nondet_tol=0.0)

    _, mod = _symcon_module(2, 32, 7)
    types = torch.tensor([0, 1, 1], dtype=torch.int32, device=DEV)
    x = torch.randn(3, 16, 32, generator=g, dtype=F64) * 0.7
    assert torch.autograd.gradcheck(lambda a: mod(a, types), (leaf(x),), eps=1e-6, atol=1e-6, rtol=1e-6, nondet_tol=0.0)
