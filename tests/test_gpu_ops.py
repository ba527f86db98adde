"""GPU parity of every C-ABI entry point against the fp64 CPU oracle on the same seeded inputs.

Tolerances (fp32 kernels vs fp64 oracle): relative 2e-5 with an absolute floor of 2e-6 of the
largest expected magnitude for sums of O(50) N(0,1) products; index kernels must be bit-exact.
"""
import math

import numpy as np
import pytest
import torch

from oracle import ops as O
from tests.util import close, mp_inputs, random_graph

pytestmark = pytest.mark.gpu

RTOL = 2e-5
ATOL = 2e-6
DEV = "cuda"


def _say(*a):
    print(*a, flush=True)


# ------------------------------------------------------------------------------------------------
# index kernels: bit-exact
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize(
    "nnodes,avg,iso,seed",
    [(1, 1, 0.0, 0), (7, 3, 0.5, 1), (1000, 30, 0.0, 2), (4097, 5, 0.3, 3), (300, 700, 0.1, 4), (50, 0, 0.0, 5)],
)
def test_first_occurences_exact(cabi, nnodes, avg, iso, seed):
    _say("first_occurences", nnodes, avg, iso, seed)
    _, recv = random_graph(nnodes, avg, seed, isolated_frac=iso)
    ref = O.first_occurences(recv, nnodes)
    got = cabi.first_occurences(recv.to(DEV), nnodes).cpu()
    assert torch.equal(got, ref)


@pytest.mark.parametrize("n,nkeys,seed", [(0, 5, 0), (1, 1, 1), (1000, 10, 2), (122880, 4096, 3), (5000, 1, 4), (3000, 10000, 5),
                                          # few keys, large buckets (atoms grouped by element): the workgroup-histogram route
                                          (100000, 1, 6), (100000, 11, 7), (200003, 64, 8), (4096, 3, 9), (4095, 3, 10),
                                          (70000, 65, 11)])
def test_stable_key_sort_exact(cabi, n, nkeys, seed):
    _say("stable_key_sort", n, nkeys, seed)
    keys = torch.from_numpy(np.random.default_rng(seed).integers(0, nkeys, n).astype(np.int32))
    perm_ref, off_ref = O.stable_key_sort(keys, nkeys)
    perm, off = cabi.stable_key_sort(keys.to(DEV), nkeys)
    assert torch.equal(off.cpu(), off_ref)
    assert torch.equal(perm.cpu(), perm_ref)


def test_stable_key_sort_skips_keys_out_of_range(cabi):
    """Items whose key lies outside [0, nkeys) are left out on both routes (that is where atoms whose one-hot row names
    no element go): offsets[nkeys] counts the items placed."""
    for n, nkeys in ((1000, 10), (50000, 10)):
        rng = np.random.default_rng(n)
        keys = rng.integers(-2, nkeys + 2, n).astype(np.int32)
        perm, off = cabi.stable_key_sort(torch.from_numpy(keys).to(DEV), nkeys)
        valid = np.flatnonzero((keys >= 0) & (keys < nkeys))
        order = valid[np.argsort(keys[valid], kind="stable")]
        total = int(off[-1])
        assert total == valid.size
        assert np.array_equal(perm.cpu().numpy()[:total], order.astype(np.int32))
        assert np.array_equal(off.cpu().numpy(), np.searchsorted(keys[order], np.arange(nkeys + 1)).astype(np.int32))


def test_receiver_list_status(cabi):
    """The check of what the CSR kernel assumes of its input: sorted, values in range."""
    good = torch.tensor([0, 0, 1, 3, 3, 7], dtype=torch.int32, device=DEV)
    assert cabi.receiver_list_status(good, 8) == (False, False)
    assert cabi.receiver_list_status(good, 7) == (False, True)
    bad = torch.tensor([0, 2, 1, 3], dtype=torch.int32, device=DEV)
    assert cabi.receiver_list_status(bad, 4) == (True, False)
    assert cabi.receiver_list_status(torch.tensor([5, -1], dtype=torch.int32, device=DEV), 4) == (True, True)
    assert cabi.receiver_list_status(torch.zeros(0, dtype=torch.int32, device=DEV), 4) == (False, False)
    big = torch.arange(300000, dtype=torch.int32, device=DEV) // 7
    assert cabi.receiver_list_status(big, 300000 // 7 + 1) == (False, False)
    big[123456] = 0
    assert cabi.receiver_list_status(big, 300000 // 7 + 1) == (True, False)
    # with the debug switch on, the binding refuses such a list instead of computing offsets from it
    old = cabi.DEBUG
    cabi.DEBUG = True
    try:
        with pytest.raises(cabi.CudaMaceError, match="non-decreasing"):
            cabi.first_occurences(bad, 4)
        assert torch.equal(cabi.first_occurences(good, 8).cpu(), O.first_occurences(good.cpu(), 8))
    finally:
        cabi.DEBUG = old


# ------------------------------------------------------------------------------------------------
# message passing
# ------------------------------------------------------------------------------------------------
MP_CASES = [
    # nnodes, avg degree, channels, degree mode, isolated fraction, seed
    (64, 8, 32, "poisson", 0.2, 0),
    (200, 30, 64, "poisson", 0.0, 1),
    (512, 30, 96, "fixed", 0.0, 2),
    (300, 52, 128, "poisson", 0.05, 3),
    (40, 150, 128, "poisson", 0.0, 4),  # segments longer than one 64-edge chunk
    (100, 20, 160, "poisson", 0.1, 5),
    (150, 40, 192, "poisson", 0.0, 6),
    (60, 10, 224, "poisson", 0.0, 7),
    (80, 25, 256, "poisson", 0.3, 8),
    (3, 1, 128, "fixed", 0.0, 9),
    (4096, 30, 96, "fixed", 0.0, 0),  # benchmark configuration 2 at its real size: 122 880 edges, uniform random senders
]


def _mp_case(nnodes, avg, C, mode, iso, seed):
    snd, rcv = random_graph(nnodes, avg, seed, degree_mode=mode, isolated_frac=iso)
    E = snd.numel()
    X, v, R, G = mp_inputs(nnodes, E, C, seed)
    Y = O.spherical_harmonics(v) if E else torch.zeros(16, 0, dtype=torch.float64)
    return snd, rcv, X, Y.contiguous(), R, G


@pytest.mark.parametrize("case", MP_CASES, ids=lambda c: "N%d_d%d_C%d_%s_s%d" % (c[0], c[1], c[2], c[3], c[5]))
def test_mp_forward(cabi, case):
    _say("mp_forward", case)
    nnodes = case[0]
    snd, rcv, X, Y, R, _ = _mp_case(*case)
    ref = O.mp_forward(X, Y, R, snd, rcv, nnodes)
    fo = cabi.first_occurences(rcv.to(DEV), nnodes)
    out = cabi.mp_forward(X.float().to(DEV), Y.float().to(DEV), R.float().to(DEV), snd.to(DEV), fo, nnodes)
    close(out, ref, RTOL, ATOL)


@pytest.mark.parametrize("C", [64, 96, 128, 160, 224])
def test_mp_forward_every_edge_count(cabi, C):
    """Node i receives i edges, i = 0 .. 140: the forward takes a slot's edges in blocks of eight, four, two and one (which
    of them depends on the channels per lane), so every remainder of every block size occurs, in one chunk of 64 staged
    edges and across chunks; per-component weights take two edges at a time."""
    import numpy as np

    _say("mp_forward every edge count", C)
    nnodes = 141
    rng = np.random.default_rng(C)
    rcv = torch.from_numpy(np.repeat(np.arange(nnodes), np.arange(nnodes)).astype(np.int32))
    E = rcv.numel()
    snd = torch.from_numpy(rng.integers(0, nnodes, E).astype(np.int32))
    X, v, R, _ = mp_inputs(nnodes, E, C, C)
    Y = O.spherical_harmonics(v).contiguous()
    fo = cabi.first_occurences(rcv.to(DEV), nnodes)
    out = cabi.mp_forward(X.float().to(DEV), Y.float().to(DEV), R.float().to(DEV), snd.to(DEV), fo, nnodes)
    close(out, O.mp_forward(X, Y, R, snd, rcv, nnodes), RTOL, ATOL)
    assert float(out[0].abs().max()) == 0.0  # the node without edges
    if C <= 128:
        g = torch.Generator().manual_seed(C + 1)
        R16 = torch.randn(E, 16, C, generator=g, dtype=torch.float64)
        out16 = cabi.mp_forward(X.float().to(DEV), Y.float().to(DEV), R16.float().to(DEV), snd.to(DEV), fo, nnodes)
        close(out16, O.mp_forward(X, Y, R16, snd, rcv, nnodes), RTOL, ATOL)


@pytest.mark.parametrize("case", MP_CASES, ids=lambda c: "N%d_d%d_C%d_%s_s%d" % (c[0], c[1], c[2], c[3], c[5]))
def test_mp_backward(cabi, case):
    _say("mp_backward", case)
    nnodes = case[0]
    snd, rcv, X, Y, R, G = _mp_case(*case)
    gX_ref, gY_ref, gR_ref = O.mp_backward(X, Y, R, G, snd, rcv)
    d = lambda t: t.float().to(DEV)
    fo = cabi.first_occurences(rcv.to(DEV), nnodes)
    perm, off = cabi.stable_key_sort(snd.to(DEV), nnodes)
    gX, gY, gR = cabi.mp_backward(d(X), d(Y), d(R), d(G), snd.to(DEV), fo, perm, off, nnodes)
    close(gR, gR_ref, RTOL, ATOL)
    close(gY, gY_ref, RTOL, ATOL)
    close(gX, gX_ref, RTOL, ATOL)


PER_M_CASES = [(64, 8, 32, "poisson", 0.2, 0), (300, 52, 128, "poisson", 0.05, 3), (40, 150, 128, "poisson", 0.0, 4),
               (100, 20, 160, "poisson", 0.1, 5), (150, 40, 192, "poisson", 0.0, 6), (60, 10, 224, "poisson", 0.0, 7),
               (80, 25, 256, "poisson", 0.3, 8), (4096, 30, 96, "fixed", 0.0, 0)]


@pytest.mark.parametrize("case", PER_M_CASES, ids=lambda c: "N%d_d%d_C%d_%s_s%d" % (c[0], c[1], c[2], c[3], c[5]))
def test_mp_per_component_weights(cabi, case):
    """Message passing with radial weights per component, R [E, 16, C] (the literal shape of benchmark configuration 2:
    4096 nodes x 30 edges, 96 channels, weights edges x 16 x 96): forward and the three gradients against the oracle,
    and equality with the per-degree op when the weights of a degree's components coincide."""
    _say("mp per component", case)
    nnodes, C = case[0], case[2]
    snd, rcv, X, Y, R4, G = _mp_case(*case)
    E = snd.numel()
    R = torch.randn(E, 16, C, generator=torch.Generator().manual_seed(case[5] + 100), dtype=torch.float64)
    d = lambda t: t.float().to(DEV)
    fo = cabi.first_occurences(rcv.to(DEV), nnodes)
    perm, off = cabi.stable_key_sort(snd.to(DEV), nnodes)
    out = cabi.mp_forward(d(X), d(Y), d(R), snd.to(DEV), fo, nnodes)
    close(out, O.mp_forward(X, Y, R, snd, rcv, nnodes), RTOL, ATOL)
    gX, gY, gR = cabi.mp_backward(d(X), d(Y), d(R), d(G), snd.to(DEV), fo, perm, off, nnodes)
    gX_ref, gY_ref, gR_ref = O.mp_backward(X, Y, R, G, snd, rcv)
    assert gR.shape == (E, 16, C)
    close(gR, gR_ref, RTOL, ATOL)
    close(gY, gY_ref, RTOL, ATOL)
    close(gX, gX_ref, RTOL, ATOL)
    only_y = cabi.mp_backward(d(X), d(Y), d(R), d(G), snd.to(DEV), fo, None, None, nnodes, need_gX=False, need_gR=False)
    assert only_y[0] is None and only_y[2] is None and torch.equal(only_y[1], gY)
    expanded = d(R4)[:, O.L_OF_M.to(DEV), :].contiguous()
    same = cabi.mp_forward(d(X), d(Y), expanded, snd.to(DEV), fo, nnodes)
    close(same, cabi.mp_forward(d(X), d(Y), d(R4), snd.to(DEV), fo, nnodes).double().cpu(), 1e-6, 1e-6)


def test_mp_backward_subsets(cabi):
    """Only the requested gradients are produced; each equals the full computation."""
    case = (120, 20, 128, "poisson", 0.1, 21)
    _say("mp_backward_subsets", case)
    nnodes = case[0]
    snd, rcv, X, Y, R, G = _mp_case(*case)
    d = lambda t: t.float().to(DEV)
    fo = cabi.first_occurences(rcv.to(DEV), nnodes)
    perm, off = cabi.stable_key_sort(snd.to(DEV), nnodes)
    full = cabi.mp_backward(d(X), d(Y), d(R), d(G), snd.to(DEV), fo, perm, off, nnodes)
    for mask in range(1, 7):
        need = dict(need_gX=bool(mask & 1), need_gY=bool(mask & 2), need_gR=bool(mask & 4))
        part = cabi.mp_backward(d(X), d(Y), d(R), d(G), snd.to(DEV), fo, perm, off, nnodes, **need)
        for got, want, on in zip(part, full, (need["need_gX"], need["need_gY"], need["need_gR"])):
            if on:
                assert torch.equal(got, want)
            else:
                assert got is None


def test_mp_reproducible_bitwise(cabi):
    """No atomics: two runs give identical bits."""
    case = (256, 30, 96, "poisson", 0.0, 31)
    nnodes = case[0]
    snd, rcv, X, Y, R, G = _mp_case(*case)
    d = lambda t: t.float().to(DEV)
    fo = cabi.first_occurences(rcv.to(DEV), nnodes)
    perm, off = cabi.stable_key_sort(snd.to(DEV), nnodes)
    a = cabi.mp_forward(d(X), d(Y), d(R), snd.to(DEV), fo, nnodes)
    b = cabi.mp_forward(d(X), d(Y), d(R), snd.to(DEV), fo, nnodes)
    assert torch.equal(a, b)
    ga = cabi.mp_backward(d(X), d(Y), d(R), d(G), snd.to(DEV), fo, perm, off, nnodes)
    gb = cabi.mp_backward(d(X), d(Y), d(R), d(G), snd.to(DEV), fo, perm, off, nnodes)
    for u, v in zip(ga, gb):
        assert torch.equal(u, v)


def test_mp_rejects_bad_arguments(cabi):
    X = torch.zeros(4, 48, device=DEV)
    Y = torch.zeros(16, 0, device=DEV)
    R = torch.zeros(0, 4, 48, device=DEV)
    snd = torch.zeros(0, dtype=torch.int32, device=DEV)
    fo = torch.zeros(8, dtype=torch.int32, device=DEV)
    with pytest.raises(RuntimeError, match="multiple of 32"):
        cabi.mp_forward(X, Y, R, snd, fo, 4)
    with pytest.raises(RuntimeError, match="GPU"):
        cabi.mp_forward(torch.zeros(4, 32), Y, R, snd, fo, 4)


# ------------------------------------------------------------------------------------------------
# spherical harmonics
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("E,seed", [(1, 0), (1000, 1), (100003, 2)])
def test_sh_forward_backward(cabi, E, seed):
    _say("sh", E, seed)
    g = torch.Generator().manual_seed(seed)
    xyz = torch.randn(E, 3, generator=g, dtype=torch.float64) * 2.5
    gY = torch.randn(16, E, generator=g, dtype=torch.float64)
    ref = O.spherical_harmonics(xyz)
    gref = O.spherical_harmonics_backward(xyz, gY)
    Y = cabi.sh_forward(xyz.float().to(DEV))
    gx = cabi.sh_backward(xyz.float().to(DEV), gY.float().to(DEV))
    close(Y, ref, 1e-5, 2e-6)
    close(gx, gref, 2e-5, 2e-6)


# ------------------------------------------------------------------------------------------------
# spline
# ------------------------------------------------------------------------------------------------
# from 32 768 edges on the forward without derivative and the backward run on their LDS-table kernels: full rows of
# slices, a last slice of 8 of 32 outputs, and more edges than one pass of chunks holds (256 workgroups x 8 192)
@pytest.mark.parametrize("E,J,seed", [(1, 128, 0), (777, 384, 1), (5000, 512, 2), (300, 768, 3), (40_000, 512, 4),
                                      (70_001, 72, 5), (2_200_003, 8, 6)])
def test_spline_forward_backward(cabi, E, J, seed):
    _say("spline", E, J, seed)
    g = torch.Generator().manual_seed(seed)
    r_max = 5.0
    knots_np, h = np.linspace(1e-12, r_max + 1.0, 256, retstep=True)
    knots = torch.from_numpy(knots_np)
    table = torch.sin(knots[:, None] * torch.linspace(0.3, 3.0, J, dtype=torch.float64)[None, :]) * torch.randn(
        1, J, generator=g, dtype=torch.float64
    )
    coeffs = O.spline_coefficients(knots, table)
    r = torch.rand(E, generator=g, dtype=torch.float64) * 5.6 + 0.4  # some beyond r_max
    gR = torch.randn(E, J, generator=g, dtype=torch.float64)
    # evaluate the oracle at the fp32-rounded radii the kernel sees
    r32 = r.float()
    val_ref, der_ref = O.spline_eval(r32.double(), knots, coeffs, float(h), r_max, deriv=True)
    gr_ref = O.spline_backward(gR, der_ref)
    d = lambda t: t.float().to(DEV)
    val, der = cabi.spline_forward(d(r), d(knots), d(coeffs), float(h), r_max, want_deriv=True)
    val_only = cabi.spline_forward(d(r), d(knots), d(coeffs), float(h), r_max)
    gr = cabi.spline_backward(d(r), d(knots), d(coeffs), d(gR), float(h), r_max)
    assert torch.equal(val, val_only)
    close(val, val_ref, 2e-5, 2e-6)
    close(der, der_ref, 2e-5, 5e-6)
    # a sum of J signed terms: the error bound scales with the sum of their magnitudes (5e-6: over millions of edges with
    # only 8 outputs the cancellations inside b + 2 c x + 3 d x^2, x in fp32, reach 2.1 times the 2e-6 that a few
    # thousand edges stay within, in the direct kernel and in the LDS-table kernel alike)
    bound = 5e-6 * (gR.abs() * der_ref.abs()).sum(-1) + 1e-30
    assert bool(((gr.double().cpu() - gr_ref).abs() <= bound).all())
    assert float(val[(r32 > r_max).to(DEV)].abs().sum()) == 0.0


# ------------------------------------------------------------------------------------------------
# linears (fp32 MFMA)
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("N,K,Nout,seed", [(1, 32, 32, 0), (33, 64, 64, 1), (1000, 128, 128, 2), (257, 96, 96, 3), (100, 192, 192, 4), (70, 256, 256, 5), (50, 64, 128, 6), (50, 160, 96, 7)])
def test_linear(cabi, N, K, Nout, seed):
    _say("linear", N, K, Nout, seed)
    g = torch.Generator().manual_seed(seed)
    X = torch.randn(N, 16, K, generator=g, dtype=torch.float64)
    W = torch.randn(4, K, Nout, generator=g, dtype=torch.float64)
    ref = O.linear(X, W)
    WT = W.transpose(-1, -2).contiguous()
    out = cabi.linear(X.float().to(DEV), WT.float().to(DEV))
    close(out, ref, 1e-5, 2e-6)
    # the reference's own acceptance threshold (tests/linear.py:142-143): mean abs error < 5e-5
    assert float((out.double().cpu() - ref).abs().mean()) < 5e-5


@pytest.mark.parametrize("N,C,ne,seed", [(1, 32, 1, 0), (500, 128, 10, 1), (333, 96, 4, 2), (64, 192, 10, 3)])
def test_elemental_linear(cabi, N, C, ne, seed):
    _say("elemental_linear", N, C, ne, seed)
    g = torch.Generator().manual_seed(seed)
    X = torch.randn(N, 16, C, generator=g, dtype=torch.float64)
    W = torch.randn(ne, 4, C, C, generator=g, dtype=torch.float64)
    elem = torch.randint(0, ne, (N,), generator=g)
    one_hot = torch.nn.functional.one_hot(elem, ne).double()
    ref = O.elemental_linear(X, W, one_hot)
    perm, off = cabi.stable_key_sort(elem.int().to(DEV), ne)
    WT = W.transpose(-1, -2).contiguous()
    out = cabi.linear(X.float().to(DEV), WT.float().to(DEV), perm, off)
    close(out, ref, 1e-5, 2e-6)


@pytest.mark.parametrize("N,K,Nout,ne,seed", [(1, 32, 32, 1, 0), (700, 128, 128, 10, 1), (130, 96, 64, 3, 2)])
def test_scalar_elemental_linear_and_zero_group(cabi, N, K, Nout, ne, seed):
    """Single-component features (the layer-2 skip connection) and rows whose one-hot names no element."""
    _say("scalar_elemental_linear", N, K, Nout, ne, seed)
    g = torch.Generator().manual_seed(seed)
    X = torch.randn(N, K, generator=g, dtype=torch.float64)
    W = torch.randn(ne, K, Nout, generator=g, dtype=torch.float64)
    elem = torch.randint(0, ne + 1, (N,), generator=g)  # value ne = "no element"
    ref = torch.einsum("nk,nkj->nj", X, torch.cat([W, torch.zeros(1, K, Nout, dtype=torch.float64)])[elem]) / math.sqrt(K)
    perm, off = cabi.stable_key_sort(elem.int().to(DEV), ne + 1)
    WT = W.transpose(-1, -2).contiguous().float().to(DEV)
    out = cabi.linear(X.float().to(DEV), WT, perm, off, zero_last_group=True)
    close(out, ref, 1e-5, 2e-6)
    assert float(out[(elem == ne).to(DEV)].abs().sum()) == 0.0
    # the same through the 16-component path
    X16 = torch.randn(N, 16, K, generator=g, dtype=torch.float64)
    W16 = torch.randn(ne, 4, K, Nout, generator=g, dtype=torch.float64)
    one_hot = torch.nn.functional.one_hot(elem, ne + 1)[:, :ne].double()
    ref16 = O.elemental_linear(X16, W16, one_hot)
    out16 = cabi.linear(X16.float().to(DEV), W16.transpose(-1, -2).contiguous().float().to(DEV), perm, off, zero_last_group=True)
    close(out16, ref16, 1e-5, 2e-6)


@pytest.mark.parametrize("N,C,ne,seed", [(1, 32, 1, 0), (21, 64, 4, 1), (700, 128, 10, 2), (5000, 96, 10, 3), (25000, 128, 10, 4)])
def test_node_glue_chains(cabi, N, C, ne, seed):
    """The three [N, C] linears between the layers as one launch per direction: against the fp64 definition, and bit for
    bit against the three separate launches of the linear kernel they stand for (rows without an element included)."""
    _say("node_glue", N, C, ne, seed)
    g = torch.Generator().manual_seed(seed)
    rnd = lambda *shape: torch.randn(*shape, generator=g, dtype=torch.float64)  # noqa: E731
    B1, gX2, d_h2 = rnd(N, C), rnd(N, C), rnd(N, C)
    Wp, Wu, Ws = rnd(C, C) / math.sqrt(C), rnd(C, C) / math.sqrt(C), rnd(ne, C, C)
    w1, nw = rnd(C), torch.rand(N, generator=g, dtype=torch.float64)
    scale, skip_scale = 0.8, 1.0 / math.sqrt(C * ne)
    elem = torch.randint(0, ne + 1, (N,), generator=g)  # value ne = "no element"
    Ws0 = torch.cat([Ws, torch.zeros(1, C, C, dtype=torch.float64)])[elem]  # [N, C, C]
    h1_ref = B1 @ Wp
    sc_ref = skip_scale * torch.einsum("nk,nkj->nj", h1_ref, Ws0)
    X2_ref = h1_ref @ Wu
    f32 = lambda t: t.float().to(DEV).contiguous()  # noqa: E731
    T = lambda t: t.transpose(-1, -2).contiguous()  # noqa: E731
    perm, off = cabi.stable_key_sort(elem.int().to(DEV), ne + 1)
    h1, sc, X2 = cabi.node_glue_forward(f32(B1), f32(T(Wp)), f32(T(Ws)), f32(T(Wu)), perm, off, skip_scale)
    close(h1, h1_ref, 1e-5, 2e-6)
    close(sc, sc_ref, 1e-5, 2e-6)
    close(X2, X2_ref, 1e-5, 2e-6)
    assert float(sc[(elem == ne).to(DEV)].abs().sum()) == 0.0
    h1_s = cabi.linear(f32(B1), f32(T(Wp)), scale=1.0)
    sc_s = cabi.linear(h1_s, f32(T(Ws)), perm, off, scale=skip_scale, zero_last_group=True)
    X2_s = cabi.linear(h1_s, f32(T(Wu)), scale=1.0)
    assert torch.equal(h1, h1_s) and torch.equal(sc, sc_s) and torch.equal(X2, X2_s)
    for weights in (None, nw):
        wn = torch.ones(N, dtype=torch.float64) if weights is None else weights
        g1_ref = (-1.0 * scale * w1)[None, :] * wn[:, None]  # the kernel's order of the fp64 products
        gh1_ref = gX2 @ Wu.t() + g1_ref - skip_scale * torch.einsum("nj,nkj->nk", d_h2, Ws0)
        gB_ref = gh1_ref @ Wp.t()
        gB = cabi.node_glue_backward(f32(gX2), f32(d_h2), f32(Wu), f32(Ws), f32(Wp), w1.to(DEV), scale,
                                     None if weights is None else weights.to(DEV), perm, off, skip_scale)
        close(gB, gB_ref, 1e-5, 2e-6)
        g1 = f32(g1_ref)  # rounded once from the fp64 product, as the kernel forms it
        a = cabi.linear(f32(gX2), f32(Wu), scale=1.0, residual=g1)
        b = cabi.linear(f32(d_h2), f32(Ws), perm, off, scale=-skip_scale, zero_last_group=True, residual=a)
        c = cabi.linear(b, f32(Wp), scale=1.0)
        assert torch.equal(gB, c)
    with pytest.raises(cabi.CudaMaceError, match="32, 64, 96 or 128"):
        cabi.node_glue_forward(torch.zeros(4, 160, device=DEV), torch.zeros(160, 160, device=DEV), torch.zeros(1, 160, 160, device=DEV),
                               torch.zeros(160, 160, device=DEV), torch.zeros(4, dtype=torch.int32, device=DEV),
                               torch.zeros(3, dtype=torch.int32, device=DEV), 1.0)


@pytest.mark.parametrize("N,C,ne,seed", [(2048, 128, 1, 0), (2500, 128, 10, 1), (4099, 96, 5, 2), (3000, 64, 3, 3), (6000, 128, 130, 4)])
def test_linear_many_rows(cabi, N, C, ne, seed):
    """16-component features with at least 2048 nodes and 64 / 96 / 128 square weights run on the kernel that keeps the
    weight block in LDS (one workgroup per compute unit walking 32-row tiles); more than 128 weight groups stay on the
    tiled kernels.  Groups of very different sizes, an empty group, a group of one node, tiles that end inside a group,
    rows of no group, with and without row_scale; twice, for the same bits."""
    _say("linear_many_rows", N, C, ne, seed)
    g = torch.Generator().manual_seed(seed)
    X = torch.randn(N, 16, C, generator=g, dtype=torch.float64).float().double()
    S = torch.randn(N, C, generator=g, dtype=torch.float64).float().double()
    W = torch.randn(ne, 4, C, C, generator=g, dtype=torch.float64).float().double()
    p = torch.rand(ne + 1, generator=g, dtype=torch.float64) ** 3 + 1e-3
    elem = torch.multinomial(p, N, replacement=True, generator=g)  # value ne = "no element"
    if ne >= 3:
        elem[elem == 1] = 0  # an empty group
        elem[elem == 2] = 0
        elem[N // 2] = 2     # a group of one node
    Xd, Sd = X.float().to(DEV), S.float().to(DEV)
    WT = W.transpose(-1, -2).contiguous().float().to(DEV)
    # one weight group for all nodes
    close(cabi.linear(Xd, WT[0]), O.linear(X, W[0]), 1e-5, 2e-6)
    close(cabi.linear(Xd, WT[0], row_scale=Sd), O.linear(X * S[:, None, :], W[0]), 1e-5, 2e-6)
    # per-element weights, rows of the last key are zero
    ref = torch.zeros(N, 16, C, dtype=torch.float64)
    ref_s = torch.zeros(N, 16, C, dtype=torch.float64)
    for e in range(ne):
        rows = (elem == e).nonzero()[:, 0]
        if rows.numel():
            ref[rows] = O.linear(X[rows], W[e])
            ref_s[rows] = O.linear(X[rows] * S[rows][:, None, :], W[e])
    perm, off = cabi.stable_key_sort(elem.int().to(DEV), ne + 1)
    out = cabi.linear(Xd, WT, perm, off, zero_last_group=True)
    close(out, ref, 1e-5, 2e-6)
    assert float(out[(elem == ne).to(DEV)].abs().sum()) == 0.0
    out_s = cabi.linear(Xd, WT, perm, off, zero_last_group=True, row_scale=Sd)
    close(out_s, ref_s, 1e-5, 2e-6)
    assert torch.equal(out, cabi.linear(Xd, WT, perm, off, zero_last_group=True))
    # every node in a group (no zero rows): the keys of the rows of no group move to the last element
    elem2 = torch.where(elem == ne, torch.full_like(elem, ne - 1), elem)
    rows = (elem == ne).nonzero()[:, 0]
    ref[rows] = O.linear(X[rows], W[ne - 1])
    perm2, off2 = cabi.stable_key_sort(elem2.int().to(DEV), ne)
    close(cabi.linear(Xd, WT, perm2, off2), ref, 1e-5, 2e-6)


@pytest.mark.parametrize("N,C", [(25000, 128), (100000, 192), (5000, 96)])
def test_linear_at_benchmark_sizes(cabi, N, C):
    """The channel mixing at the node and channel counts of benchmark configurations 4, 5 and 3, per-element weights
    with row_scale (the backward launch of the model): 1 500 random rows against the fp64 oracle, and linearity in X
    over the whole output (the kernel applied to a X1 + b X2 equals a out1 + b out2 to fp32 rounding)."""
    _say("linear_at_benchmark_sizes", N, C)
    ne = 10
    g = torch.Generator(device=DEV).manual_seed(N + C)
    X1 = torch.randn(N, 16, C, device=DEV, generator=g)
    X2 = torch.randn(N, 16, C, device=DEV, generator=g)
    S = torch.randn(N, C, device=DEV, generator=g)
    WT = torch.randn(ne, 4, C, C, device=DEV, generator=g)
    elem = torch.randint(0, ne, (N,), device=DEV, generator=g)
    perm, off = cabi.stable_key_sort(elem.int(), ne)
    out1 = cabi.linear(X1, WT, perm, off, row_scale=S)
    rows = torch.randperm(N, device=DEV, generator=g)[:1500]
    W = WT.transpose(-1, -2).double().cpu()
    er, Xr, Sr = elem[rows].cpu(), X1[rows].double().cpu(), S[rows].double().cpu()
    ref = torch.zeros(rows.numel(), 16, C, dtype=torch.float64)
    for e in range(ne):
        sel = (er == e).nonzero()[:, 0]
        if sel.numel():
            ref[sel] = O.linear(Xr[sel] * Sr[sel][:, None, :], W[e])
    close(out1[rows], ref, 1e-5, 2e-6)
    out2 = cabi.linear(X2, WT, perm, off, row_scale=S)
    a, b = 0.75, -1.5  # exact in fp32, so the combined input is rounded once per element
    out12 = cabi.linear(a * X1 + b * X2, WT, perm, off, row_scale=S)
    scale = float(out1.abs().max())
    assert float((out12 - (a * out1 + b * out2)).abs().max()) < 2e-5 * scale
    del out12, out2, X2
    # plain weights, no row_scale (the forward launch of the second layer)
    outp = cabi.linear(X1, WT[0])
    close(outp[rows], O.linear(Xr, W[0]), 1e-5, 2e-6)


# ------------------------------------------------------------------------------------------------
# symmetric contraction with synthetic sparse tables
# ------------------------------------------------------------------------------------------------
def _random_tables(seed, n3=40, n2=10, P3=23, P2=4):
    """Random monomial lists with 1-3 (path, value) terms each, plus the dense U they stand for."""
    rng = np.random.default_rng(seed)
    triples = set()
    while len(triples) < n3:
        triples.add(tuple(sorted(rng.integers(0, 16, 3).tolist())))
    pairs = set()
    while len(pairs) < n2:
        pairs.add(tuple(sorted(rng.integers(0, 16, 2).tolist())))
    U3 = torch.zeros(16, 16, 16, P3, dtype=torch.float64)
    U2 = torch.zeros(16, 16, P2, dtype=torch.float64)
    mono3, off3, path3, val3 = [], [0], [], []
    for (i, j, k) in sorted(triples):
        mono3.append(i | (j << 8) | (k << 16))
        for _ in range(int(rng.integers(1, 4))):
            p, v = int(rng.integers(0, P3)), float(rng.normal())
            U3[i, j, k, p] += v  # the whole coefficient sits on the sorted position
            path3.append(p)
            val3.append(v)
        off3.append(len(path3))
    mono2, off2, path2, val2 = [], [0], [], []
    for (i, j) in sorted(pairs):
        mono2.append(i | (j << 8))
        p, v = int(rng.integers(0, P2)), float(rng.normal())
        U2[i, j, p] += v
        path2.append(p)
        val2.append(v)
        off2.append(len(path2))
    ti = lambda a: torch.tensor(a, dtype=torch.int32)
    tf = lambda a: torch.tensor(a, dtype=torch.float32)
    return U3, U2, ti(mono3), ti(off3), ti(path3), tf(val3), ti(mono2), ti(off2), ti(path2), tf(val2)


@pytest.mark.parametrize("N,C,ne,seed", [(1, 32, 1, 0), (37, 128, 10, 1), (20, 96, 3, 2), (9, 192, 4, 3), (5, 256, 2, 4)])
def test_symcon_synthetic_tables(cabi, N, C, ne, seed):
    _say("symcon", N, C, ne, seed)
    U3, U2, mono3, off3, path3, val3, mono2, off2, path2, val2 = _random_tables(seed)
    g = torch.Generator().manual_seed(seed)
    X = torch.randn(N, 16, C, generator=g, dtype=torch.float64)
    W3 = torch.randn(ne, 23, C, generator=g, dtype=torch.float64)
    W2 = torch.randn(ne, 4, C, generator=g, dtype=torch.float64)
    W1 = torch.randn(ne, 1, C, generator=g, dtype=torch.float64)
    types = torch.randint(0, ne, (N,), generator=g).int()
    gout = torch.randn(N, C, generator=g, dtype=torch.float64)
    # the oracle sees the fp32-rounded table values
    U3r, U2r = torch.zeros_like(U3), torch.zeros_like(U2)
    for t in range(mono3.numel()):
        w = int(mono3[t])
        for q in range(int(off3[t]), int(off3[t + 1])):
            U3r[w & 255, (w >> 8) & 255, (w >> 16) & 255, int(path3[q])] += float(val3[q])
    for t in range(mono2.numel()):
        w = int(mono2[t])
        for q in range(int(off2[t]), int(off2[t + 1])):
            U2r[w & 255, (w >> 8) & 255, int(path2[q])] += float(val2[q])
    Xa = X.clone().requires_grad_(True)
    ref = O.symmetric_contraction(Xa, types, U3r, U2r, W3, W2, W1)
    (ref * gout).sum().backward()
    d = lambda t: t.to(DEV)
    f = lambda t: t.float().to(DEV)
    T3, T2, T1 = cabi.symcon_tables(d(off3), d(path3), d(val3), d(off2), d(path2), d(val2), f(W3), f(W2), f(W1))
    perm, offs = cabi.stable_key_sort(d(types), ne)
    out, grad = cabi.symcon_forward(f(X), perm, offs, d(mono3), d(mono2), T3, T2, T1)
    out_nograd, none = cabi.symcon_forward(f(X), perm, offs, d(mono3), d(mono2), T3, T2, T1, want_grad=False)
    gX = cabi.symcon_backward(grad, f(gout))
    assert none is None and torch.equal(out, out_nograd)
    close(out, ref.detach(), 3e-5, 3e-6)
    close(gX, Xa.grad, 3e-5, 3e-6)


# ------------------------------------------------------------------------------------------------
# edge geometry (vectors, lengths, scatter of edge gradients to atoms)
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("nnodes,avg,iso,seed", [(1, 2, 0.0, 0), (50, 8, 0.3, 1), (3000, 52, 0.0, 2), (20, 200, 0.0, 3)])
def test_edge_geometry(cabi, nnodes, avg, iso, seed):
    _say("edge_geometry", nnodes, avg, iso, seed)
    row_b, row_a = random_graph(nnodes, avg, seed, isolated_frac=iso)  # row_a sorted
    E = row_a.numel()
    g = torch.Generator().manual_seed(seed)
    pos = (torch.rand(nnodes, 3, generator=g, dtype=torch.float64) * 20).requires_grad_(True)
    shifts = (torch.randn(E, 3, generator=g, dtype=torch.float64) * 3).requires_grad_(True)
    gv = torch.randn(E, 3, generator=g, dtype=torch.float64)
    gl = torch.randn(E, generator=g, dtype=torch.float64)
    vec_ref, len_ref = O.edge_geometry(pos, row_a, row_b, shifts)
    # the kernel receives fp32 gradients: give the oracle the same rounded values
    ((vec_ref * gv.float().double()).sum() + (len_ref * gl.float().double()).sum()).backward()
    d = lambda t: t.detach().to(DEV)
    fo = cabi.first_occurences(d(row_a), nnodes)
    perm, off = cabi.stable_key_sort(d(row_b), nnodes)
    vec, length = cabi.edge_geometry_forward(d(pos), d(row_a), d(row_b), d(shifts))
    gpos, gshift = cabi.edge_geometry_backward(d(pos), d(row_a), d(row_b), d(shifts), fo, perm, off, d(gv).float(), d(gl).float(),
                                               need_positions=True, need_shifts=True)
    assert torch.equal(vec.cpu(), vec_ref.detach().float()) and torch.equal(length.cpu(), len_ref.detach().float())
    close(gpos, pos.grad, 1e-12, 1e-13)
    close(gshift, shifts.grad, 1e-12, 1e-13)
    only_vec, _ = cabi.edge_geometry_backward(d(pos), d(row_a), d(row_b), d(shifts), fo, perm, off, d(gv).float(), None)
    pos.grad = None
    vec2, _ = O.edge_geometry(pos, row_a, row_b, shifts)
    (vec2 * gv.float().double()).sum().backward()
    close(only_vec, pos.grad, 1e-12, 1e-13)
    # row map: the same positions stored in a permuted order give bit-identical vectors, and the position gradient
    # comes out in that order
    rows = torch.randperm(nnodes, generator=g).int()
    stored = torch.empty_like(pos.detach())
    stored[rows.long()] = pos.detach()  # atom n sits in row rows[n]
    vec_m, len_m = cabi.edge_geometry_forward(d(stored), d(row_a), d(row_b), d(shifts), node_rows=d(rows))
    assert torch.equal(vec_m, vec) and torch.equal(len_m, length)
    gpos_m, _ = cabi.edge_geometry_backward(d(stored), d(row_a), d(row_b), d(shifts), fo, perm, off, d(gv).float(), d(gl).float(),
                                            need_positions=True, node_rows=d(rows))
    assert torch.equal(gpos_m[d(rows).long()], gpos)


# ---- readouts ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("N,C,H,seed", [(1, 32, 16, 0), (1000, 128, 16, 1), (37, 96, 5, 2), (515, 256, 1, 3), (16, 64, 16, 4), (50, 30, 7, 5), (20000, 128, 16, 6)])
def test_readout_forward_backward(cabi, N, C, H, seed):
    g = torch.Generator().manual_seed(seed)
    h1 = torch.randn(N, C, generator=g).double()
    h2 = torch.randn(N, C, generator=g).double()
    w1 = torch.randn(C, generator=g, dtype=torch.float64) / C ** 0.5
    W2a = torch.randn(C, H, generator=g, dtype=torch.float64) / C ** 0.5
    w2b = torch.randn(H, generator=g, dtype=torch.float64) / H ** 0.5
    gn = torch.randn(N, generator=g, dtype=torch.float64)
    cst, scale, shift = 1.6791767923989418, 0.8, -0.3
    a1, a2 = h1.clone().requires_grad_(True), h2.clone().requires_grad_(True)
    ref = O.readout_energies(a1, a2, w1, W2a, w2b, cst, scale, shift)
    (ref * gn).sum().backward()
    dev = lambda t: t.to(DEV)
    es, d2, feats = cabi.readout_forward(dev(h1.float()), dev(h2.float()), dev(w1), dev(W2a), dev(w2b), cst, scale, shift)
    close(es, ref.detach(), 1e-12, 1e-12)  # fp64 arithmetic on identical (fp32-representable) inputs
    assert torch.equal(feats.cpu(), torch.cat([h1, h2], dim=1))
    # optional row map of the feature output: node n goes to row rows[n]; energies stay in place
    rows = torch.randperm(N, generator=g).int()
    es_m, _, feats_m = cabi.readout_forward(dev(h1.float()), dev(h2.float()), dev(w1), dev(W2a), dev(w2b), cst, scale, shift,
                                            feats_rows=dev(rows))
    assert torch.equal(es_m, es) and torch.equal(feats_m.cpu()[rows.long()], torch.cat([h1, h2], dim=1))
    g1, g2 = cabi.readout_backward(dev(gn), dev(w1), d2, scale)
    close(g1, a1.grad, 1e-6, 1e-7)
    close(g2, a2.grad, 1e-6, 1e-7)
    only2 = cabi.readout_backward(dev(gn), dev(w1), d2, scale, need_h1=False)
    assert only2[0] is None and torch.equal(only2[1], g2)


def test_linear_row_scale(cabi):
    """row_scale folds an element-wise factor shared by the 16 components into the operand load."""
    g = torch.Generator().manual_seed(3)
    N, K, Nout = 300, 96, 128
    X = torch.randn(N, 16, K, generator=g, dtype=torch.float64).float().double()
    S = torch.randn(N, K, generator=g, dtype=torch.float64).float().double()
    W = torch.randn(4, K, Nout, generator=g, dtype=torch.float64).float().double()
    ref = O.linear(X * S[:, None, :], W)
    got = cabi.linear(X.float().to(DEV), W.transpose(-1, -2).contiguous().float().to(DEV), row_scale=S.float().to(DEV))
    close(got, ref, 1e-5, 2e-6)


@pytest.mark.parametrize("K,Nout", [(128, 128), (64, 160), (32, 96)])
def test_linear_residual(cabi, K, Nout):
    """residual is added to the written rows, for 16-component and scalar features (both kernel variants: 128 and 96
    columns run on the LDS-ring kernel when K has more than one chunk, 160 columns and K = 32 on the plain one)."""
    g = torch.Generator().manual_seed(5)
    N = 333
    X = torch.randn(N, 16, K, generator=g, dtype=torch.float64).float().double()
    R = torch.randn(N, 16, Nout, generator=g, dtype=torch.float64).float().double()
    W = torch.randn(4, K, Nout, generator=g, dtype=torch.float64).float().double()
    got = cabi.linear(X.float().to(DEV), W.transpose(-1, -2).contiguous().float().to(DEV), residual=R.float().to(DEV))
    close(got, O.linear(X, W) + R, 1e-5, 2e-6)
    Xs, Rs, Ws = X[:, 0].contiguous(), R[:, 0].contiguous(), W[0]
    got = cabi.linear(Xs.float().to(DEV), Ws.t().contiguous().float().to(DEV), scale=1.0, residual=Rs.float().to(DEV))
    close(got, Xs @ Ws + Rs, 1e-5, 2e-6)
