"""Message passing with in-kernel radial spline: parity with the fp64 oracle (spline evaluation followed by the
message-passing definition, gradients by autograd) and bit-level consistency with the two-step GPU path."""
import numpy as np
import pytest
import torch

from oracle import ops as O
from tests.util import close, mp_inputs, random_graph

pytestmark = pytest.mark.gpu

CASES = [
    # nnodes, avg degree, channels, isolated fraction, seed
    (50, 6, 32, 0.2, 0),
    (200, 30, 64, 0.0, 1),
    (300, 52, 96, 0.05, 2),
    (300, 52, 128, 0.0, 3),
    (30, 160, 128, 0.0, 4),
    (120, 40, 192, 0.1, 5),
    (60, 20, 256, 0.0, 6),
    (70, 30, 160, 0.1, 7),   # 40 of 64 lanes carry channels
    (50, 90, 224, 0.0, 8),   # 56 of 64 lanes; segments longer than one 64-edge chunk
]


def _case(nnodes, avg, C, iso, seed):
    snd, rcv = random_graph(nnodes, avg, seed, isolated_frac=iso)
    E = snd.numel()
    X, v, _, G = mp_inputs(nnodes, E, C, seed)
    g = torch.Generator().manual_seed(seed + 100)
    r = torch.rand(E, generator=g, dtype=torch.float64) * 4.6 + 0.7  # a few beyond r_max = 5
    r = r.float().double()  # the kernel sees fp32 lengths
    Y = O.spherical_harmonics(v).contiguous()
    knots_np, h = np.linspace(1e-12, 6.0, 256, retstep=True)
    knots = torch.from_numpy(knots_np)
    J = 4 * C
    table = torch.sin(knots[:, None] * torch.linspace(0.5, 2.5, J, dtype=torch.float64)[None, :]) * torch.randn(
        1, J, generator=g, dtype=torch.float64)
    coeffs = O.spline_coefficients(knots, table).float().double()  # the kernel sees fp32 coefficients
    return snd, rcv, X, Y, r, knots.float().double(), coeffs, float(np.float32(h)), G


@pytest.mark.parametrize("case", CASES, ids=lambda c: "N%d_d%d_C%d_s%d" % (c[0], c[1], c[2], c[4]))
def test_mp_spline_forward_backward(cabi, case):
    print("mp_spline", case, flush=True)
    nnodes, C = case[0], case[2]
    snd, rcv, X, Y, r, knots, coeffs, h, G = _case(*case)
    E = snd.numel()
    Xa, Ya, ra = (t.clone().requires_grad_(True) for t in (X, Y, r))
    R = O.spline_eval(ra, knots, coeffs, h, 5.0).view(E, 4, C)
    ref = O.mp_forward(Xa, Ya, R, snd, rcv, nnodes)
    (ref * G).sum().backward()

    d = lambda t: t.float().cuda()
    fo = cabi.first_occurences(rcv.cuda(), nnodes)
    perm, off = cabi.stable_key_sort(snd.cuda(), nnodes)
    out = cabi.mp_spline_forward(d(X), d(Y), d(r), d(knots), d(coeffs), h, 5.0, snd.cuda(), fo, nnodes)
    gX, gY, gr = cabi.mp_spline_backward(d(X), d(Y), d(r), d(knots), d(coeffs), h, 5.0, d(G), snd.cuda(), fo, perm, off, nnodes)
    close(out, ref.detach(), 2e-5, 2e-6)
    close(gX, Xa.grad, 2e-5, 2e-6)
    close(gY, Ya.grad, 2e-5, 2e-6)
    close(gr, ra.grad, 3e-5, 3e-6)

    # the two-step GPU path (spline kernel, then tabulated message passing) gives the same numbers
    R32 = cabi.spline_forward(d(r), d(knots), d(coeffs), h, 5.0)
    out2 = cabi.mp_forward(d(X), d(Y), R32.view(E, 4, C), snd.cuda(), fo, nnodes)
    close(out, out2.double().cpu(), 1e-6, 1e-6)
    gX2, gY2, gR2 = cabi.mp_backward(d(X), d(Y), R32.view(E, 4, C), d(G), snd.cuda(), fo, perm, off, nnodes)
    gr2 = cabi.spline_backward(d(r), d(knots), d(coeffs), gR2.view(E, 4 * C), h, 5.0)
    close(gY, gY2.double().cpu(), 1e-5, 1e-6)
    close(gX, gX2.double().cpu(), 1e-5, 1e-6)
    bound = 4e-6 * (gR2.view(E, -1).abs().double().cpu() * O.spline_eval(r, knots, coeffs, h, 5.0, deriv=True)[1].abs()).sum(-1) + 1e-30
    assert bool(((gr.double().cpu() - gr2.double().cpu()).abs() <= bound).all())

    # edge-vector variant: harmonics and length computed in-kernel; oracle = SH + spline + MP, gradient by autograd
    g2 = torch.Generator().manual_seed(case[4] + 7)
    vec = torch.randn(E, 3, generator=g2, dtype=torch.float64)
    vec = (vec / vec.norm(dim=1, keepdim=True) * r[:, None]).float().double()  # lengths spread like r, fp32-representable
    va = vec.clone().requires_grad_(True)
    Xb = X.clone().requires_grad_(True)
    Rv = O.spline_eval(va.norm(dim=1), knots, coeffs, h, 5.0).view(E, 4, C)
    ref_e = O.mp_forward(Xb, O.spherical_harmonics(va), Rv, snd, rcv, nnodes)
    (ref_e * G).sum().backward()
    out_e = cabi.mp_edge_forward(d(X), d(vec), d(knots), d(coeffs), h, 5.0, snd.cuda(), fo, nnodes)
    gX_e, gvec = cabi.mp_edge_backward(d(X), d(vec), d(knots), d(coeffs), h, 5.0, d(G), snd.cuda(), fo, perm, off, nnodes)
    close(out_e, ref_e.detach(), 2e-5, 2e-6)
    close(gX_e, Xb.grad, 2e-5, 2e-6)
    close(gvec, va.grad, 5e-5, 5e-6)
    gX_only, none = cabi.mp_edge_backward(d(X), d(vec), d(knots), d(coeffs), h, 5.0, d(G), snd.cuda(), fo, perm, off, nnodes,
                                          need_gvec=False)
    assert none is None and torch.equal(gX_only, gX_e)
    none, gvec_only = cabi.mp_edge_backward(d(X), d(vec), d(knots), d(coeffs), h, 5.0, d(G), snd.cuda(), fo, perm, off, nnodes,
                                            need_gX=False)
    assert none is None and torch.equal(gvec_only, gvec)

    # subsets of gradients
    only_r = cabi.mp_spline_backward(d(X), d(Y), d(r), d(knots), d(coeffs), h, 5.0, d(G), snd.cuda(), fo, perm, off, nnodes,
                                     need_gX=False, need_gY=False)
    assert only_r[0] is None and only_r[1] is None and torch.equal(only_r[2], gr)
    no_x = cabi.mp_spline_backward(d(X), d(Y), d(r), d(knots), d(coeffs), h, 5.0, d(G), snd.cuda(), fo, perm, off, nnodes,
                                   need_gX=False)
    assert no_x[0] is None and torch.equal(no_x[1], gY) and torch.equal(no_x[2], gr)


@pytest.mark.parametrize("degree", [70, 200])
def test_edges_beyond_cutoff_and_invalid_senders_cost_nothing_and_contribute_nothing(cabi, degree):
    """A list with a wide skin (most edges beyond r_max) and a few out-of-range sender indices: those edges add nothing
    to the output and get exactly zero gradients; the rest matches the oracle evaluated on the live edges alone.  The
    kernels stage 64 live edges at a time out of as many raw ones as that takes: 70 raw edges per node fill one chunk from
    two reads, 200 make chunks that end in the middle of a read."""
    nnodes, C, seed = 90, 128, 11
    snd, rcv = random_graph(nnodes, degree, seed)
    E = snd.numel()
    X, _, _, G = mp_inputs(nnodes, E, C, seed)
    g = torch.Generator().manual_seed(seed)
    r = torch.rand(E, generator=g, dtype=torch.float64) * 9.0 + 0.7  # r_max = 5: about half the edges are beyond it
    vec = torch.randn(E, 3, generator=g, dtype=torch.float64)
    vec = (vec / vec.norm(dim=1, keepdim=True) * r[:, None]).float().double()
    snd = snd.clone()
    bad = torch.randperm(E, generator=g)[:40]
    snd[bad[:20]] = nnodes + 3
    snd[bad[20:]] = -1
    knots_np, h = np.linspace(1e-12, 6.0, 256, retstep=True)
    knots = torch.from_numpy(knots_np)
    table = torch.cos(knots[:, None] * torch.linspace(0.3, 2.0, 4 * C, dtype=torch.float64)[None, :])
    coeffs = O.spline_coefficients(knots, table).float().double()
    h = float(np.float32(h))
    live = (vec.norm(dim=1).float() <= 5.0) & (snd >= 0) & (snd < nnodes)
    assert 0.3 < float(live.double().mean()) < 0.7

    va = vec[live].clone().requires_grad_(True)
    Xa = X.clone().requires_grad_(True)
    Rv = O.spline_eval(va.norm(dim=1), knots.float().double(), coeffs, h, 5.0).view(-1, 4, C)
    ref = O.mp_forward(Xa, O.spherical_harmonics(va), Rv, snd[live], rcv[live], nnodes)
    (ref * G).sum().backward()

    d = lambda t: t.float().cuda()
    fo = cabi.first_occurences(rcv.cuda(), nnodes)
    perm, off = cabi.stable_key_sort(snd.cuda(), nnodes)
    out = cabi.mp_edge_forward(d(X), d(vec), d(knots), d(coeffs), h, 5.0, snd.cuda(), fo, nnodes)
    gX, gvec = cabi.mp_edge_backward(d(X), d(vec), d(knots), d(coeffs), h, 5.0, d(G), snd.cuda(), fo, perm, off, nnodes)
    close(out, ref.detach(), 2e-5, 2e-6)
    close(gX, Xa.grad, 2e-5, 2e-6)
    close(gvec[live.cuda()], va.grad, 5e-5, 5e-6)
    assert float(gvec[~live.cuda()].abs().max()) == 0.0
    gvec_only = cabi.mp_edge_backward(d(X), d(vec), d(knots), d(coeffs), h, 5.0, d(G), snd.cuda(), fo, perm, off, nnodes,
                                      need_gX=False)[1]
    assert torch.equal(gvec_only, gvec)


# ---- many receiver nodes: the forward from edge vectors runs on the kernel that keeps its part of the table in LDS ----
def _edge_case(nnodes, avg, C, iso, seed, nknots=256, heavy=0):
    """Receiver-sorted random graph with edge vectors of lengths 0.7 .. 5.3 (r_max = 5), a few senders out of range,
    optionally one node with `heavy` extra edges (more edge blocks than the kernel's node sort tells apart)."""
    snd, rcv = random_graph(nnodes, avg, seed, isolated_frac=iso)
    if heavy:
        g0 = torch.Generator().manual_seed(seed + 5)
        node = nnodes // 3
        extra = torch.randint(0, nnodes, (heavy,), generator=g0, dtype=torch.int32)
        at = int(torch.searchsorted(rcv, torch.tensor(node, dtype=torch.int32)))
        snd = torch.cat([snd[:at], extra, snd[at:]])
        rcv = torch.cat([rcv[:at], torch.full((heavy,), node, dtype=torch.int32), rcv[at:]])
    E = snd.numel()
    g = torch.Generator().manual_seed(seed + 100)
    X = torch.randn(nnodes, C, generator=g, dtype=torch.float64)
    r = torch.rand(E, generator=g, dtype=torch.float64) * 4.6 + 0.7
    vec = torch.randn(E, 3, generator=g, dtype=torch.float64)
    vec = (vec / vec.norm(dim=1, keepdim=True) * r[:, None]).float().double()
    snd = snd.clone()
    bad = torch.randperm(E, generator=g)[:30]
    snd[bad[:15]] = nnodes + 5
    snd[bad[15:]] = -1
    knots_np, h = np.linspace(1e-12, 6.0, nknots, retstep=True)
    knots = torch.from_numpy(knots_np)
    table = torch.sin(knots[:, None] * torch.linspace(0.5, 2.5, 4 * C, dtype=torch.float64)[None, :]) * torch.randn(
        1, 4 * C, generator=g, dtype=torch.float64)
    coeffs = O.spline_coefficients(knots, table).float().double()
    return snd, rcv, X, vec, knots.float().double(), coeffs, float(np.float32(h))


MANY_NODES = [
    # nnodes, avg degree, channels, isolated fraction, seed, knots, extra edges of one node
    (2100, 14, 32, 0.1, 0, 256, 0),
    (2300, 9, 64, 0.0, 1, 256, 300),   # one node with more than 63 blocks of four edges
    (2048, 21, 96, 0.05, 2, 200, 0),
    (3000, 6, 160, 0.3, 3, 256, 0),
    (2500, 3, 256, 0.0, 4, 272, 0),    # the largest table the kernel keeps in LDS
]


@pytest.mark.parametrize("case", MANY_NODES, ids=lambda c: "N%d_d%d_C%d_k%d" % (c[0], c[1], c[2], c[5]))
def test_mp_edge_forward_many_nodes(cabi, case):
    """Parity with the fp64 oracle (harmonics, spline, message-passing definition) on the live edges; edges beyond the
    cutoff or with a sender out of range add nothing; nodes without edges come out as zeros; the result is the same
    on a second call (which wave serves a node changes from run to run, the node's result must not)."""
    print("mp_edge_forward many nodes", case, flush=True)
    nnodes, C = case[0], case[2]
    snd, rcv, X, vec, knots, coeffs, h = _edge_case(*case)
    live = (vec.norm(dim=1).float() <= 5.0) & (snd >= 0) & (snd < nnodes)
    Rv = O.spline_eval(vec[live].norm(dim=1), knots, coeffs, h, 5.0).view(-1, 4, C)
    ref = O.mp_forward(X, O.spherical_harmonics(vec[live]), Rv, snd[live], rcv[live], nnodes)
    d = lambda t: t.float().cuda()
    fo = cabi.first_occurences(rcv.cuda(), nnodes)
    out = cabi.mp_edge_forward(d(X), d(vec), d(knots), d(coeffs), h, 5.0, snd.cuda(), fo, nnodes)
    close(out, ref, 2e-5, 2e-6)
    empty = torch.bincount(rcv.long(), minlength=nnodes) == 0
    assert float(out[empty.cuda()].abs().max()) == 0.0 if bool(empty.any()) else True
    again = cabi.mp_edge_forward(d(X), d(vec), d(knots), d(coeffs), h, 5.0, snd.cuda(), fo, nnodes)
    assert torch.equal(out, again)


def test_mp_edge_forward_many_nodes_agrees_with_harmonics_and_lengths_path(cabi):
    """40 000 receiver nodes at 256 channels: a workgroup of the LDS-table kernel sorts and serves its nodes in more than
    one batch.  Checked against the kernel that takes harmonics and lengths (same radial table, same per-edge
    arithmetic, another summation order), and against the oracle on a sample of nodes."""
    nnodes, C = 40000, 256
    snd, rcv, X, vec, knots, coeffs, h = _edge_case(nnodes, 3, C, 0.1, 9)
    d = lambda t: t.float().cuda()
    fo = cabi.first_occurences(rcv.cuda(), nnodes)
    out = cabi.mp_edge_forward(d(X), d(vec), d(knots), d(coeffs), h, 5.0, snd.cuda(), fo, nnodes)
    Y = cabi.sh_forward(d(vec))
    length = d(vec).norm(dim=1)  # rounding of the length may differ from the kernel's in the last bit
    other = cabi.mp_spline_forward(d(X), Y, length, d(knots), d(coeffs), h, 5.0, snd.cuda(), fo, nnodes)
    close(out, other.double().cpu(), 1e-4, 1e-5)
    nodes = torch.arange(0, nnodes, 997)
    pick = torch.isin(rcv.long(), nodes)
    live = pick & (vec.norm(dim=1).float() <= 5.0) & (snd >= 0) & (snd < nnodes)
    Rv = O.spline_eval(vec[live].norm(dim=1), knots, coeffs, h, 5.0).view(-1, 4, C)
    ref = O.mp_forward(X, O.spherical_harmonics(vec[live]), Rv, snd[live], rcv[live], nnodes)
    close(out[nodes.cuda()], ref[nodes], 2e-5, 2e-6)
