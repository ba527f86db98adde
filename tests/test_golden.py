"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py from the fp64 oracle).

CPU: the oracle still reproduces every stored vector from the stored inputs, and the input generator is stable.
GPU: the HIP library matches the stored vectors through the C ABI (bit-exact for index work, fp32 tolerances otherwise),
and the optimised model matches the stored energy and forces of the 21-atom cluster.
"""
import numpy as np
import pytest
import torch

from tests.golden import make_golden as G
from tests.util import close

DEV = "cuda"


def _split(fix):
    d = {k[3:]: v for k, v in fix.items() if k.startswith("in_")}
    o = {k[4:]: v for k, v in fix.items() if k.startswith("out_")}
    return d, o


def test_oracle_reproduces_ops_fixture():
    d, want = _split(G.load("ops_small.npz"))
    fresh = G.ops_inputs()
    assert set(fresh) == set(d)
    for k in d:  # the seeded generator still yields the stored inputs (matrix products may differ in the last bit per host)
        if d[k].is_floating_point():
            torch.testing.assert_close(fresh[k].double(), d[k], rtol=1e-13, atol=1e-13, msg=k)
        else:
            assert torch.equal(fresh[k], d[k]), k
    got = G.ops_outputs(d)
    assert set(got) == set(want)
    for k, v in got.items():
        if v.is_floating_point():
            torch.testing.assert_close(v, want[k], rtol=1e-12, atol=1e-13 * max(1.0, float(want[k].abs().max())), msg=k)
        else:
            assert torch.equal(v, want[k]), k


def test_oracle_reproduces_model_fixture():
    fix = G.load("model_c1.npz")
    data, up = G.model_case()
    assert torch.equal(data["positions"], fix["positions"]) and torch.equal(data["edge_index"], fix["edge_index"])
    got = G.model_outputs(data, up)
    for k, v in got.items():
        torch.testing.assert_close(v, fix["out_" + k], rtol=1e-10, atol=1e-12, msg=k)


@pytest.mark.gpu
def test_hip_library_matches_ops_fixture(cabi):
    d, want = _split(G.load("ops_small.npz"))
    f = lambda t: t.float().to(DEV)
    dev = lambda t: t.to(DEV)
    # index kernels: bit-exact
    assert torch.equal(cabi.first_occurences(dev(d["idx_receiver"]), 9).cpu(), want["idx_first_occ"])
    perm, off = cabi.stable_key_sort(dev(d["idx_keys"]), 5)
    assert torch.equal(perm.cpu(), want["idx_perm"]) and torch.equal(off.cpu(), want["idx_offsets"])
    # harmonics
    close(cabi.sh_forward(f(d["sh_xyz"])), want["sh_Y"], 1e-5, 2e-6)
    close(cabi.sh_backward(f(d["sh_xyz"]), f(d["sh_G"])), want["sh_gxyz"], 2e-5, 2e-6)
    # message passing (harmonics of the stored vectors from the library itself)
    nn = d["mp_X"].shape[0]
    snd, rcv = dev(d["mp_sender"]), dev(d["mp_receiver"])
    Y = cabi.sh_forward(f(d["mp_vec"]))
    fo = cabi.first_occurences(rcv, nn)
    perm, off = cabi.stable_key_sort(snd, nn)
    close(cabi.mp_forward(f(d["mp_X"]), Y, f(d["mp_R"]), snd, fo, nn), want["mp_out"], 2e-5, 2e-6)
    gX, gY, gR = cabi.mp_backward(f(d["mp_X"]), Y, f(d["mp_R"]), f(d["mp_G"]), snd, fo, perm, off, nn)
    close(gX, want["mp_gX"], 2e-5, 2e-6), close(gY, want["mp_gY"], 2e-5, 2e-6), close(gR, want["mp_gR"], 2e-5, 2e-6)
    # ... and in double
    Y64 = cabi.sh_forward(dev(d["mp_vec"]))
    close(cabi.mp_forward(dev(d["mp_X"]), Y64, dev(d["mp_R"]), snd, fo, nn), want["mp_out"], 1e-12, 1e-13)
    # spline
    h = float(d["sp_knots"][1] - d["sp_knots"][0])
    val, der = cabi.spline_forward(f(d["sp_r"]), f(d["sp_knots"]), f(want["sp_coeffs"]), h, G.SP_RMAX, want_deriv=True)
    close(val, want["sp_val"], 2e-5, 2e-6), close(der, want["sp_der"], 2e-5, 5e-6)
    gr = cabi.spline_backward(f(d["sp_r"]), f(d["sp_knots"]), f(want["sp_coeffs"]), f(d["sp_G"]), h, G.SP_RMAX)
    bound = 4e-6 * (d["sp_G"].abs() * want["sp_der"].abs()).sum(-1) + 1e-30
    assert bool(((gr.double().cpu() - want["sp_gr"]).abs() <= bound).all())
    val64 = cabi.spline_forward(dev(d["sp_r"]), dev(d["sp_knots"]), dev(want["sp_coeffs"]), h, G.SP_RMAX)
    close(val64, want["sp_val"], 1e-12, 1e-13)
    # linears: forward with the transposed blocks, backward with the blocks themselves
    WT = f(d["lin_W"].transpose(-1, -2).contiguous())
    close(cabi.linear(f(d["lin_X"]), WT), want["lin_out"], 1e-5, 2e-6)
    close(cabi.linear(f(d["lin_G"]), f(d["lin_W"])), want["lin_gX"], 1e-5, 2e-6)
    eperm, eoff = cabi.stable_key_sort(dev(d["lin_elem"]), 4)
    WeT = f(d["lin_We"].transpose(-1, -2).contiguous())
    out = cabi.linear(f(d["lin_X"]), WeT, eperm, eoff, zero_last_group=True)
    close(out, want["lin_e_out"], 1e-5, 2e-6)
    close(cabi.linear(f(d["lin_G"]), f(d["lin_We"]), eperm, eoff, zero_last_group=True), want["lin_e_gX"], 1e-5, 2e-6)
    # edge geometry
    E = d["mp_sender"].numel()
    vec, length = cabi.edge_geometry_forward(dev(d["geo_pos"]), rcv, snd, dev(d["geo_shifts"]))
    close(vec, want["geo_vec"], 1e-6, 1e-7), close(length, want["geo_len"], 1e-6, 1e-7)
    gpos, _ = cabi.edge_geometry_backward(dev(d["geo_pos"]), rcv, snd, dev(d["geo_shifts"]), fo, perm, off, f(d["geo_Gv"]),
                                          f(d["geo_Gl"]))
    close(gpos, want["geo_gpos"], 2e-5, 2e-6)
    assert vec.shape == (E, 3)
    # readout
    e, _, _ = cabi.readout_forward(f(d["ro_h1"]), f(d["ro_h2"]), dev(d["ro_w1"]), dev(d["ro_W2a"]), dev(d["ro_w2b"]),
                                   G.RO_CONST["act_cst"], G.RO_CONST["scale"], G.RO_CONST["shift"])
    close(e, want["ro_e"], 1e-12, 1e-13)
    # neighbour list: identical integers
    ri, rj, us = cabi.neighbour_list(dev(d["nl_pos"]), dev(d["nl_cell"]), G.NL_PBC, G.NL_CUTOFF)
    assert torch.equal(torch.stack((ri, rj)).cpu().long(), want["nl_edge_index"])
    assert torch.equal(us.cpu().long(), want["nl_unit_shifts"])


@pytest.mark.gpu
def test_symmetric_contraction_matches_fixture(cabi):
    """The op module on the stored weights (real l_max = 3 coupling tensors) against the stored value and gradient."""
    from cuda_mace.models.upstream_like import _SymmetricContraction
    from cuda_mace.ops.symmetric_contraction import SymmetricContraction

    d, want = _split(G.load("ops_small.npz"))
    up = _SymmetricContraction(32, 2, torch.Generator().manual_seed(0))
    con = up.contractions[0]
    with torch.no_grad():
        con.weights_max.copy_(d["sc_W3"]), con.weights[0].copy_(d["sc_W2"]), con.weights[1].copy_(d["sc_W1"])
    mod = SymmetricContraction(up, device=DEV)
    x = d["sc_X"].float().to(DEV).requires_grad_(True)
    out = mod(x, d["sc_types"].to(DEV)).squeeze(1)
    (out * d["sc_G"].float().to(DEV)).sum().backward()
    close(out.detach(), want["sc_out"], 3e-5, 3e-6)
    close(x.grad, want["sc_gX"], 3e-5, 3e-6)


@pytest.mark.gpu
def test_model_matches_fixture(cabi):
    from cuda_mace.models import OptimizedInvariantMACE
    from cuda_mace.utils.synthetic import to_device

    fix = G.load("model_c1.npz")
    data, up = G.model_case()
    model = OptimizedInvariantMACE(up, device=DEV)
    out = model(to_device(data, DEV))
    e, e_ref = float(out["energy"].detach().sum()), float(fix["out_energy"].sum())
    assert abs(e - e_ref) <= 1e-5 * abs(e_ref)
    assert float((out["forces"].double().cpu() - fix["out_forces"]).abs().max()) <= 1e-4
    torch.testing.assert_close(out["node_energy"].double().cpu(), fix["out_node_energy"], rtol=1e-4,
                               atol=1e-5 * float(fix["out_node_energy"].abs().max()))
