"""Writes the golden fixtures in this directory from the fp64 CPU oracle on seeded inputs.

    python tests/golden/make_golden.py

The reference holds no golden vectors for this path (every one of its tests evaluates third-party packages live), and
neither it nor those packages can be imported offline, so these vectors come from the repository's own oracle, whose
functions are pinned by closed forms and library routines in tests/test_oracle_pins.py.  They freeze the oracle's
answers: tests/test_golden.py checks that the oracle still reproduces them (CPU) and that the HIP library matches them
(GPU).  Inputs are stored as float32-representable values so that the fp32 kernels see exactly the stored numbers.

  ops_small.npz   one small case per op: message passing, harmonics, spline, linears, contraction, CSR offsets,
                  stable sort, edge geometry, readout, neighbour list
  model_c1.npz    the 21-atom, 64-channel cluster (random-init weights, seed 0): energy, forces, node energies
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
for p in (ROOT, os.path.join(ROOT, "cuda-mace_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

from oracle import mace_model as M  # noqa: E402
from oracle import ops as O  # noqa: E402
from oracle.u_tensors import u_tensors  # noqa: E402
from tests.util import random_graph  # noqa: E402


def f32(t: torch.Tensor) -> torch.Tensor:
    """Rounds to the nearest float32, kept in float64."""
    return t.float().double()


def ops_inputs():
    """Seeded inputs of every op case (float64 tensors holding float32-representable values; int32 indices)."""
    g = torch.Generator().manual_seed(2024)
    rn = lambda *s: f32(torch.randn(*s, generator=g, dtype=torch.float64))
    d = {}
    # message passing: 12 nodes (two without edges), 32 channels
    nn, C = 12, 32
    snd, rcv = random_graph(nn, 5, 7, isolated_frac=0.15)
    E = snd.numel()
    d.update(mp_sender=snd, mp_receiver=rcv, mp_X=rn(nn, C), mp_vec=rn(E, 3), mp_R=rn(E, 4, C), mp_G=rn(nn, 16, C))
    # harmonics
    d.update(sh_xyz=rn(48, 3) * 2.0, sh_G=rn(16, 48))
    # spline: 24 knots on [1e-12, 6], 8 outputs, radii partly beyond r_max = 5
    knots = torch.linspace(1e-12, 6.0, 24, dtype=torch.float64)
    table = f32(torch.sin(knots[:, None] * torch.linspace(0.3, 2.0, 8, dtype=torch.float64)[None, :]))
    d.update(sp_knots=knots, sp_table=table, sp_r=f32(torch.rand(40, generator=g, dtype=torch.float64) * 5.6 + 0.3),
             sp_G=rn(40, 8))
    # linears: K = 32, three elements, one row that names no element
    ne = 3
    elem = torch.tensor([0, 2, 1, 3, 0, 1, 2], dtype=torch.int64)
    d.update(lin_X=rn(7, 16, C), lin_W=rn(4, C, C), lin_We=rn(ne, 4, C, C), lin_elem=elem.int(), lin_G=rn(7, 16, C))
    # contraction with the real l_max = 3 coupling tensors
    d.update(sc_X=rn(6, 16, C) * 0.8, sc_types=torch.tensor([0, 1, 1, 0, 1, 0], dtype=torch.int32), sc_W3=rn(2, 23, C),
             sc_W2=rn(2, 4, C), sc_W1=rn(2, 1, C), sc_G=rn(6, C))
    # index kernels
    d.update(idx_receiver=torch.tensor([0, 0, 2, 2, 2, 5, 7, 7], dtype=torch.int32),
             idx_keys=torch.tensor([3, 1, 3, 0, 1, 1, 4, 0, 3], dtype=torch.int32))
    # edge geometry on the message-passing graph
    d.update(geo_pos=torch.randn(nn, 3, generator=g, dtype=torch.float64) * 3.0,
             geo_shifts=torch.randn(E, 3, generator=g, dtype=torch.float64).round() * 4.0, geo_Gv=rn(E, 3), geo_Gl=rn(E))
    # readout
    d.update(ro_h1=rn(9, C), ro_h2=rn(9, C), ro_w1=torch.randn(C, generator=g, dtype=torch.float64) / C ** 0.5,
             ro_W2a=torch.randn(C, 16, generator=g, dtype=torch.float64) / C ** 0.5,
             ro_w2b=torch.randn(16, generator=g, dtype=torch.float64) / 4.0)
    # neighbour list: 30 atoms in a triclinic cell, periodic along two axes, some atoms outside the cell
    cell = torch.tensor([[7.0, 0.0, 0.0], [1.5, 6.5, 0.0], [0.5, -1.0, 8.0]], dtype=torch.float64)
    frac = torch.rand(30, 3, generator=g, dtype=torch.float64) * 1.4 - 0.2
    d.update(nl_cell=cell, nl_pos=frac @ cell)
    return d


NL_PBC = (True, True, False)
NL_CUTOFF = 3.5
RO_CONST = dict(act_cst=1.6791767923989418, scale=0.8, shift=-0.3)
SP_RMAX = 5.0


def ops_outputs(d):
    """Everything the oracle computes from ops_inputs()."""
    o = {}
    nn = d["mp_X"].shape[0]
    Y = O.spherical_harmonics(d["mp_vec"]).contiguous()
    o["mp_out"] = O.mp_forward(d["mp_X"], Y, d["mp_R"], d["mp_sender"], d["mp_receiver"], nn)
    o["mp_gX"], o["mp_gY"], o["mp_gR"] = O.mp_backward(d["mp_X"], Y, d["mp_R"], d["mp_G"], d["mp_sender"], d["mp_receiver"])
    o["sh_Y"] = O.spherical_harmonics(d["sh_xyz"])
    o["sh_gxyz"] = O.spherical_harmonics_backward(d["sh_xyz"], d["sh_G"])
    h = float(d["sp_knots"][1] - d["sp_knots"][0])
    o["sp_coeffs"] = O.spline_coefficients(d["sp_knots"], d["sp_table"])
    o["sp_val"], o["sp_der"] = O.spline_eval(d["sp_r"], d["sp_knots"], o["sp_coeffs"], h, SP_RMAX, deriv=True)
    o["sp_gr"] = O.spline_backward(d["sp_G"], o["sp_der"])
    X = d["lin_X"].clone().requires_grad_(True)
    out = O.linear(X, d["lin_W"])
    (out * d["lin_G"]).sum().backward()
    o["lin_out"], o["lin_gX"] = out.detach(), X.grad.clone()
    one_hot = torch.nn.functional.one_hot(d["lin_elem"].long(), 4)[:, :3].double()
    X = d["lin_X"].clone().requires_grad_(True)
    out = O.elemental_linear(X, d["lin_We"], one_hot)
    (out * d["lin_G"]).sum().backward()
    o["lin_e_out"], o["lin_e_gX"] = out.detach(), X.grad.clone()
    _, U2, U3 = (torch.from_numpy(u) for u in u_tensors())
    X = d["sc_X"].clone().requires_grad_(True)
    out = O.symmetric_contraction(X, d["sc_types"], U3, U2, d["sc_W3"], d["sc_W2"], d["sc_W1"])
    (out * d["sc_G"]).sum().backward()
    o["sc_out"], o["sc_gX"] = out.detach(), X.grad.clone()
    o["idx_first_occ"] = O.first_occurences(d["idx_receiver"], 9)
    o["idx_perm"], o["idx_offsets"] = O.stable_key_sort(d["idx_keys"], 5)
    pos = d["geo_pos"].clone().requires_grad_(True)
    vec, length = O.edge_geometry(pos, d["mp_receiver"], d["mp_sender"], d["geo_shifts"])
    ((vec * d["geo_Gv"]).sum() + (length * d["geo_Gl"]).sum()).backward()
    o["geo_vec"], o["geo_len"], o["geo_gpos"] = vec.detach(), length.detach(), pos.grad.clone()
    o["ro_e"] = O.readout_energies(d["ro_h1"], d["ro_h2"], d["ro_w1"], d["ro_W2a"], d["ro_w2b"], RO_CONST["act_cst"],
                                   RO_CONST["scale"], RO_CONST["shift"])
    ei, us = O.neighbour_list(d["nl_pos"].numpy(), d["nl_cell"].numpy(), NL_PBC, NL_CUTOFF)
    o["nl_edge_index"], o["nl_unit_shifts"] = torch.from_numpy(ei), torch.from_numpy(us)
    return o


def model_case():
    """Benchmark configuration 1: the 21-atom {H, C, N, O} cluster in an 8 A cube, 64 channels, weights from seed 0."""
    from cuda_mace.models import SyntheticInvariantMACE
    from cuda_mace.utils.synthetic import make_system

    data = make_system(21, 4, seed=0, density=None, cluster_box=8.0)
    avg = data["edge_index"].shape[1] / 21
    up = SyntheticInvariantMACE(channels=64, atomic_numbers=(1, 6, 7, 8), avg_num_neighbors=avg, seed=0)
    return data, up


def model_outputs(data, up):
    ref = M.energy_and_forces(up.export_params(), data)
    return {k: ref[k].detach() for k in ("energy", "interaction_energy", "node_energy", "forces")}


def _compact(t: torch.Tensor) -> np.ndarray:
    """float64 data that is exactly representable in float32 is stored as float32."""
    if t.dtype == torch.float64 and bool((t.float().double() == t).all()):
        return t.float().numpy()
    return t.numpy()


def load(name: str):
    """{key: tensor} of a fixture; floating-point arrays come back as float64."""
    with np.load(os.path.join(HERE, name)) as z:
        out = {k: torch.from_numpy(z[k]) for k in z.files}
    return {k: (v.double() if v.dtype == torch.float32 else v) for k, v in out.items()}


def main():
    d = ops_inputs()
    o = ops_outputs(d)
    np.savez_compressed(os.path.join(HERE, "ops_small.npz"), **{"in_" + k: _compact(v) for k, v in d.items()},
                        **{"out_" + k: v.numpy() for k, v in o.items()})
    data, up = model_case()
    out = model_outputs(data, up)
    np.savez_compressed(os.path.join(HERE, "model_c1.npz"), positions=data["positions"].numpy(),
                        node_attrs=data["node_attrs"].numpy(), edge_index=data["edge_index"].numpy(),
                        **{"out_" + k: v.numpy() for k, v in out.items()})
    for name in ("ops_small.npz", "model_c1.npz"):
        print(name, os.path.getsize(os.path.join(HERE, name)), "bytes")


if __name__ == "__main__":
    main()
