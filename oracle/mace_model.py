"""fp64 CPU restatement of the upstream invariant MACE energy + forces path.  TEST INFRASTRUCTURE ONLY
(and the CPU-baseline leg of the benchmark).

The reference accelerates an upstream `mace` (0.3.x) ScaleShiftMACE with hidden irreps Cx0e, l_max = 3,
correlation 3 and two interaction layers, and takes that upstream model as its own accuracy reference
(tools/model_surgery.py:66-143).  Upstream mace/e3nn are third-party packages that are not available
offline; this file states the same forward pass from the weights alone (plain tensors in `params`), the way
upstream evaluates it: gather -> per-edge tensor product [E, 16, C] -> scatter-sum over receivers, exact
radial MLP (no spline), dense nested contraction, autograd forces.  Data flow and normalisations follow
the reference's own use of the upstream modules (models/InvariantMACE.py:41-53, 56-74, 226-240, 287-347).

Conventions: upstream's, i.e. sender = edge_index[0], receiver = edge_index[1], edge vector =
pos[receiver] - pos[sender] + shift.  The reference swaps sender and receiver (models/InvariantMACE.py:99-100),
which flips the sign of odd-l message components and leaves energies and forces unchanged.

Equality with upstream mace on a trained checkpoint is PARITY UNPINNED (upstream unavailable offline).
What pins this file (tests/test_oracle_model.py): message passing, per-l / per-element linears and readouts are the
op definitions of oracle/ops.py (each pinned there); Bessel orthonormality by quadrature; the envelope's boundary
conditions; the activation constant by Gauss-Hermite quadrature; the 1/sqrt(fan_in) convention by the unit second
moment of the radial network's output; the nested contraction against the brute-force-pinned dense form; invariances
and F = -dE/dx finite differences of the whole.
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch

from . import ops as O
from .u_tensors import u_tensors

SILU_2MOM = 1.6791767923989418


def bessel_basis(r: torch.Tensor, r_max: float, num_bessel: int) -> torch.Tensor:
    """[E] -> [E, num_bessel]: b_n(r) = sqrt(2 / r_max) sin(n pi r / r_max) / r, n = 1..num_bessel; orthonormal on
    [0, r_max] under the measure r^2 dr (pinned by quadrature in tests/test_oracle_model.py)."""
    n = torch.arange(1, num_bessel + 1, dtype=r.dtype)
    return math.sqrt(2.0 / r_max) * torch.sin(n * math.pi / r_max * r[:, None]) / r[:, None]


def polynomial_cutoff(x: torch.Tensor, p: int) -> torch.Tensor:
    """Envelope f(x) = 1 - (p+1)(p+2)/2 x^p + p(p+2) x^(p+1) - p(p+1)/2 x^(p+2) for x < 1, else 0: the polynomial
    of that shape with f(0) = 1 and f(1) = f'(1) = f''(1) = 0 (those four conditions fix the three coefficients;
    pinned in tests/test_oracle_model.py)."""
    env = 1.0 - (p + 1) * (p + 2) / 2.0 * x ** p + p * (p + 2.0) * x ** (p + 1) - p * (p + 1) / 2.0 * x ** (p + 2)
    return env * (x < 1.0).to(x.dtype)


def radial_basis(r: torch.Tensor, r_max: float, num_bessel: int, p: int) -> torch.Tensor:
    """[E] -> [E, num_bessel]: Bessel functions times the polynomial cutoff envelope."""
    return bessel_basis(r, r_max, num_bessel) * polynomial_cutoff(r / r_max, p)[:, None]


def radial_mlp(feats: torch.Tensor, weights) -> torch.Tensor:
    z = feats
    for i, W in enumerate(weights):
        z = z @ W.to(z.dtype) / math.sqrt(W.shape[0])
        if i + 1 < len(weights):
            z = SILU_2MOM * torch.nn.functional.silu(z)
    return z


def contraction_nested(X, elem, W3, W2, W1, U3, U2):
    """out[n, c] = sum_i x_i (U1W1_i + sum_j x_j (U2W2_ij + sum_k U3W3_ijk x_k)), evaluated element by element."""
    out = torch.zeros(X.shape[0], X.shape[2], dtype=X.dtype)
    for e in torch.unique(elem).tolist():
        idx = torch.nonzero(elem == e).squeeze(1)
        xe = X[idx]
        c3 = torch.einsum("ijkp,pc->ijkc", U3, W3[e].to(X.dtype))
        c2 = torch.einsum("ijp,pc->ijc", U2, W2[e].to(X.dtype))
        t = torch.einsum("ijkc,nkc->nijc", c3, xe) + c2[None]
        t = torch.einsum("nijc,njc->nic", t, xe)
        t[:, 0, :] = t[:, 0, :] + W1[e, 0].to(X.dtype)
        out = out.index_add(0, idx, torch.einsum("nic,nic->nc", t, xe))
    return out


def energy_and_forces(params: Dict[str, object], data: Dict[str, torch.Tensor], dtype=torch.float64,
                      compute_forces: bool = True, edge_chunk: Optional[int] = None,
                      node_weights: Optional[torch.Tensor] = None):
    """Returns dict(energy [1], interaction_energy [1], node_energy [N], forces [N, 3], node_feats [N, 2C]).
    With node_weights [N] the forces are minus the gradient of sum_n node_weights[n] * node_energy[n] (what a rank of
    a domain-decomposed MD code reports: weight 1 for its own atoms, 0 for ghosts); energies are unweighted."""
    C = int(params["channels"])
    ne = int(params["num_elements"])
    pos = data["positions"].detach().to(dtype).clone().requires_grad_(compute_forces)
    attrs = data["node_attrs"].to(dtype)
    elem = attrs.argmax(dim=1)
    snd, rcv = data["edge_index"][0], data["edge_index"][1]
    N = pos.shape[0]
    U1, U2, U3 = (torch.from_numpy(u).to(dtype) for u in u_tensors())

    vec = pos[rcv] - pos[snd] + data["shifts"].to(dtype)
    r = vec.norm(dim=1)
    Y = O.spherical_harmonics(vec).t()  # [E, 16]
    basis = radial_basis(r, float(params["r_max"]), int(params["num_bessel"]), int(params["p"]))

    node_e0 = attrs @ params["E0"].to(dtype)
    h = attrs @ params["W_emb"].to(dtype) / math.sqrt(ne)
    feats = []
    for t, lay in enumerate(params["layers"]):
        sc = None
        if t == 1:
            sc = torch.einsum("nu,ne,uew->nw", h, attrs, lay["W_skip"][0].to(dtype)) / math.sqrt(C * ne)
        u = h @ lay["W_up"].to(dtype) / math.sqrt(C)
        R = radial_mlp(basis, lay["mlp"]).view(-1, 4, C)
        # per-edge tensor product and scatter-sum over receivers: the op definition pinned in oracle/ops.py
        A = O.mp_forward(u, Y.t(), R, snd, rcv, N)
        A = O.linear(A, lay["W_lin"].to(dtype)) / float(lay["avg_num_neighbors"])
        if t == 0:
            # per-element linear: blocks W_skip[l][:, e, :] with 1/sqrt(ne) folded in (models/InvariantMACE.py:61-64),
            # 1/sqrt(C) applied by the op
            Wsk = lay["W_skip"].to(dtype).permute(2, 0, 1, 3) / math.sqrt(ne)  # [ne, 4, C, C]
            A = O.elemental_linear(A, Wsk, attrs)
        # a layer may name the coupling basis its weights refer to; otherwise the oracle's own derivation
        U3l = lay["U3"].to(dtype) if "U3" in lay else U3
        U2l = lay["U2"].to(dtype) if "U2" in lay else U2
        B = contraction_nested(A, elem, lay["W3"], lay["W2"], lay["W1"], U3l, U2l)
        h = B @ lay["W_prod"].to(dtype) / math.sqrt(C)
        if sc is not None:
            h = h + sc
        feats.append(h)
    hidden = params["W_read1"].shape[1]
    node_inter = O.readout_energies(feats[0], feats[1], params["w_read0"].to(dtype)[:, 0] / math.sqrt(C),
                                    params["W_read1"].to(dtype) / math.sqrt(C),
                                    params["w_read2"].to(dtype)[:, 0] / math.sqrt(hidden), SILU_2MOM,
                                    float(params["scale"]), float(params["shift"]))
    inter_e = node_inter.sum().view(1)
    forces = None
    if compute_forces:
        seeded = inter_e.sum() if node_weights is None else (node_inter * node_weights.to(dtype)).sum()
        (g,) = torch.autograd.grad(seeded, pos)
        forces = -g
    return dict(energy=(node_e0.sum() + inter_e).detach(), interaction_energy=inter_e.detach(),
                node_energy=(node_e0 + node_inter).detach(), forces=forces,
                node_feats=torch.cat(feats, dim=1).detach())
