"""A randomly initialised invariant-MACE model object with the attribute tree of an upstream model.

`OptimizedInvariantMACE(mace_model)` reads weights and sub-modules from an upstream `mace`
ScaleShiftMACE (reference models/InvariantMACE.py:168-244).  Upstream `mace`/`e3nn` are not
dependencies of this package; this file provides plain-torch blocks with the same attributes and
call signatures, so that a model with random weights (or weights copied from elsewhere) can be
handed to `OptimizedInvariantMACE`.  A genuine upstream model object works the same way.

Architecture (mace 0.3.x ScaleShiftMACE, invariant case): hidden `Cx0e`, l_max = 3, correlation 3, two
interaction layers (RealAgnosticInteractionBlock, then RealAgnosticResidualInteractionBlock), Bessel basis
with polynomial cutoff, radial MLP [64, 64, 64] with silu, linear and non-linear (16x0e) readouts.
Every linear map divides by sqrt(fan_in) (e3nn convention), activations are scaled to unit second moment.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

from ..utils.irreps import Instruction, Irreps

SILU_2MOM = 1.6791767923989418  # 1 / sqrt(E[silu(z)^2]), z ~ N(0, 1)


class _Linear0e(torch.nn.Module):
    """o3.Linear between scalar blocks: y = x @ W / sqrt(fan_in); `weight` is stored flat like e3nn does."""

    def __init__(self, n_in: int, n_out: int, generator: torch.Generator):
        super().__init__()
        self.irreps_in = Irreps("%dx0e" % n_in)
        self.irreps_out = Irreps("%dx0e" % n_out)
        self.weight = torch.nn.Parameter(torch.randn(n_in * n_out, generator=generator, dtype=torch.float64))
        self.n_in, self.n_out = n_in, n_out

    def forward(self, x):
        return x @ self.weight.view(self.n_in, self.n_out).to(x.dtype) / math.sqrt(self.n_in)


class _LinearPerL(torch.nn.Module):
    """o3.Linear  Cx0e+Cx1o+Cx2e+Cx3o -> same: one [C, C] block per l, flat weight in instruction order."""

    def __init__(self, channels: int, generator: torch.Generator):
        super().__init__()
        spec = "+".join("%dx%d%s" % (channels, l, "eo"[l % 2]) for l in range(4))
        self.irreps_in = Irreps(spec)
        self.irreps_out = Irreps(spec)
        self.instructions = [Instruction(l, l, (channels, channels), 1.0 / math.sqrt(channels)) for l in range(4)]
        self.weight = torch.nn.Parameter(torch.randn(4 * channels * channels, generator=generator, dtype=torch.float64))


class _SkipTP(torch.nn.Module):
    """o3.FullyConnectedTensorProduct(irreps_in1, ne x 0e -> irreps_out): per l a weight [C, ne, C];
    out[n, w] = sum_{u, e} x[n, u] attrs[n, e] W[u, e, w] / sqrt(C * ne).  Callable for scalar features."""

    def __init__(self, channels: int, num_elements: int, lmax: int, generator: torch.Generator):
        super().__init__()
        spec = "+".join("%dx%d%s" % (channels, l, "eo"[l % 2]) for l in range(lmax + 1))
        self.irreps_in1 = Irreps(spec)
        self.irreps_in2 = Irreps("%dx0e" % num_elements)
        self.irreps_out = Irreps(spec)
        self.channels, self.num_elements, self.lmax = channels, num_elements, lmax
        self.weight = torch.nn.Parameter(
            torch.randn((lmax + 1) * channels * num_elements * channels, generator=generator, dtype=torch.float64))

    def forward(self, node_feats, node_attrs):
        assert self.lmax == 0, "only the scalar skip connection is evaluated through this module"
        W = self.weight.view(self.channels, self.num_elements, self.channels).to(node_feats.dtype)
        return torch.einsum("nu,ne,uew->nw", node_feats, node_attrs.to(node_feats.dtype), W) / math.sqrt(
            self.channels * self.num_elements)


class _RadialMLP(torch.nn.Module):
    """e3nn nn.FullyConnectedNet([num_bessel, 64, 64, 64, 4C], silu): z <- act(z @ W / sqrt(fan_in)),
    act = SILU_2MOM * silu, last layer linear."""

    def __init__(self, sizes: List[int], generator: torch.Generator):
        super().__init__()
        self.weights = torch.nn.ParameterList(
            [torch.nn.Parameter(torch.randn(a, b, generator=generator, dtype=torch.float64)) for a, b in zip(sizes[:-1], sizes[1:])])

    def forward(self, x):
        for i, W in enumerate(self.weights):
            x = x @ W.to(x.dtype) / math.sqrt(W.shape[0])
            if i + 1 < len(self.weights):
                x = SILU_2MOM * torch.nn.functional.silu(x)
        return x


class _RadialEmbedding(torch.nn.Module):
    """Bessel basis sqrt(2/r_max) sin(n pi r / r_max) / r, n = 1..num_bessel, times the polynomial cutoff
    1 - (p+1)(p+2)/2 x^p + p(p+2) x^(p+1) - p(p+1)/2 x^(p+2), x = r / r_max (zero beyond r_max)."""

    def __init__(self, r_max: float, num_bessel: int, p: int):
        super().__init__()
        self.r_max, self.p = float(r_max), int(p)
        self.register_buffer("bessel_weights", math.pi / r_max * torch.arange(1, num_bessel + 1, dtype=torch.float64))
        self.out_dim = num_bessel

    def forward(self, edge_lengths, node_attrs=None, edge_index=None, atomic_numbers=None):
        r = edge_lengths  # [E, 1]
        bessel = math.sqrt(2.0 / self.r_max) * torch.sin(self.bessel_weights.to(r.dtype) * r) / r
        x = r / self.r_max
        p = float(self.p)
        env = (1.0 - (p + 1) * (p + 2) / 2 * x ** self.p + p * (p + 2) * x ** (self.p + 1) - p * (p + 1) / 2 * x ** (self.p + 2))
        return bessel * (env * (x < 1.0).to(r.dtype))


class _NodeEmbedding(_Linear0e):
    pass


class _AtomicEnergies(torch.nn.Module):
    def __init__(self, energies: torch.Tensor):
        super().__init__()
        self.register_buffer("atomic_energies", energies.double().view(1, -1))  # [heads = 1, ne]

    def forward(self, x):
        return x @ self.atomic_energies.to(x.dtype).t()  # [N, heads]


class _LinearReadout(torch.nn.Module):
    def __init__(self, channels: int, generator: torch.Generator):
        super().__init__()
        self.linear = _Linear0e(channels, 1, generator)

    def forward(self, x, heads=None):
        return self.linear(x)


class _Normalize2Mom(torch.nn.Module):
    """f scaled to unit second moment under a standard normal input (what e3nn's normalize2mom wraps a gate in)."""

    def __init__(self, f, cst: float):
        super().__init__()
        self.f = f
        self.cst = float(cst)

    def forward(self, x):
        return self.cst * self.f(x)


class _Activation(torch.nn.Module):
    """Gate on scalar features, holding its functions in `acts` like e3nn's nn.Activation."""

    def __init__(self):
        super().__init__()
        self.acts = torch.nn.ModuleList([_Normalize2Mom(torch.nn.functional.silu, SILU_2MOM)])

    def forward(self, x):
        return self.acts[0](x)


class _NonLinearReadout(torch.nn.Module):
    def __init__(self, channels: int, hidden: int, generator: torch.Generator):
        super().__init__()
        self.linear_1 = _Linear0e(channels, hidden, generator)
        self.non_linearity = _Activation()
        self.linear_2 = _Linear0e(hidden, 1, generator)

    def forward(self, x, heads=None):
        return self.linear_2(self.non_linearity(self.linear_1(x)))


class _ScaleShift(torch.nn.Module):
    def __init__(self, scale: float, shift: float):
        super().__init__()
        self.register_buffer("scale", torch.tensor([scale], dtype=torch.float64))
        self.register_buffer("shift", torch.tensor([shift], dtype=torch.float64))

    def forward(self, x, head=None):
        return self.scale.to(x.dtype) * x + self.shift.to(x.dtype)


class _Contraction(torch.nn.Module):
    """Weight holder of one output irrep: weights_max [ne, 23, C] (order 3), weights = [[ne, 4, C], [ne, 1, C]]."""

    def __init__(self, num_elements: int, channels: int, generator: torch.Generator, coupling=None):
        super().__init__()
        if coupling is not None:
            # upstream's contraction modules keep the coupling tensors their weights refer to as buffers of these names
            for nu, U in zip((1, 2, 3), coupling):
                self.register_buffer("U_matrix_%d" % nu, U.clone())
        self.weights_max = torch.nn.Parameter(torch.randn(num_elements, 23, channels, generator=generator, dtype=torch.float64) / 23)
        self.weights = torch.nn.ParameterList([
            torch.nn.Parameter(torch.randn(num_elements, 4, channels, generator=generator, dtype=torch.float64) / 4),
            torch.nn.Parameter(torch.randn(num_elements, 1, channels, generator=generator, dtype=torch.float64)),
        ])


def permuted_coupling_basis(seed: int):
    """(U1, U2, U3) of ops/u_matrix.py with the paths of U2 and U3 in a seeded random order and with seeded random
    signs: another valid basis of the same invariants, as a model trained elsewhere may carry."""
    import numpy as np

    from ..ops.u_matrix import _u_tensors_np

    U1, U2, U3 = _u_tensors_np()
    rng = np.random.default_rng(seed)
    out = [torch.from_numpy(U1.copy())]
    for U in (U2, U3):
        order = rng.permutation(U.shape[-1])
        signs = rng.choice(np.array([-1.0, 1.0]), size=U.shape[-1])
        out.append(torch.from_numpy(U[..., order] * signs))
    return tuple(out)


class _SymmetricContraction(torch.nn.Module):
    def __init__(self, channels: int, num_elements: int, generator: torch.Generator, coupling=None):
        super().__init__()
        self.irreps_in = Irreps("+".join("%dx%d%s" % (channels, l, "eo"[l % 2]) for l in range(4)))
        self.irreps_out = Irreps("%dx0e" % channels)
        self.contractions = torch.nn.ModuleList([_Contraction(num_elements, channels, generator, coupling)])


class _ProductBasis(torch.nn.Module):
    """EquivariantProductBasisBlock: symmetric contraction, linear, optional residual."""

    def __init__(self, channels: int, num_elements: int, use_sc: bool, generator: torch.Generator, coupling=None):
        super().__init__()
        self.symmetric_contractions = _SymmetricContraction(channels, num_elements, generator, coupling)
        self.linear = _Linear0e(channels, channels, generator)
        self.use_sc = use_sc

    def forward(self, node_feats, sc, node_attrs):
        node_feats = self.symmetric_contractions(node_feats, node_attrs)
        if self.use_sc and sc is not None:
            return self.linear(node_feats) + sc
        return self.linear(node_feats)


class _Interaction(torch.nn.Module):
    def __init__(self, channels: int, num_elements: int, num_bessel: int, radial_mlp: List[int], residual: bool,
                 avg_num_neighbors: float, generator: torch.Generator):
        super().__init__()
        self.linear_up = _Linear0e(channels, channels, generator)
        self.conv_tp_weights = _RadialMLP([num_bessel] + list(radial_mlp) + [4 * channels], generator)
        self.linear = _LinearPerL(channels, generator)
        self.skip_tp = _SkipTP(channels, num_elements, 0 if residual else 3, generator)
        self.avg_num_neighbors = float(avg_num_neighbors)


class SyntheticInvariantMACE(torch.nn.Module):
    """Random-init invariant MACE with the upstream attribute tree (weights ~ N(0, 1), fp64)."""

    def __init__(self, channels: int = 128, atomic_numbers=(1, 6, 7, 8), r_max: float = 5.0, num_bessel: int = 8,
                 num_polynomial_cutoff: int = 5, radial_mlp=(64, 64, 64), mlp_hidden: int = 16,
                 avg_num_neighbors: float = 1.0, atomic_energies: Optional[torch.Tensor] = None, scale: float = 1.0,
                 shift: float = 0.0, seed: int = 0, coupling_basis_seed: Optional[int] = None):
        """coupling_basis_seed: when given, the contraction modules carry `U_matrix_1/2/3` buffers (as upstream's do)
        holding a permuted, sign-flipped path basis, and their weights refer to that basis."""
        super().__init__()
        g = torch.Generator().manual_seed(seed)
        coupling = None if coupling_basis_seed is None else permuted_coupling_basis(coupling_basis_seed)
        ne = len(atomic_numbers)
        self.channels, self.num_elements = channels, ne
        self.register_buffer("atomic_numbers", torch.tensor(list(atomic_numbers), dtype=torch.int64))
        self.register_buffer("r_max", torch.tensor(r_max, dtype=torch.float64))
        self.register_buffer("num_interactions", torch.tensor(2, dtype=torch.int64))
        self.node_embedding = _NodeEmbedding(ne, channels, g)
        self.radial_embedding = _RadialEmbedding(r_max, num_bessel, num_polynomial_cutoff)
        e0 = torch.zeros(ne, dtype=torch.float64) if atomic_energies is None else atomic_energies
        self.atomic_energies_fn = _AtomicEnergies(e0)
        self.interactions = torch.nn.ModuleList([
            _Interaction(channels, ne, num_bessel, list(radial_mlp), False, avg_num_neighbors, g),
            _Interaction(channels, ne, num_bessel, list(radial_mlp), True, avg_num_neighbors, g),
        ])
        self.products = torch.nn.ModuleList([_ProductBasis(channels, ne, False, g, coupling),
                                             _ProductBasis(channels, ne, True, g, coupling)])
        self.readouts = torch.nn.ModuleList([_LinearReadout(channels, g), _NonLinearReadout(channels, mlp_hidden, g)])
        self.scale_shift = _ScaleShift(scale, shift)

    def export_params(self) -> Dict[str, object]:
        """Plain tensors of every weight, for an independent evaluation of the same model."""
        C, ne = self.channels, self.num_elements
        layers = []
        for t in range(2):
            it, pr = self.interactions[t], self.products[t]
            con = pr.symmetric_contractions.contractions[0]
            lmax = it.skip_tp.lmax
            layers.append(dict(
                W_up=it.linear_up.weight.detach().view(C, C).clone(),
                mlp=[w.detach().clone() for w in it.conv_tp_weights.weights],
                W_lin=it.linear.weight.detach().view(4, C, C).clone(),
                W_skip=it.skip_tp.weight.detach().view(lmax + 1, C, ne, C).clone(),
                W3=con.weights_max.detach().clone(), W2=con.weights[0].detach().clone(), W1=con.weights[1].detach().clone(),
                W_prod=pr.linear.weight.detach().view(C, C).clone(),
                avg_num_neighbors=it.avg_num_neighbors,
            ))
            if hasattr(con, "U_matrix_3"):  # the basis the weights refer to, when the module carries one
                layers[-1].update(U2=con.U_matrix_2.detach().clone(), U3=con.U_matrix_3.detach().clone())
        ro0, ro1 = self.readouts
        return dict(
            channels=C, num_elements=ne, r_max=float(self.r_max), num_bessel=self.radial_embedding.out_dim,
            p=self.radial_embedding.p, W_emb=self.node_embedding.weight.detach().view(ne, C).clone(),
            E0=self.atomic_energies_fn.atomic_energies.detach().view(-1).clone(), layers=layers,
            w_read0=ro0.linear.weight.detach().view(C, 1).clone(),
            W_read1=ro1.linear_1.weight.detach().view(C, -1).clone(), w_read2=ro1.linear_2.weight.detach().view(-1, 1).clone(),
            scale=float(self.scale_shift.scale), shift=float(self.scale_shift.shift),
        )

    def forward(self, *args, **kwargs):
        raise NotImplementedError("weight container for OptimizedInvariantMACE; it has no forward of its own")
