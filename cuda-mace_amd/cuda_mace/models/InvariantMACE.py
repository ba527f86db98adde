"""OptimizedInvariantMACE: an invariant MACE model whose hot path runs on the gfx950 HIP kernels.

Drop-in for the reference's cuda_mace/models/InvariantMACE.py: same class names, same constructor
argument (an upstream-like model object whose attribute tree is read, see :168-244 there), same
`forward(data, training, compute_force, compute_virials, compute_stress, compute_displacement)` and the
same output dictionary (:366-377).  The pieces the reference borrows from upstream `mace`
(`scatter_sum`, `get_edge_vectors_and_lengths`, `get_outputs`, `get_symmetric_displacement`) are small
torch functions here, because upstream is not a dependency.
"""
from __future__ import annotations

from copy import deepcopy
from math import sqrt
from typing import Dict, Optional, Tuple

import numpy as np
import torch

from cuda_mace.ops.cubic_spline import CubicSpline
from cuda_mace.ops.invariant_message_passing import InvariantMessagePassingTP
from cuda_mace.ops.linear import ElementalLinear, Linear, ScalarElementalLinear
from cuda_mace.ops.spherical_harmonics import SphericalHarmonics
from cuda_mace.ops.symmetric_contraction import SymmetricContraction as CUDAContraction
from cuda_mace import _cabi as cabi
from cuda_mace.ops._autograd import (EdgeGeometryAutograd, LinearContractionAutograd, ReadoutEnergyAutograd, ScalarLinearAutograd,
                                     _cached, _cached_for, _cached_per, groups_of, groups_of_one_hot, monomials_from_packed)
from cuda_mace.utils.irreps import Instruction


# ---- the few upstream helpers the forward needs ------------------------------------------------------
def scatter_sum(src: torch.Tensor, index: torch.Tensor, dim: int = -1, dim_size: Optional[int] = None,
                ptr: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Sum of src over equal index values.  With `ptr` (index is sorted and ptr holds the segment boundaries, as for the
    atoms of a batch of graphs) the sums are taken segment by segment in a fixed order, so that they do not vary from
    run to run as atomic additions do."""
    dim = dim % src.dim()
    size = list(src.shape)
    size[dim] = int(dim_size) if dim_size is not None else int(index.max()) + 1
    if size[dim] == 1:
        # single graph: a plain reduction, whose summation order does not vary from run to run
        return src.sum(dim=dim, keepdim=True)
    if ptr is not None and ptr.numel() == size[dim] + 1:
        return torch.segment_reduce(src, "sum", offsets=ptr, axis=dim)
    out = torch.zeros(size, dtype=src.dtype, device=src.device)
    return out.index_add_(dim, index, src)


def get_edge_vectors_and_lengths(positions, edge_index, shifts) -> Tuple[torch.Tensor, torch.Tensor]:
    """vectors = positions[edge_index[1]] - positions[edge_index[0]] + shifts (upstream convention)."""
    vectors = positions[edge_index[1]] - positions[edge_index[0]] + shifts
    return vectors, torch.linalg.norm(vectors, dim=-1, keepdim=True)


class _RowsOfSortedIndex(torch.autograd.Function):
    """src[index] for a non-decreasing index whose segment boundaries are `bounds` (a list of ints: bounds[g] = first
    position with index g).  The backward is one reduction per segment (a slice each); the plain gather's backward adds every row into
    the few rows of src with atomics, which serialises when thousands of rows share one, and torch.segment_reduce gives a
    segment to a single thread."""

    @staticmethod
    def forward(ctx, src, index, bounds):
        ctx.bounds = bounds  # python ints, read from the device once per index tensor by the caller
        return src.index_select(0, index)

    @staticmethod
    def backward(ctx, grad):
        b = ctx.bounds
        return torch.stack([grad[b[g]:b[g + 1]].sum(dim=0) for g in range(len(b) - 1)]), None, None


def get_symmetric_displacement(positions, unit_shifts, cell, edge_index, num_graphs, batch):
    """Applies a symmetric strain (zero, but differentiable) to positions and cell so that
    d energy / d displacement gives the virial."""
    if cell is None:
        cell = torch.zeros(num_graphs * 3, 3, dtype=positions.dtype, device=positions.device)
    sender = edge_index[0]
    displacement = torch.zeros((num_graphs, 3, 3), dtype=positions.dtype, device=positions.device)
    displacement.requires_grad_(True)
    symmetric = 0.5 * (displacement + displacement.transpose(-1, -2))
    cell = cell.view(-1, 3, 3)
    cell = cell + torch.matmul(cell, symmetric)
    if num_graphs == 1:
        # one graph: products with the one matrix broadcast, whose backward is a sum over the rows (the gathered form
        # below makes autograd add every atom's and every edge's 3 x 3 contribution into the one strain / cell with
        # atomics: 0.5 s at 1.3 million edges; as a matrix product the backward is a 3 x E by E x 3 GEMM, 37 ms there)
        positions = positions + (positions.unsqueeze(-1) * symmetric[0].unsqueeze(0)).sum(dim=1)
        shifts = (unit_shifts.to(cell.dtype).unsqueeze(-1) * cell[0].unsqueeze(0)).sum(dim=1)
    else:
        # what depends on the lists alone (the graph of every edge, whether atoms and edges come graph by graph, and where
        # the graphs' segments begin) is read from the device once per pair of tensors, not per step: a steady-state
        # evaluation then has no host synchronisation here
        def segments():
            graphs = torch.arange(num_graphs + 1, device=batch.device, dtype=batch.dtype)
            edge_graph = batch[sender]
            sorted_lists = bool((batch[1:] >= batch[:-1]).all()) and bool((edge_graph[1:] >= edge_graph[:-1]).all())
            if not sorted_lists:
                return edge_graph, False, None, None
            return (edge_graph, True, [int(v) for v in torch.searchsorted(batch, graphs).tolist()],
                    [int(v) for v in torch.searchsorted(edge_graph, graphs).tolist()])

        edge_graph, sorted_lists, atom_bounds, edge_bounds = _cached_for(edge_index, "_cm_strain_segments_%d" % num_graphs, batch,
                                                                          segments)
        if sorted_lists:  # atoms and edges graph by graph, as every collated batch has them
            per_atom = _RowsOfSortedIndex.apply(symmetric, batch, atom_bounds)
            per_edge = _RowsOfSortedIndex.apply(cell, edge_graph, edge_bounds)
        else:
            per_atom, per_edge = symmetric[batch], cell[edge_graph]
        positions = positions + torch.einsum("be,bec->bc", positions, per_atom)
        shifts = torch.einsum("be,bec->bc", unit_shifts.to(cell.dtype), per_edge)
    return positions, shifts, displacement, cell


_CONSTANTS: Dict[tuple, torch.Tensor] = {}


def _constant(value: float, shape, dtype, device) -> torch.Tensor:
    """A tensor filled with `value`, made once per (value, shape, dtype, device) and never written again: saves a fill
    kernel per step for seeds and all-zero outputs."""
    key = (float(value), tuple(shape), dtype, device)
    hit = _CONSTANTS.get(key)
    if hit is None:
        hit = _CONSTANTS[key] = torch.full(tuple(shape), float(value), dtype=dtype, device=device)
    return hit


def get_outputs(energy, positions, displacement, cell, training=False, compute_force=True, compute_virials=False,
                compute_stress=False):
    """forces = -dE/dpositions; virials = -dE/ddisplacement; stress = -virials / volume.  The backward pass is seeded with
    -1 (a constant tensor kept per device), so that it delivers forces and virials themselves and no negation runs."""
    forces = virials = stress = None
    grad_outputs = [_constant(-1.0, energy.shape, energy.dtype, energy.device)]
    want_virials = compute_virials or compute_stress
    if compute_force and want_virials:
        forces, virials = torch.autograd.grad([energy], [positions, displacement], grad_outputs=grad_outputs,
                                              retain_graph=training, create_graph=training, allow_unused=True)
        if virials is None:
            virials = torch.zeros_like(displacement)
    elif compute_force:
        (forces,) = torch.autograd.grad([energy], [positions], grad_outputs=grad_outputs, retain_graph=training,
                                        create_graph=training, allow_unused=True)
    if compute_force and forces is None:
        forces = torch.zeros_like(positions)
    if compute_stress and virials is not None and cell is not None:
        cell3 = cell.view(-1, 3, 3)
        volume = torch.linalg.det(cell3).abs().view(-1, 1, 1)
        stress = -virials / volume
    return forces, virials, stress, None, None


def _select_head(per_head: torch.Tensor, node_heads: torch.Tensor) -> torch.Tensor:
    """per_head[n, node_heads[n]] (the reference's `[arange, node_heads]` indexing, models/InvariantMACE.py:287-289, 336),
    written as a gather so that its backward is a plain scatter instead of a sort-based index_put."""
    if per_head.dim() == 1:
        return per_head
    if per_head.shape[1] == 1:
        return per_head[:, 0]
    return torch.gather(per_head, 1, node_heads.view(-1, 1)).squeeze(1)


def fused_readout_parameters(readouts, scale_shift):
    """Weights of the readout pair in the form the fused readout kernel takes, or None when the modules are not the
    standard pair of a two-layer invariant model (a linear readout to one scalar, then linear -> normalised silu gate ->
    linear to one scalar, single head, scalar scale and shift).  Attribute names follow upstream's readout blocks
    (`linear`; `linear_1`, `non_linearity`, `linear_2`), whose modules the reference keeps as they are
    (models/InvariantMACE.py:196)."""
    try:
        r0, r1 = readouts
        lin0, lin1, lin2 = r0.linear, r1.linear_1, r1.linear_2
        gate = r1.non_linearity.acts[0]
        dims = [(l.__dict__["irreps_in"].num_irreps, l.__dict__["irreps_out"].num_irreps) for l in (lin0, lin1, lin2)]
        (c0, o0), (c1, hidden), (h2, o2) = dims
        if not (o0 == 1 and o2 == 1 and c0 == c1 and h2 == hidden and 1 <= hidden <= 16 and c0 <= 256):
            return None
        if getattr(gate, "f", None) is not torch.nn.functional.silu or len(r1.non_linearity.acts) != 1:
            return None
        if scale_shift.scale.numel() != 1 or scale_shift.shift.numel() != 1:
            return None
        w1 = lin0.weight.data.double().reshape(c0) / sqrt(c0)
        W2a = lin1.weight.data.double().reshape(c1, hidden) / sqrt(c1)
        w2b = lin2.weight.data.double().reshape(hidden) / sqrt(hidden)
        return {"w1": w1.contiguous(), "W2a": W2a.contiguous(), "w2b": w2b.contiguous(), "act_cst": float(gate.cst),
                "scale": float(scale_shift.scale), "shift": float(scale_shift.shift)}
    except (AttributeError, KeyError, TypeError, ValueError, IndexError, RuntimeError):
        return None


# ---- model pieces -----------------------------------------------------------------------------------------
class SymmetricContractionWrapper(torch.nn.Module):
    def __init__(self, symmetric_contractions):
        super().__init__()
        self.symmetric_contractions = symmetric_contractions

    def forward(self, x, y):
        # y: one-hot [nnodes, nelements] as upstream passes it, or already the int32 element index
        if y.dim() == 2:
            y = y.argmax(dim=-1).int()
        return self.symmetric_contractions(x, y).squeeze(1)


class linear_matmul(torch.nn.Module):
    """x @ W / sqrt(fan_in) for scalar features, from an e3nn-Linear-like module (reference :41-53)."""

    def __init__(self, linear_e3nn):
        super().__init__()
        n_in = linear_e3nn.__dict__["irreps_in"].num_irreps
        n_out = linear_e3nn.__dict__["irreps_out"].num_irreps
        self.register_buffer("weights", (linear_e3nn.weight.data.reshape(n_in, n_out) / n_in ** 0.5).float())
        self.register_buffer("weights_transposed", self.weights.t().contiguous())
        # widths the MFMA linear kernel takes (multiples of 32 up to 256); anything else goes to torch.matmul as in the reference
        self.on_kernel = all(w % 32 == 0 and 32 <= w <= 256 for w in (n_in, n_out))

    def forward(self, x, residual=None):
        """residual (optional, shape of the result): added to the product, in the kernel's epilogue where the kernel runs."""
        if self.on_kernel and x.is_cuda and x.dtype == torch.float32 and x.dim() == 2:
            # same fp32-equivalent GEMM as the per-l linears; a third faster than the library GEMM at these sizes
            if residual is not None and residual.dtype == torch.float32 and residual.shape == (x.shape[0], self.weights.shape[1]):
                return ScalarLinearAutograd.apply(x, self.weights_transposed, self.weights, residual)
            y = ScalarLinearAutograd.apply(x, self.weights_transposed, self.weights, None)
        else:
            y = torch.matmul(x, self.weights)
        return y if residual is None else y + residual


def element_linear_to_cuda(skip_tp):
    """Per-element, per-l weight blocks of the first layer's skip tensor product (reference :56-74)."""
    num_elements = skip_tp.__dict__["irreps_in2"].dim
    n_channels = skip_tp.__dict__["irreps_in1"][0].dim
    lmax = skip_tp.__dict__["irreps_in1"].lmax
    ws = skip_tp.weight.data.float().reshape([lmax + 1, n_channels, num_elements, n_channels]).permute(2, 0, 1, 3)
    ws = ws.flatten(1) / sqrt(num_elements)
    instructions = [Instruction(l, l, (n_channels, n_channels), 1.0 / sqrt(n_channels)) for l in range(lmax + 1)]
    return ElementalLinear(skip_tp.__dict__["irreps_in1"], skip_tp.__dict__["irreps_out"], instructions, ws, num_elements)


def scalar_skip_to_cuda(skip_tp):
    """The residual skip connection of the second layer (a fully connected tensor product of scalar features with the
    one-hot species, weight [C, ne, C], normalised by 1/sqrt(C * ne)) as a per-element linear on the MFMA kernel."""
    num_elements = skip_tp.__dict__["irreps_in2"].dim
    n_in = skip_tp.__dict__["irreps_in1"].num_irreps
    n_out = skip_tp.__dict__["irreps_out"].num_irreps
    ws = skip_tp.weight.data.double().reshape(n_in, num_elements, n_out).permute(1, 0, 2) / sqrt(num_elements)
    return ScalarElementalLinear(ws)


class _FloatLinearView:
    """Presents an e3nn-Linear-like module with fp32 weights without converting the module in place; `divide_by`
    folds the reference's `linear(message) / avg_num_neighbors` (models/InvariantMACE.py:114) into the weights."""

    def __init__(self, linear, divide_by: float = 1.0):
        self.irreps_in, self.irreps_out = linear.irreps_in, linear.irreps_out
        self.instructions = linear.instructions
        self.weight = (linear.weight.data.double() / float(divide_by)).float()


def _message_passing(tp, node_feats, edge_attrs, edge_feats, sender, receiver, edge_lengths, edge_spline, edge_vectors):
    """Tabulated radial weights (edge_feats [E, 4C], the reference's data flow); or, when edge_feats is None, radial
    weights evaluated inside the message-passing kernels from the spline of the edge lengths; or, when edge_attrs is
    None too, harmonics and radial weights both evaluated inside the kernels from the fp32 edge vectors."""
    if edge_feats is not None:
        return tp.forward(node_feats, edge_attrs, edge_feats.view(edge_feats.shape[0], -1, node_feats.shape[-1]), sender,
                          receiver, node_feats.shape[0])
    if edge_attrs is None:
        return tp.forward_edges(node_feats, edge_vectors, edge_spline, sender, receiver, node_feats.shape[0])
    return tp.forward_spline(node_feats, edge_attrs, edge_lengths, edge_spline, sender, receiver, node_feats.shape[0])


class InvariantInteraction(torch.nn.Module):
    """First layer: linear_up, message passing, per-l linear, per-element linear."""

    def __init__(self, mace_model):
        super().__init__()
        inter = mace_model.interactions[0]
        self.linear_up = linear_matmul(inter.linear_up)
        self.linear = Linear(_FloatLinearView(inter.linear, divide_by=inter.avg_num_neighbors))
        self.tp = InvariantMessagePassingTP()
        self.skip_tp = element_linear_to_cuda(inter.skip_tp)
        self.avg_num_neighbors = inter.avg_num_neighbors
        # The per-l linear and the per-element linear that follows it are both linear in the message, so they compose
        # into one per-element map  W[e, l] = W_linear[l] . W_skip[e, l] / sqrt(C)  (the kernel supplies the second
        # 1/sqrt(C)).  Composed in fp64 once; saves one [N,16,C] GEMM pass in forward and one in backward.
        K = self.linear.weights.shape[-2]
        composed = torch.einsum("lij,eljk->elik", self.linear.weights.double(), self.skip_tp.weights.double()) / sqrt(K)
        self.register_buffer("composed_weights", composed.float().contiguous())
        self.register_buffer("composed_weights_transposed", composed.float().transpose(-1, -2).contiguous())
        self.compose_linears = True

    def forward(self, node_attrs, node_feats, edge_attrs, edge_feats, edge_index, sender=None, receiver=None,
                edge_lengths=None, edge_spline=None, edge_vectors=None, node_feats_are_up: bool = False,
                apply_linear: bool = True):
        """node_feats_are_up: node_feats is already linear_up(embedding) (the model caches it per species tensor).
        apply_linear=False returns the message before the channel-mixing linears (the model then runs them fused with
        the symmetric contraction, see `fused_linear`)."""
        if sender is None:
            sender, receiver = edge_index[1].int(), edge_index[0].int()
        if not node_feats_are_up:
            node_feats = self.linear_up(node_feats)
        message = _message_passing(self.tp, node_feats, edge_attrs, edge_feats, sender, receiver, edge_lengths, edge_spline,
                                   edge_vectors)
        if not apply_linear:
            return message, None
        if self.compose_linears:
            message = self.skip_tp.cuda_obj.forward(message, self.composed_weights, self.composed_weights_transposed, node_attrs)
        else:
            message = self.linear(message)  # 1/avg_num_neighbors is folded into its weights
            message = self.skip_tp(message, node_attrs)
        return message, None

    def fused_linear(self):
        """(W_T, W, scale, per_element) of the channel mixing between message passing and the contraction."""
        K = self.composed_weights.shape[-2]
        return self.composed_weights_transposed, self.composed_weights, 1.0 / sqrt(K), True


class InvariantResidualInteraction(torch.nn.Module):
    """Second layer: residual skip connection on the scalar features, linear_up, message passing, per-l linear."""

    def __init__(self, mace_model):
        super().__init__()
        inter = mace_model.interactions[1]
        self.linear_up = linear_matmul(inter.linear_up)
        self.linear = Linear(_FloatLinearView(inter.linear, divide_by=inter.avg_num_neighbors))
        self.tp = InvariantMessagePassingTP()
        self.skip_tp = scalar_skip_to_cuda(inter.skip_tp)
        self.avg_num_neighbors = inter.avg_num_neighbors

    def forward(self, node_attrs, node_feats, edge_attrs, edge_feats, edge_index, sender=None, receiver=None,
                edge_lengths=None, edge_spline=None, edge_vectors=None, node_feats_are_up: bool = False,
                apply_linear: bool = True):
        if sender is None:
            sender, receiver = edge_index[1].int(), edge_index[0].int()
        sc = self.skip_tp(node_feats, node_attrs)
        node_feats = self.linear_up(node_feats)
        message = _message_passing(self.tp, node_feats, edge_attrs, edge_feats, sender, receiver, edge_lengths, edge_spline,
                                   edge_vectors)
        if apply_linear:
            message = self.linear(message)  # 1/avg_num_neighbors is folded into its weights
        return message, sc

    def fused_linear(self):
        K = self.linear.weights.shape[-2]
        return self.linear.weights_transposed, self.linear.weights, 1.0 / sqrt(K), False


class _WeightsToken:
    """Identity of one model's (frozen) weights; a cache entry that holds it can never be taken for another model's."""


class OptimizedInvariantMACE(torch.nn.Module):
    # forward() honours data["node_weights"] (see _forward_ordered); wrappers that need per-atom seeds check for this
    supports_node_weights = True

    def __init__(self, mace_model: torch.nn.Module, device="cuda", num_spline_knots: int = 256, fused_radial: bool = True,
                 fused_readout: bool = True, fused_contraction: bool = True, spatial_order_min_atoms: Optional[int] = 8192,
                 native_step: bool = True):
        """fused_radial=True evaluates the spherical harmonics and the radial spline inside the message-passing kernels
        (same numbers; no [16, nedges] or [nedges, 4C] tensors in memory); False keeps the reference's separate
        SphericalHarmonics -> CubicSpline -> message passing steps.  fused_readout=True evaluates both readouts, scale
        and shift in one fp64 kernel per direction when the readout modules have the standard form; False (or any other
        form, or several heads) runs the modules themselves in fp64 as the reference does.  fused_contraction=True runs the
        channel-mixing linear before each symmetric contraction and the contraction as one autograd node whose backward is
        a single kernel; False keeps the reference's separate Linear / ElementalLinear and SymmetricContraction ops.
        native_step=True (with all three fusions on) hands an inference step without strain -- energy and forces of one
        head -- to the library as ONE call that enqueues every kernel of the forward and of the backward chain itself
        (no interpreter or autograd engine between the launches; same kernels, order and numbers as the autograd path,
        which still serves training, virials / stress and compute_force=False).
        spatial_order_min_atoms: from this many atoms on, the model works on a relabelled copy of the graph in which
        atoms that are close in space have close indices (derived once per edge_index tensor), so that the gathers of
        sender rows hit in cache; outputs come back in the caller's order.  None switches the relabelling off."""
        super().__init__()
        self.spatial_order_min_atoms = spatial_order_min_atoms
        self._weights_token = _WeightsToken()  # what caches of weight-dependent, species-only tensors are keyed on
        self.fused_radial = bool(fused_radial)
        assert int(mace_model.num_interactions) == 2, "exactly two interaction layers are supported"
        self.register_buffer("atomic_numbers", deepcopy(mace_model.atomic_numbers))
        self.register_buffer("r_max", deepcopy(mace_model.r_max))
        self.register_buffer("num_interactions", deepcopy(mace_model.num_interactions))

        self.node_embedding = deepcopy(mace_model.node_embedding)
        self.radial_embedding = deepcopy(mace_model.radial_embedding)
        self.spherical_harmonics = SphericalHarmonics()
        self.atomic_energies_fn = deepcopy(mace_model.atomic_energies_fn)

        self.interactions = torch.nn.ModuleList([InvariantInteraction(mace_model), InvariantResidualInteraction(mace_model)])
        self.products = deepcopy(mace_model.products)
        self.readouts = deepcopy(mace_model.readouts).to(torch.float64)

        for i in range(int(mace_model.num_interactions)):
            contraction = CUDAContraction(mace_model.products[i].symmetric_contractions, device=device)
            self.products[i].symmetric_contractions = SymmetricContractionWrapper(contraction)
            self.products[i].linear = linear_matmul(mace_model.products[i].linear)

        # tabulate R(r) = conv_tp_weights(radial_embedding(r)) of each layer in fp64, spline it in fp32
        r_np, h = np.linspace(1e-12, float(self.r_max) + 1.0, num_spline_knots, retstep=True)
        r = torch.tensor(r_np, dtype=torch.float64)
        with torch.no_grad():
            radial = deepcopy(mace_model.radial_embedding).double().cpu()
            bessel_j = radial(r.unsqueeze(-1), None, None, None)
            if isinstance(bessel_j, tuple):
                bessel_j = bessel_j[0]
            edge_splines = []
            for interaction in mace_model.interactions:
                R = deepcopy(interaction.conv_tp_weights).double().cpu()(bessel_j)
                edge_splines.append(CubicSpline(r.float(), R.float(), float(h), float(self.r_max)))
        self.edge_splines = torch.nn.ModuleList(edge_splines)

        self.scale_shift = deepcopy(mace_model.scale_shift).double()
        # both readouts, scale and shift as one fp64 kernel per direction when the modules have the standard form;
        # otherwise the modules themselves run, as in the reference
        fused = fused_readout_parameters(mace_model.readouts, mace_model.scale_shift)
        self.fused_readout = bool(fused_readout) and fused is not None
        if self.fused_readout:
            self.register_buffer("readout_w1", fused["w1"])
            self.register_buffer("readout_W2a", fused["W2a"])
            self.register_buffer("readout_w2b", fused["w2b"])
            self.readout_constants = (fused["act_cst"], fused["scale"], fused["shift"])
        self.fused_contraction = bool(fused_contraction)
        self.to(device)
        self._contraction_builtin = None  # folded coefficient tables are made on the GPU, at the latest by the first step
        if self.fused_contraction and torch.device(device).type == "cuda":
            self._fold_contraction_tables()
        # inference model: the custom ops differentiate with respect to features and geometry only, so no weight
        # needs a gradient; frozen weights also let autograd skip dX of the first layer, whose input depends on
        # the species alone
        for p in self.parameters():
            p.requires_grad_(False)
        # kept for reference like upstream does, but not as a registered sub-module: moving or casting the
        # optimised model must not touch the caller's original model
        object.__setattr__(self, "orig_model", mace_model)
        self.native_step = bool(native_step)
        object.__setattr__(self, "_native", None)  # NativeStep, built on first use (holds device addresses: not pickled)

    def __getstate__(self):
        state = dict(self.__dict__)
        state["_native"] = None
        return state

    def _native_step_of(self):
        if self._native is None:
            from cuda_mace.ops.native_step import NativeStep

            if self._contraction_builtin is None:
                self._fold_contraction_tables()
            object.__setattr__(self, "_native", NativeStep(self) if NativeStep.supported(self) else False)
        return self._native or None

    def _native_step_for(self, data, training: bool, compute_force: bool, compute_displacement: bool):
        """The library's one-call step, if this evaluation can run on it: inference with forces (virials and stress come
        from the same per-edge gradients), one head, positions on the GPU, no strain tensor asked for."""
        if not (self.native_step and not training and compute_force and not compute_displacement and "head" not in data
                and data["positions"].is_cuda):
            return None
        return self._native_step_of()

    def _fold_contraction_tables(self):
        """Per layer: the packed coupling tables regrouped into monomials (host, once) and folded with the per-element
        weights into coefficient tables on the device."""
        builtin3, builtin2 = cabi.symcon_builtin_structure()
        self._contraction_builtin = []
        for i, product in enumerate(self.products):
            mod = product.symmetric_contractions.symmetric_contractions
            (m3, o3, p3, v3), (m2, o2, p2, v2) = monomials_from_packed(mod.U3_num_nonsparse, mod.U3_indices, mod.U3_values,
                                                                       mod.U2_num_nonsparse, mod.U2_indices, mod.U2_values)
            dev = mod.weights_3.device
            t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)  # noqa: E731
            T3, T2, T1 = cabi.symcon_tables(t(o3), t(p3), t(v3), t(o2), t(p2), t(v2), mod.weights_3[0].contiguous(),
                                            mod.weights_2[0].contiguous(), mod.weights_1[0].contiguous())
            self._contraction_builtin.append(bool(np.array_equal(m3, builtin3) and np.array_equal(m2, builtin2)))
            for name, val in (("mono3", t(m3)), ("mono2", t(m2)), ("T3", T3), ("T2", T2), ("T1", T1)):
                self.register_buffer("contraction_%s_%d" % (name, i), val)

    def _contraction_tables(self, i: int):
        g = lambda name: getattr(self, "contraction_%s_%d" % (name, i))  # noqa: E731
        return g("mono3"), g("mono2"), g("T3"), g("T2"), g("T1"), self._contraction_builtin[i]

    def _spatial_order(self, data: Dict[str, torch.Tensor]):
        """Relabelling of one neighbour list: atoms sorted by (graph, cell of a 3-D grid of at least half the cutoff,
        original index), edges re-sorted by the new row-0 label and, inside a row-0 segment, by the row-1 label with the
        pairs beyond the cutoff (the skin shell of a Verlet list) last, nearest first: the native step cuts every segment
        back to its last pair inside the cutoff, and with this order the pairs that drift inside between two list builds
        are the first of the shell, so the cut stays close to the pairs that count.  One library call on the device
        (cm_graph_prepare), no host synchronisation; it also delivers the CSR offsets and the sender-sorted view of the new
        list, which are left where the ops look for them.  Returns (perm new -> old [N], inverse [N], edge_perm new -> old
        [E], relabelled edge_index [2, E], relabelled batch [N]).  Any permutation is valid; this one is cheap and keeps
        neighbours within a few hundred indices of each other."""
        pos = data["positions"].detach().double().contiguous()
        batch, edge_index = data["batch"], data["edge_index"]
        n, ngraphs = pos.shape[0], int(data["ptr"].numel()) - 1
        row0, row1 = _cached(edge_index, "_cm_int32_rows", None,
                             lambda: (edge_index[0].int().contiguous(), edge_index[1].int().contiguous()))
        shifts = data["shifts"].detach().double().contiguous()
        # cells per axis from the size alone (a host constant): enough for cells of half a cutoff at 0.05 atoms / A^3
        bins = int(min(64, max(1, np.ceil((n / max(ngraphs, 1) / 0.05) ** (1.0 / 3.0) / (0.5 * float(self.r_max))))))
        while ngraphs * bins ** 3 >= 2 ** 24:
            bins -= 1
        g = cabi.graph_prepare(pos, row0, row1, shifts, None if ngraphs == 1 else batch.int().contiguous(), ngraphs,
                               float(self.r_max), bins)
        perm, inverse, edge_perm = g["node_perm"].long(), g["node_inverse"].long(), g["edge_perm"].long()
        receiver, sender = g["receiver"], g["sender"]
        new_edges = torch.stack((receiver, sender)).long()
        # what the ops derive from a list is already there: leave it where they look it up
        new_edges.__dict__["_cm_int32_rows"] = ((new_edges._version, new_edges.data_ptr(), None), (receiver, sender))
        receiver.__dict__["_cm_csr"] = ((receiver._version, receiver.data_ptr(), n), g["first_occ"])
        sender.__dict__["_cm_sender_view"] = ((sender._version, sender.data_ptr(), n), (g["sender_perm"], g["sender_offsets"]))
        if data["shifts"].dtype == torch.float64:
            t = data["shifts"]
            edge_index.__dict__["_cm_spatial_shifts"] = (t, (edge_index._version, edge_index.data_ptr(), t._version), g["shifts"])
        return perm, inverse, edge_perm, new_edges, batch.index_select(0, perm)

    def forward(self, data: Dict[str, torch.Tensor], training: bool = False, compute_force: bool = True,
                compute_virials: bool = False, compute_stress: bool = False,
                compute_displacement: bool = False, compute_node_feats: bool = True) -> Dict[str, Optional[torch.Tensor]]:
        """compute_node_feats=False (no counterpart in the reference, which always returns the [N, 2C] fp64 features):
        "node_feats" may come back as None; the one-call step then skips that output (51 MB at 25 000 atoms x 128
        channels), which an MD driver never reads."""
        n = data["positions"].shape[0]
        if self.spatial_order_min_atoms is None or n < self.spatial_order_min_atoms or training:
            return self._forward_ordered(data, training, compute_force, compute_virials, compute_stress, compute_displacement,
                                         compute_node_feats=compute_node_feats)
        # Same step on the relabelled graph.  Everything that depends only on the neighbour list or the species is
        # derived once per tensor object; per call the positions are gathered into the new order and forces, node
        # energies and node features gathered back (fixed-order gathers: results stay reproducible bit for bit).
        perm, inverse, edge_perm, edge_index, batch = _cached(data["edge_index"], "_cm_spatial_order", None,
                                                              lambda: self._spatial_order(data))
        inner = dict(data)
        # Without strain the positions stay in the caller's order: the geometry kernels read them (and write the forces)
        # through the row map.  The strain path transforms positions per graph and works on a gathered copy; the
        # one-call step needs no strain for virials and stress.
        direct = (not (compute_virials or compute_stress or compute_displacement)
                  or self._native_step_for(data, training, compute_force, compute_displacement) is not None)
        # With compute_force=False the caller differentiates the returned energies itself (a wrapper that sums the
        # energies of some atoms only): the positions then stay attached to the caller's tensor.
        own = data["positions"].detach() if compute_force else data["positions"]
        inner["positions"] = own if direct else own.index_select(0, perm)
        inner["edge_index"], inner["batch"] = edge_index, batch
        inner["node_attrs"] = _cached_for(data["edge_index"], "_cm_spatial_attrs", data["node_attrs"],
                                          lambda: data["node_attrs"].index_select(0, perm))
        for name in ("shifts", "unit_shifts"):
            if name in data:
                t = data[name]
                inner[name] = _cached_for(data["edge_index"], "_cm_spatial_" + name, t, lambda t=t: t.index_select(0, edge_perm))
        if data.get("node_weights") is not None:
            t = data["node_weights"]
            inner["node_weights"] = _cached_for(data["edge_index"], "_cm_spatial_node_weights", t, lambda: t.index_select(0, perm))
        rows = _cached(data["edge_index"], "_cm_spatial_rows32", None, lambda: (perm.int(), inverse))
        # per-node outputs come back in the caller's order (node_rows)
        return self._forward_ordered(inner, training, compute_force, compute_virials, compute_stress, compute_displacement,
                                     node_rows=rows, positions_in_caller_order=direct, compute_node_feats=compute_node_feats)

    def _forward_ordered(self, data: Dict[str, torch.Tensor], training: bool = False, compute_force: bool = True,
                         compute_virials: bool = False, compute_stress: bool = False, compute_displacement: bool = False,
                         node_rows=None, positions_in_caller_order: bool = False,
                         compute_node_feats: bool = True) -> Dict[str, Optional[torch.Tensor]]:
        """node_rows = (rows int32 [N], inverse int64 [N]): node n of `data` is node rows[n] of the caller, and the
        per-node outputs (forces, node_energy, node_feats) are returned in the caller's order.
        positions_in_caller_order: data["positions"] (and hence the forces) are rows of the caller, read through rows."""
        data["positions"].requires_grad_(True)
        positions = data["positions"]
        node_attrs = data["node_attrs"]
        batch = data["batch"]
        node_heads = data["head"][batch] if "head" in data else None  # None: every node reads head 0
        zero_heads = None if node_heads is not None else _cached(batch, "_cm_zero_heads", None, lambda: torch.zeros_like(batch))
        num_graphs = data["ptr"].numel() - 1
        shifts = data["shifts"]
        cell = data.get("cell")

        native = None
        if node_rows is None or positions_in_caller_order:
            native = self._native_step_for(data, training, compute_force, compute_displacement)
        displacement = _constant(0.0, (num_graphs, 3, 3), positions.dtype, positions.device)  # replaced below when strained
        if native is None and (compute_virials or compute_stress or compute_displacement):
            positions, shifts, displacement, cell = get_symmetric_displacement(
                positions=positions, unit_shifts=data["unit_shifts"], cell=cell, edge_index=data["edge_index"],
                num_graphs=num_graphs, batch=batch)

        # What depends on the species alone -- the atomic reference energies, the node embedding and the first layer's
        # linear_up of it (weights are frozen) -- is evaluated once per node_attrs tensor and reused while that tensor
        # is unchanged, like the index structures below.
        def species_only():
            with torch.no_grad():
                attrs64 = node_attrs.double()
                return (self.atomic_energies_fn(attrs64),
                        self.interactions[0].linear_up(self.node_embedding(attrs64).float()))

        e0_per_head, node_feats_up = _cached_for(node_attrs, "_cm_species_only", self._weights_token, species_only)
        node_e0 = _select_head(e0_per_head, zero_heads if node_heads is None else node_heads)
        # data["node_weights"] [N] (optional): every node energy enters the graph's energy, and hence the quantity the
        # forces, virials and stress derive from, with this weight (1 for a rank's own atoms, 0 for ghost copies in a
        # domain-decomposed MD code); node_energy itself stays unweighted.
        node_weights = data.get("node_weights")
        if node_weights is not None:
            node_weights = node_weights.detach().to(torch.float64)

        def graph_e0(weights=node_weights):
            """(Weighted) sum of the atomic reference energies per graph.  The one-call step evaluates it once per
            list (it rides in the step's graph handle); the autograd path evaluates it per call."""
            if weights is not None:
                return scatter_sum(src=node_e0 * weights, index=batch, dim=0, dim_size=num_graphs, ptr=data["ptr"])
            if num_graphs == 1 and node_heads is None:
                # one graph: the sum of the atomic reference energies is a function of the species tensor alone, too
                return _cached_for(node_attrs, "_cm_e0_sum", self._weights_token, lambda: node_e0.sum(dim=0, keepdim=True))
            return scatter_sum(src=node_e0, index=batch, dim=0, dim_size=num_graphs, ptr=data["ptr"])

        node_feats = None

        # index structures shared by both layers, cached on the caller's tensors so that they are rebuilt only when
        # the neighbour list / the species change: int32 edge lists (their CSR offsets and sender-sorted view are in
        # turn cached on these), the fp32 one-hot matrix and the element index per node
        edge_index = data["edge_index"]
        receiver, sender = _cached(edge_index, "_cm_int32_rows", None,
                                   lambda: (edge_index[0].int().contiguous(), edge_index[1].int().contiguous()))
        node_attrs32, atom_types = _cached(node_attrs, "_cm_species", None,
                                           lambda: (node_attrs.detach().float(), node_attrs.detach().argmax(dim=-1).int()))

        if native is not None:
            rows32 = None if node_rows is None else node_rows[0]
            # one entry per model on the list's tensor, keyed on this model's weights token itself (the handle holds
            # X1, which depends on this model's weights)
            handle = _cached_per(edge_index, "_cm_native_graphs", self._weights_token, node_attrs,
                                 lambda: native.graph(edge_index, receiver, sender, node_attrs32, atom_types, data["ptr"],
                                                      node_feats_up, rows32, node_e0, graph_e0(None)))
            if node_weights is not None:
                plain = handle
                handle = _cached_per(data["node_weights"], "_cm_native_graphs_weighted", self._weights_token, plain,
                                     lambda: plain.with_node_weights(node_weights, graph_e0()))
            want_virials = compute_virials or compute_stress
            res = native(handle, positions, shifts, want_feats=compute_node_feats, want_virials=want_virials)
            inter_e = res["interaction_energy"]
            virials = res["virials"].to(positions.dtype) if want_virials else None
            stress = None
            if compute_stress and cell is not None:
                c3 = cell.view(-1, 3, 3).to(virials.dtype)  # the volume as a triple product: a few element-wise launches
                volume = (c3[:, 0] * torch.linalg.cross(c3[:, 1], c3[:, 2], dim=-1)).sum(dim=-1).abs()
                stress = -virials / volume.view(-1, 1, 1)
            # energy = e0 + interaction energy and node_energy = node_e0 + its interaction part (already in the caller's
            # order) are written by the step's own kernels: the atomic reference energies ride in the handle
            return {
                "energy": res["energy"], "node_energy": res["node_energy"], "interaction_energy": inter_e,
                "forces": res["forces"].to(data["positions"].dtype), "virials": virials, "stress": stress, "hessian": None,
                "displacement": displacement, "node_feats": res["node_feats"], "edge_forces": None,
            }

        # vectors = positions[edge_index[1]] - positions[edge_index[0]] + shifts in fp64, rounded once to fp32
        vectors32, lengths32 = EdgeGeometryAutograd.apply(positions, shifts, receiver, sender,
                                                          node_rows[0] if positions_in_caller_order else None)
        # fused mode: the message-passing kernels take the vectors themselves and evaluate the harmonics per edge
        edge_attrs = None if self.fused_radial else self.spherical_harmonics.forward(vectors32)

        fused_readout = self.fused_readout and node_heads is None
        node_es_list, node_feats_list = [], []
        for interaction, product, readout, edge_spline in zip(self.interactions, self.products, self.readouts, self.edge_splines):
            edge_feats = None if self.fused_radial else edge_spline.forward(lengths32)
            node_feats, sc = interaction(node_attrs=node_attrs32,
                                         node_feats=node_feats_up if node_feats is None else node_feats,
                                         edge_attrs=edge_attrs, edge_feats=edge_feats, edge_index=data["edge_index"],
                                         sender=sender, receiver=receiver, edge_lengths=lengths32, edge_spline=edge_spline,
                                         edge_vectors=vectors32, node_feats_are_up=node_feats is None,
                                         apply_linear=not self.fused_contraction)
            if self.fused_contraction:
                if self._contraction_builtin is None:
                    self._fold_contraction_tables()
                layer = len(node_feats_list)
                W_T, W, scale, per_element = interaction.fused_linear()
                ne = node_attrs32.shape[1]
                contracted = LinearContractionAutograd.apply(
                    node_feats, W_T, W, scale, groups_of_one_hot(node_attrs32) if per_element else None,
                    groups_of(atom_types, ne), self._contraction_tables(layer))
                # fp32 [N, C]; the skip connection is added in the linear kernel's epilogue
                node_feats = product.linear(contracted, sc if sc is not None and getattr(product, "use_sc", True) else None)
            else:
                node_feats = product(node_feats=node_feats, sc=sc, node_attrs=atom_types)  # fp32 [N, C]
            node_feats_list.append(node_feats)
            if not fused_readout:
                heads = zero_heads if node_heads is None else node_heads
                node_es_list.append(_select_head(readout(node_feats.double(), heads), heads))

        if fused_readout:
            act_cst, scale, shift = self.readout_constants
            node_inter_es, node_feats_out = ReadoutEnergyAutograd.apply(
                node_feats_list[0], node_feats_list[1], self.readout_w1, self.readout_W2a, self.readout_w2b, act_cst, scale, shift,
                None if node_rows is None else node_rows[0])
        else:
            node_feats_out = torch.cat([f.double() for f in node_feats_list], dim=-1)
            if node_rows is not None:
                node_feats_out = node_feats_out.index_select(0, node_rows[1])
            node_inter_es = torch.sum(torch.stack(node_es_list, dim=0), dim=0)
            node_inter_es = self.scale_shift(node_inter_es, zero_heads if node_heads is None else node_heads)
        weighted_es = node_inter_es.double() if node_weights is None else node_inter_es.double() * node_weights
        inter_e = scatter_sum(src=weighted_es, index=batch, dim=-1, dim_size=num_graphs, ptr=data["ptr"])

        total_energy = graph_e0() + inter_e
        node_energy = node_e0 + node_inter_es
        if node_rows is not None:  # node_feats is already written in the caller's order
            node_energy = node_energy.index_select(0, node_rows[1])

        forces, virials, stress, hessian, edge_forces = get_outputs(
            energy=inter_e, positions=data["positions"], displacement=displacement, cell=cell, training=training,
            compute_force=compute_force, compute_virials=compute_virials, compute_stress=compute_stress)
        if node_rows is not None and not positions_in_caller_order and forces is not None:
            forces = forces.index_select(0, node_rows[1])

        return {
            "energy": total_energy, "node_energy": node_energy, "interaction_energy": inter_e, "forces": forces,
            "virials": virials, "stress": stress, "hessian": hessian, "displacement": displacement,
            "node_feats": node_feats_out, "edge_forces": edge_forces,
        }
