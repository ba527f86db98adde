"""The whole energy + forces step as one call into the library (cm_mace_step): the kernels of the forward and of the
backward chain are enqueued by the C side, with no interpreter or autograd engine between the launches.

`NativeStep` gathers what that call needs from an `OptimizedInvariantMACE`: the frozen weights as one C struct (built
once per model), the index structures of a neighbour list and species tensor as another (built once per list), and a
workspace that is reused from step to step.  Same kernels, same order, same numbers as the autograd path of the model.
"""
from __future__ import annotations

import ctypes
from typing import Dict, Optional

import numpy as np
import torch

from .. import _cabi as cabi
from ._autograd import _cached, csr_of, groups_of, groups_of_one_hot, sender_view_of

_fp = ctypes.c_void_p


class _Weights(ctypes.Structure):
    _fields_ = [
        ("channels", ctypes.c_int), ("nelements", ctypes.c_int), ("nknots", ctypes.c_int), ("hidden", ctypes.c_int),
        ("r_width", ctypes.c_float), ("r_max", ctypes.c_float),
        ("r_knots", _fp), ("spline", _fp * 2), ("mix_WT", _fp * 2), ("mix_W", _fp * 2), ("mix_scale", ctypes.c_float * 2),
        ("T3", _fp * 2), ("T2", _fp * 2), ("T1", _fp * 2), ("mono3", _fp * 2), ("mono2", _fp * 2),
        ("n3", ctypes.c_int * 2), ("n2", ctypes.c_int * 2),
        ("prod_WT", _fp * 2), ("prod_W", _fp * 2), ("up_WT", _fp), ("up_W", _fp), ("skip_WT", _fp), ("skip_W", _fp),
        ("skip_scale", ctypes.c_float), ("w1", _fp), ("W2a", _fp), ("w2b", _fp),
        ("act_cst", ctypes.c_double), ("scale", ctypes.c_double), ("shift", ctypes.c_double),
    ]


class _Graph(ctypes.Structure):
    _fields_ = [
        ("nnodes", ctypes.c_int64), ("nedges", ctypes.c_int64), ("ngraphs", ctypes.c_int),
        ("receiver", _fp), ("sender", _fp), ("first_occ", _fp), ("sender_perm", _fp), ("sender_offsets", _fp),
        ("elem_perm", _fp), ("elem_offsets", _fp), ("onehot_perm", _fp), ("onehot_offsets", _fp),
        ("node_rows", _fp), ("graph_ptr", _fp), ("X1", _fp), ("node_weights", _fp), ("node_e0", _fp), ("graph_e0", _fp),
    ]



def _ptr(t: Optional[torch.Tensor], dtype, name: str):
    return cabi._dev(t, dtype, name)


class NativeStep:
    """Built from a model whose three fusions are on (radial spline and harmonics inside message passing, linear +
    contraction, readouts); `supported(model)` tells.  Keeps references to every tensor whose address the structs hold."""

    @staticmethod
    def supported(model) -> bool:
        return bool(model.fused_radial and model.fused_contraction and model.fused_readout
                    and all(getattr(lin, "on_kernel", False) for lin in
                            (model.products[0].linear, model.products[1].linear, model.interactions[1].linear_up)))

    def __init__(self, model):
        F32, F64, I32 = torch.float32, torch.float64, torch.int32
        i0, i1 = model.interactions
        sp0, sp1 = model.edge_splines
        C = int(i1.linear_up.weights.shape[0])
        w = _Weights()
        keep = []

        def hold(t, dtype, name):
            t = t.contiguous()
            keep.append(t)
            return _ptr(t, dtype, name)

        w.channels, w.nelements = C, int(i0.composed_weights.shape[0])
        w.nknots = int(sp0.r_knots.numel())
        w.r_width, w.r_max = float(sp0._h), float(sp0._rmax)
        if not (torch.equal(sp0.r_knots, sp1.r_knots) and sp0._h == sp1._h and sp0._rmax == sp1._rmax):
            raise RuntimeError("native step: both layers must share the spline knots")
        w.r_knots = hold(sp0.r_knots, F32, "r_knots")
        for t, sp in enumerate((sp0, sp1)):
            w.spline[t] = hold(sp.coefficients, F32, "spline coefficients")
        for t, inter in enumerate((i0, i1)):
            W_T, W, scale, per_element = inter.fused_linear()
            if per_element != (t == 0):
                raise RuntimeError("native step: per-element channel mixing is expected in the first layer only")
            w.mix_WT[t], w.mix_W[t], w.mix_scale[t] = hold(W_T, F32, "mix_WT"), hold(W, F32, "mix_W"), float(scale)
            mono3, mono2, T3, T2, T1, builtin = model._contraction_tables(t)
            w.T3[t], w.T2[t], w.T1[t] = hold(T3, F32, "T3"), hold(T2, F32, "T2"), hold(T1, F32, "T1")
            w.n3[t], w.n2[t] = int(mono3.numel()), int(mono2.numel())
            w.mono3[t] = None if builtin else hold(mono3, I32, "mono3")
            w.mono2[t] = None if builtin else hold(mono2, I32, "mono2")
            lin = model.products[t].linear
            w.prod_WT[t], w.prod_W[t] = hold(lin.weights_transposed, F32, "prod_WT"), hold(lin.weights, F32, "prod_W")
        w.up_WT, w.up_W = hold(i1.linear_up.weights_transposed, F32, "up_WT"), hold(i1.linear_up.weights, F32, "up_W")
        w.skip_WT, w.skip_W = hold(i1.skip_tp.weights_transposed, F32, "skip_WT"), hold(i1.skip_tp.weights, F32, "skip_W")
        # 1/sqrt(K) in single precision, as the ElementalLinear class forms it: the two paths then agree to the bit
        w.skip_scale = float(np.float32(1.0) / np.sqrt(np.float32(i1.skip_tp.weights.shape[-2])))
        w.w1, w.W2a, w.w2b = hold(model.readout_w1, F64, "w1"), hold(model.readout_W2a, F64, "W2a"), hold(model.readout_w2b, F64, "w2b")
        w.hidden = int(model.readout_W2a.shape[1])
        w.act_cst, w.scale, w.shift = (float(v) for v in model.readout_constants)
        self.weights, self._keep, self.channels, self.nelements = w, keep, C, w.nelements
        self._workspace = None

    def graph(self, edge_index, receiver, sender, node_attrs32, atom_types, ptr, X1, node_rows, node_e0=None,
              graph_e0=None) -> "_GraphHandle":
        """Struct of the index structures of one neighbour list + species tensor (all cached on those tensors).
        node_e0 fp64 [N] (order of the lists) / graph_e0 fp64 [ngraphs]: what the step adds to the interaction part in its
        "energy" and (caller-ordered) "node_energy" outputs; None counts as zeros."""
        N = int(node_attrs32.shape[0])
        g = _Graph()
        I32 = torch.int32
        first_occ = csr_of(receiver, N)
        sperm, soff = sender_view_of(sender, N)
        eperm, eoff = groups_of(atom_types, self.nelements)
        operm, ooff = groups_of_one_hot(node_attrs32)
        ptr32 = _cached(ptr, "_cm_ptr32", None, lambda: ptr.int().contiguous())
        X1 = X1.contiguous()
        g.nnodes, g.nedges, g.ngraphs = N, int(receiver.numel()), int(ptr.numel()) - 1
        g.receiver, g.sender, g.first_occ = _ptr(receiver, I32, "receiver"), _ptr(sender, I32, "sender"), _ptr(first_occ, I32, "first_occ")
        g.sender_perm, g.sender_offsets = _ptr(sperm, I32, "sender_perm"), _ptr(soff, I32, "sender_offsets")
        g.elem_perm, g.elem_offsets = _ptr(eperm, I32, "elem_perm"), _ptr(eoff, I32, "elem_offsets")
        g.onehot_perm, g.onehot_offsets = _ptr(operm, I32, "onehot_perm"), _ptr(ooff, I32, "onehot_offsets")
        g.node_rows = _ptr(node_rows, I32, "node_rows") if node_rows is not None else None
        g.graph_ptr, g.X1 = _ptr(ptr32, I32, "graph_ptr"), _ptr(X1, torch.float32, "X1")
        g.node_weights = None
        F64 = torch.float64
        if node_e0 is not None:
            node_e0 = node_e0.detach().to(F64).contiguous()
            if node_e0.shape != (N,):
                raise cabi.CudaMaceError("native step: node_e0 must be [%d]" % N)
        if graph_e0 is not None:
            graph_e0 = graph_e0.detach().to(F64).contiguous()
            if graph_e0.shape != (int(g.ngraphs),):
                raise cabi.CudaMaceError("native step: graph_e0 must be [%d]" % int(g.ngraphs))
        g.node_e0 = _ptr(node_e0, F64, "node_e0") if node_e0 is not None else None
        g.graph_e0 = _ptr(graph_e0, F64, "graph_e0") if graph_e0 is not None else None
        return _GraphHandle(g, (receiver, sender, first_occ, sperm, soff, eperm, eoff, operm, ooff, ptr32, X1, node_rows, node_e0,
                                graph_e0))

    def __call__(self, handle: "_GraphHandle", positions: torch.Tensor, shifts: torch.Tensor, want_feats: bool = True,
                 want_virials: bool = False) -> Dict[str, torch.Tensor]:
        g = handle.struct
        N, E, C = int(g.nnodes), int(g.nedges), self.channels
        dev = positions.device
        F64 = torch.float64
        pos64 = positions.detach().to(F64).contiguous()
        sh64 = shifts.detach().to(F64).contiguous()
        if pos64.shape != (N, 3) or sh64.shape != (E, 3):
            raise cabi.CudaMaceError("native step: positions must be [%d, 3] and shifts [%d, 3]" % (N, E))
        need = cabi.lib.cm_mace_step_workspace(N, E, C)
        if torch.cuda.is_current_stream_capturing():
            # A captured step keeps the address it was recorded with for as long as its graph lives: its workspace comes
            # from the capture's own memory pool (which the graph owns), never from the buffer eager calls share, which a
            # later, larger evaluation replaces.
            ws = torch.empty(need, dtype=torch.uint8, device=dev)
        else:
            ws = self._workspace
            if ws is None or ws.numel() < need or ws.device != dev:
                ws = self._workspace = torch.empty(need, dtype=torch.uint8, device=dev)
        energy = torch.empty(int(g.ngraphs), dtype=F64, device=dev)
        node_energy = torch.empty(N, dtype=F64, device=dev)
        forces = torch.empty(N, 3, dtype=F64, device=dev)
        feats = torch.empty(N, 2 * C, dtype=F64, device=dev) if want_feats else None
        virials = torch.empty(int(g.ngraphs), 3, 3, dtype=F64, device=dev) if want_virials else None
        total = torch.empty(int(g.ngraphs), dtype=F64, device=dev)
        node_total = torch.empty(N, dtype=F64, device=dev)
        cabi._check(cabi.lib.cm_mace_step(
            ctypes.addressof(self.weights), ctypes.addressof(g), _ptr(pos64, F64, "positions"), _ptr(sh64, F64, "shifts"),
            ws.data_ptr(), ws.numel(), _ptr(energy, F64, "energy"), _ptr(node_energy, F64, "node_energy"),
            _ptr(forces, F64, "forces"), _ptr(feats, F64, "node_feats") if want_feats else None,
            _ptr(virials, F64, "virials") if want_virials else None, _ptr(total, F64, "total_energy"),
            _ptr(node_total, F64, "total_node_energy"), cabi._stream()))
        # energy / node_energy: the interaction part plus the handle's graph_e0 / node_e0, node_energy in the caller's
        # order (rows node_rows of the handle); interaction_node_energy: the interaction part alone, in list order
        return {"interaction_energy": energy, "interaction_node_energy": node_energy, "energy": total, "node_energy": node_total,
                "forces": forces, "node_feats": feats, "virials": virials}


class _GraphHandle:
    def __init__(self, struct, keep):
        self.struct, self._keep = struct, keep

    def with_node_weights(self, weights: torch.Tensor, graph_e0: Optional[torch.Tensor] = None) -> "_GraphHandle":
        """The same index structures with a weight per node energy (fp64 [nnodes], in the order of the lists): the step
        then returns sum_n weights[n] * node_energy[n] per graph and minus its gradient.  graph_e0: the constant per
        graph that goes with these weights (None keeps the handle's)."""
        if weights.shape != (int(self.struct.nnodes),):
            raise cabi.CudaMaceError("node weights must be [%d]" % int(self.struct.nnodes))
        g = _Graph()
        ctypes.memmove(ctypes.addressof(g), ctypes.addressof(self.struct), ctypes.sizeof(_Graph))
        w = weights.detach().to(torch.float64).contiguous()
        g.node_weights = _ptr(w, torch.float64, "node_weights")
        if graph_e0 is not None:
            graph_e0 = graph_e0.detach().to(torch.float64).contiguous()
            if graph_e0.shape != (int(g.ngraphs),):
                raise cabi.CudaMaceError("graph_e0 must be [%d]" % int(g.ngraphs))
            g.graph_e0 = _ptr(graph_e0, torch.float64, "graph_e0")
        return _GraphHandle(g, (self._keep, w, graph_e0))
