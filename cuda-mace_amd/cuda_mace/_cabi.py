"""ctypes binding of libcuda_mace_hip.so (the C ABI declared in include/cuda_mace_hip.h).

Torch is used only to own device memory and to name the current HIP stream; every compute call
goes through the C entry points.  There is no fallback: if the library is missing the import
fails, and if a call is given host tensors it raises.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional

import torch

_HERE = os.path.realpath(os.path.dirname(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libcuda_mace_hip.so")

if not os.path.isfile(LIB_PATH):
    raise ImportError(
        "Could not find the HIP kernel library at %s; build it with `python cuda-mace_amd/build.py`" % LIB_PATH
    )

lib = ctypes.CDLL(LIB_PATH)

_p = ctypes.c_void_p
_i64 = ctypes.c_int64
_i32 = ctypes.c_int
_f32 = ctypes.c_float
_sz = ctypes.c_size_t
_f64 = ctypes.c_double

# name -> (restype, argtypes); mirrors include/cuda_mace_hip.h one to one
SIGNATURES = {
    "cm_abi_version": (_i32, []),
    "cm_last_error": (ctypes.c_char_p, []),
    "cm_channels_supported": (_i32, [_i32]),
    "cm_trace_enabled": (_i32, []),
    "cm_trace_push": (None, [ctypes.c_char_p]),
    "cm_trace_pop": (None, []),
    "cm_first_occurences": (_i32, [_p, _i64, _i64, _p, _p]),
    "cm_receiver_list_status": (_i32, [_p, _i64, _i64, _p, _p]),
    "cm_stable_key_sort_workspace": (_sz, [_i64, _i64]),
    "cm_stable_key_sort": (_i32, [_p, _i64, _i64, _p, _p, _p, _sz, _p]),
    "cm_stable_key_sort_static_capacity": (_sz, []),
    "cm_stable_key_sort_static": (_i32, [_p, _i64, _i64, _p, _p, _p]),
    "cm_mp_forward": (_i32, [_p, _p, _p, _p, _p, _i64, _i64, _i32, _p, _p]),
    "cm_mp_backward": (_i32, [_p] * 8 + [_i64, _i64, _i32] + [_p] * 5),
    "cm_mp_forward_per_m": (_i32, [_p, _p, _p, _p, _p, _i64, _i64, _i32, _p, _p]),
    "cm_mp_backward_per_m": (_i32, [_p] * 8 + [_i64, _i64, _i32] + [_p] * 5),
    "cm_mp_spline_forward": (_i32, [_p] * 5 + [_i32, _f32, _f32, _p, _p, _i64, _i64, _i32, _p, _p]),
    "cm_mp_spline_backward": (_i32, [_p] * 5 + [_i32, _f32, _f32] + [_p] * 5 + [_i64, _i64, _i32] + [_p] * 5),
    "cm_mp_edge_forward": (_i32, [_p] * 4 + [_i32, _f32, _f32, _p, _p, _i64, _i64, _i32, _p, _p]),
    "cm_mp_edge_backward": (_i32, [_p] * 4 + [_i32, _f32, _f32] + [_p] * 5 + [_i64, _i64, _i32] + [_p] * 4),
    "cm_edge_geometry_forward": (_i32, [_p, _p, _p, _p, _p, _i64, _i64, _p, _p, _p]),
    "cm_edge_geometry_backward": (_i32, [_p] * 10 + [_i64, _i64, _p, _p, _p]),
    "cm_sh_forward": (_i32, [_p, _i64, _p, _p]),
    "cm_sh_backward": (_i32, [_p, _p, _i64, _p, _p]),
    "cm_spline_forward": (_i32, [_p, _p, _p, _i64, _i32, _i32, _f32, _f32, _p, _p, _p]),
    "cm_spline_backward": (_i32, [_p, _p, _p, _p, _i64, _i32, _i32, _f32, _f32, _p, _p]),
    "cm_linear": (_i32, [_p, _p, _p, _p, _i64, _i32, _i32, _i32, _i32, _i32, _f32, _p, _p, _p, _p]),
    "cm_symcon_tables": (_i32, [_p, _p, _p, _i32, _p, _p, _p, _i32, _p, _p, _p, _i32, _i32, _i32, _i32, _i32, _p, _p, _p, _p]),
    "cm_symcon_forward": (_i32, [_p, _p, _p, _p, _i32, _p, _i32, _p, _p, _p, _i64, _i32, _i32, _p, _p, _p]),
    "cm_symcon_builtin_structure": (_i32, [_p, _i32, _p, _i32, _p, _p]),
    "cm_symcon_backward": (_i32, [_p, _p, _i64, _i32, _p, _p]),
    "cm_readout_forward": (_i32, [_p] * 5 + [_f64, _f64, _f64, _i64, _i32, _i32, _p, _p, _p, _p, _p]),
    "cm_readout_backward": (_i32, [_p, _p, _p, _f64, _i64, _i32, _p, _p, _p]),
    "cm_graph_prepare_workspace": (_sz, [_i64, _i64, _i32, _i32]),
    "cm_graph_prepare": (_i32, [_p] * 5 + [_i64, _i64, _i32, _f64, _i32] + [_p] * 10 + [_sz, _p]),
    "cm_node_glue_supported": (_i32, [_i32]),
    "cm_node_glue_forward": (_i32, [_p] * 6 + [_i64, _i32, _i32, _f32, _p, _p, _p, _p]),
    "cm_node_glue_backward": (_i32, [_p] * 6 + [_f64, _p, _p, _p, _i64, _i32, _i32, _f32, _p, _p]),
    "cm_neighbour_list_workspace": (_sz, [_i64, _i64]),
    "cm_neighbour_list_count": (_i32, [_p, _p, _i32, _i32, _i32, _f64, _i64, _i64, _p, _sz, _p, _p, _p]),
    "cm_neighbour_list_fill": (_i32, [_p, _f64, _i64, _i64, _p, _p, _i64, _p, _p, _p, _p, _p]),
    "cm_max_displacement": (_i32, [_p, _p, _i64, _p, _p]),
    # the whole step: (weights struct *, graph struct *, positions, shifts, workspace, bytes, 4 outputs, stream)
    "cm_mace_step_timing": (_i32, [ctypes.c_uint]),
    "cm_probe_fma": (_i32, [_p, _i32, _i32, _p]),
    "cm_mace_step_timing_read": (_i32, [_p, _p, _i32]),
    "cm_mace_step_workspace": (_sz, [_i64, _i64, _i32]),
    "cm_mace_step": (_i32, [_p, _p, _p, _p, _p, _sz, _p, _p, _p, _p, _p, _p, _p, _p]),
    # fp64 instantiations: same argument lists, floating-point buffers in double
    "cm_mp_forward_f64": (_i32, [_p, _p, _p, _p, _p, _i64, _i64, _i32, _p, _p]),
    "cm_mp_backward_f64": (_i32, [_p] * 8 + [_i64, _i64, _i32] + [_p] * 5),
    "cm_sh_forward_f64": (_i32, [_p, _i64, _p, _p]),
    "cm_sh_backward_f64": (_i32, [_p, _p, _i64, _p, _p]),
    "cm_spline_forward_f64": (_i32, [_p, _p, _p, _i64, _i32, _i32, _f64, _f64, _p, _p, _p]),
    "cm_spline_backward_f64": (_i32, [_p, _p, _p, _p, _i64, _i32, _i32, _f64, _f64, _p, _p]),
    "cm_symcon_tables_f64": (_i32, [_p, _p, _p, _i32, _p, _p, _p, _i32, _p, _p, _p, _i32, _i32, _i32, _i32, _i32, _p, _p, _p, _p]),
    "cm_symcon_forward_f64": (_i32, [_p, _p, _p, _p, _i32, _p, _i32, _p, _p, _p, _i64, _i32, _i32, _p, _p, _p]),
    "cm_symcon_backward_f64": (_i32, [_p, _p, _i64, _i32, _p, _p]),
}

for _name, (_res, _args) in SIGNATURES.items():
    _fn = getattr(lib, _name)
    _fn.restype = _res
    _fn.argtypes = _args


class CudaMaceError(RuntimeError):
    pass


def _check(rc: int) -> None:
    if rc != 0:
        raise CudaMaceError("%s (code %d)" % (lib.cm_last_error().decode(), rc))


def _dev(t: Optional[torch.Tensor], dtype: torch.dtype, name: str) -> Optional[int]:
    """Device address of a contiguous tensor after checking what the C side assumes."""
    if t is None:
        return None
    if not t.is_cuda:
        raise CudaMaceError("%s must live on the GPU (got a %s tensor)" % (name, t.device))
    if t.dtype != dtype:
        raise CudaMaceError("%s must be %s (got %s)" % (name, dtype, t.dtype))
    if not t.is_contiguous():
        raise CudaMaceError("%s must be contiguous" % name)
    return t.data_ptr() if t.numel() > 0 else None


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_get_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream() -> int:
    """Handle of torch's current HIP stream on the current device (the raw query: this runs once per kernel launch and
    the public accessor costs ten times as much on the host)."""
    if _raw_stream is not None and _get_device is not None:
        return _raw_stream(_get_device())
    return torch.cuda.current_stream().cuda_stream


F32, F64, I32 = torch.float32, torch.float64, torch.int32


def _typed(name: str, like: torch.Tensor):
    """(entry point, dtype) for the precision of `like`: `name` for fp32 tensors, `name`_f64 for fp64 ones (message
    passing, harmonics, spline and contraction exist in both, as in the reference)."""
    if like.dtype == F64:
        return getattr(lib, name + "_f64"), F64
    return getattr(lib, name), F32


# ---- index kernels ---------------------------------------------------------------------------
DEBUG = os.environ.get("CUDA_MACE_DEBUG", "0") not in ("", "0")


def receiver_list_status(receiver: torch.Tensor, nnodes: int):
    """(decreases somewhere, holds a value outside [0, nnodes)) for a receiver list; synchronises."""
    status = torch.empty(2, dtype=I32, device=receiver.device)
    _check(lib.cm_receiver_list_status(_dev(receiver, I32, "receiver_list"), receiver.numel(), nnodes, _dev(status, I32, "status"), _stream()))
    unsorted, out_of_range = status.tolist()
    return bool(unsorted), bool(out_of_range)


def first_occurences(receiver: torch.Tensor, nnodes: int) -> torch.Tensor:
    """CSR offsets of a non-decreasing receiver list.  With CUDA_MACE_DEBUG set the list is checked first (one host
    synchronisation) and a list that is unsorted or out of range raises instead of giving wrong sums."""
    if DEBUG:
        unsorted, out_of_range = receiver_list_status(receiver, nnodes)
        if unsorted or out_of_range:
            raise CudaMaceError("receiver_list must be non-decreasing with values in [0, %d): %s" % (
                nnodes, " and ".join(w for w, on in (("it decreases somewhere", unsorted), ("it holds values out of range", out_of_range)) if on)))
    out = torch.empty(2 * nnodes, dtype=I32, device=receiver.device)
    _check(lib.cm_first_occurences(_dev(receiver, I32, "receiver_list"), receiver.numel(), nnodes, _dev(out, I32, "out"), _stream()))
    return out


def stable_key_sort(keys: torch.Tensor, nkeys: int):
    n = keys.numel()
    perm = torch.empty(n, dtype=I32, device=keys.device)
    offsets = torch.empty(nkeys + 1, dtype=I32, device=keys.device)
    nbytes = lib.cm_stable_key_sort_workspace(n, nkeys)
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=keys.device)
    _check(
        lib.cm_stable_key_sort(
            _dev(keys, I32, "keys"), n, nkeys, _dev(perm, I32, "perm"), _dev(offsets, I32, "offsets"),
            ws.data_ptr(), nbytes, _stream(),
        )
    )
    return perm, offsets


def stable_key_sort_static(keys: torch.Tensor, nkeys: int, perm: torch.Tensor, offsets: torch.Tensor) -> None:
    """cm_stable_key_sort_static: the same sort into caller-provided `perm` [n] and `offsets` [nkeys + 1], with the
    library's built-in scratch buffer in place of a workspace, so nothing is allocated.  Raises when the sizes exceed
    that buffer.  Calls on one GPU share the buffer and must not overlap."""
    n = keys.numel()
    if perm.numel() != n or offsets.numel() != nkeys + 1:
        raise CudaMaceError("perm must hold n = %d and offsets nkeys + 1 = %d entries" % (n, nkeys + 1))
    _check(
        lib.cm_stable_key_sort_static(
            _dev(keys, I32, "keys"), n, nkeys, _dev(perm, I32, "perm"), _dev(offsets, I32, "offsets"), _stream()
        )
    )


def graph_prepare(positions: torch.Tensor, row_i: torch.Tensor, row_j: torch.Tensor, shifts: torch.Tensor,
                  graph_of_node: Optional[torch.Tensor], ngraphs: int, r_max: float, bins: int) -> dict:
    """cm_graph_prepare: the spatially ordered, shell-last copy of a neighbour list with its CSR offsets and its view sorted
    by sender, in one call without a host synchronisation.  Returns a dict of int32 tensors (node_perm, node_inverse,
    receiver, sender, edge_perm, first_occ, sender_perm, sender_offsets) and shifts (fp64 [E, 3], reordered)."""
    N, E = positions.shape[0], row_i.numel()
    dev = positions.device
    i32 = lambda n: torch.empty(n, dtype=I32, device=dev)  # noqa: E731
    out = {"node_perm": i32(N), "node_inverse": i32(N), "receiver": i32(E), "sender": i32(E), "edge_perm": i32(E),
           "shifts": torch.empty(E, 3, dtype=F64, device=dev), "first_occ": i32(2 * N), "sender_perm": i32(E),
           "sender_offsets": i32(N + 1)}
    need = lib.cm_graph_prepare_workspace(N, E, int(ngraphs), int(bins))
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)
    _check(lib.cm_graph_prepare(
        _dev(positions, F64, "positions"), _dev(row_i, I32, "row_i"), _dev(row_j, I32, "row_j"), _dev(shifts, F64, "shifts"),
        _dev(graph_of_node, I32, "graph_of_node"), N, E, int(ngraphs), float(r_max), int(bins),
        _dev(out["node_perm"], I32, "node_perm"), _dev(out["node_inverse"], I32, "node_inverse"),
        _dev(out["receiver"], I32, "receiver"), _dev(out["sender"], I32, "sender"), _dev(out["edge_perm"], I32, "edge_perm"),
        _dev(out["shifts"], F64, "shifts_out"), _dev(out["first_occ"], I32, "first_occ"),
        _dev(out["sender_perm"], I32, "sender_perm"), _dev(out["sender_offsets"], I32, "sender_offsets"),
        ws.data_ptr(), ws.numel(), _stream()))
    return out


# ---- message passing --------------------------------------------------------------------------
def _radial_blocks(R, E: int, C: int, D) -> int:
    """4 for radial weights per degree (the reference's [nedges, 4, C]), 16 for weights per component ([nedges, 16, C],
    fp32 only)."""
    if R.numel() == E * 4 * C and not (R.dim() == 3 and R.shape[1] == 16):
        return 4
    if R.numel() == E * 16 * C and D == F32:
        return 16
    raise CudaMaceError("radial must hold nedges*4*channels = %d values (or nedges*16*channels in fp32), got %d" % (E * 4 * C, R.numel()))


def mp_forward(X, Y, R, sender, first_occ, nnodes: int) -> torch.Tensor:
    fn, D = _typed("cm_mp_forward", X)
    C = X.shape[-1]
    E = sender.numel()
    if Y.shape != (16, E):
        raise CudaMaceError("Y must be [16, nedges] = [16, %d], got %s" % (E, tuple(Y.shape)))
    if _radial_blocks(R, E, C, D) == 16:
        fn = lib.cm_mp_forward_per_m
    if X.shape[0] != nnodes:
        raise CudaMaceError("X must be [nnodes, channels]")
    out = torch.empty(nnodes, 16, C, dtype=D, device=X.device)
    _check(
        fn(
            _dev(X, D, "X"), _dev(Y, D, "Y"), _dev(R, D, "radial"), _dev(sender, I32, "sender_list"),
            _dev(first_occ, I32, "first_occurences"), nnodes, E, C, _dev(out, D, "out"), _stream(),
        )
    )
    return out


def mp_backward(X, Y, R, grad_out, sender, first_occ, sender_perm, sender_offsets, nnodes: int,
                need_gX: bool = True, need_gY: bool = True, need_gR: bool = True):
    fn, D = _typed("cm_mp_backward", X)
    C = X.shape[-1]
    E = sender.numel()
    dev = X.device
    blocks = _radial_blocks(R, E, C, D)
    if blocks == 16:
        fn = lib.cm_mp_backward_per_m
    gX = torch.empty(nnodes, C, dtype=D, device=dev) if need_gX else None
    gY = torch.empty(16, E, dtype=D, device=dev) if need_gY else None
    gR = torch.empty(E, blocks, C, dtype=D, device=dev) if need_gR else None
    scratch = torch.empty(E, C, dtype=D, device=dev) if need_gX else None
    _check(
        fn(
            _dev(X, D, "X"), _dev(Y, D, "Y"), _dev(R, D, "radial"), _dev(grad_out, D, "grad_out"),
            _dev(sender, I32, "sender_list"), _dev(first_occ, I32, "first_occurences"),
            _dev(sender_perm, I32, "sender_perm") if need_gX else None,
            _dev(sender_offsets, I32, "sender_offsets") if need_gX else None,
            nnodes, E, C, _dev(gX, D, "gX"), _dev(gY, D, "gY"), _dev(gR, D, "gR"), _dev(scratch, D, "scratch"), _stream(),
        )
    )
    return gX, gY, gR


def mp_spline_forward(X, Y, r, r_knots, coeffs, r_width: float, r_max: float, sender, first_occ, nnodes: int) -> torch.Tensor:
    C = X.shape[-1]
    E = sender.numel()
    if Y.shape != (16, E) or r.numel() != E:
        raise CudaMaceError("Y must be [16, nedges] and r [nedges] with nedges = %d" % E)
    if coeffs.shape != (r_knots.numel() - 1, 4, 4 * C):
        raise CudaMaceError("coeffs must be [nknots-1, 4, 4*channels] = %s, got %s" % ((r_knots.numel() - 1, 4, 4 * C), tuple(coeffs.shape)))
    out = torch.empty(nnodes, 16, C, dtype=F32, device=X.device)
    _check(
        lib.cm_mp_spline_forward(
            _dev(X, F32, "X"), _dev(Y, F32, "Y"), _dev(r, F32, "r"), _dev(r_knots, F32, "r_knots"), _dev(coeffs, F32, "coeffs"),
            r_knots.numel(), float(r_width), float(r_max), _dev(sender, I32, "sender_list"),
            _dev(first_occ, I32, "first_occurences"), nnodes, E, C, _dev(out, F32, "out"), _stream(),
        )
    )
    return out


def mp_spline_backward(X, Y, r, r_knots, coeffs, r_width: float, r_max: float, grad_out, sender, first_occ, sender_perm,
                       sender_offsets, nnodes: int, need_gX: bool = True, need_gY: bool = True, need_gr: bool = True):
    C = X.shape[-1]
    E = sender.numel()
    dev = X.device
    gX = torch.empty(nnodes, C, dtype=F32, device=dev) if need_gX else None
    gY = torch.empty(16, E, dtype=F32, device=dev) if need_gY else None
    gr = torch.empty(E, dtype=F32, device=dev) if need_gr else None
    scratch = torch.empty(E, C, dtype=F32, device=dev) if need_gX else None
    _check(
        lib.cm_mp_spline_backward(
            _dev(X, F32, "X"), _dev(Y, F32, "Y"), _dev(r, F32, "r"), _dev(r_knots, F32, "r_knots"), _dev(coeffs, F32, "coeffs"),
            r_knots.numel(), float(r_width), float(r_max), _dev(grad_out, F32, "grad_out"), _dev(sender, I32, "sender_list"),
            _dev(first_occ, I32, "first_occurences"), _dev(sender_perm, I32, "sender_perm") if need_gX else None,
            _dev(sender_offsets, I32, "sender_offsets") if need_gX else None, nnodes, E, C,
            _dev(gX, F32, "gX"), _dev(gY, F32, "gY"), _dev(gr, F32, "grad_r"), _dev(scratch, F32, "scratch"), _stream(),
        )
    )
    return gX, gY, gr


def mp_edge_forward(X, vectors, r_knots, coeffs, r_width: float, r_max: float, sender, first_occ, nnodes: int) -> torch.Tensor:
    C = X.shape[-1]
    E = sender.numel()
    if vectors.shape != (E, 3):
        raise CudaMaceError("vectors must be [nedges, 3] with nedges = %d" % E)
    if coeffs.shape != (r_knots.numel() - 1, 4, 4 * C):
        raise CudaMaceError("coeffs must be [nknots-1, 4, 4*channels] = %s, got %s" % ((r_knots.numel() - 1, 4, 4 * C), tuple(coeffs.shape)))
    out = torch.empty(nnodes, 16, C, dtype=F32, device=X.device)
    _check(
        lib.cm_mp_edge_forward(
            _dev(X, F32, "X"), _dev(vectors, F32, "vectors"), _dev(r_knots, F32, "r_knots"), _dev(coeffs, F32, "coeffs"),
            r_knots.numel(), float(r_width), float(r_max), _dev(sender, I32, "sender_list"),
            _dev(first_occ, I32, "first_occurences"), nnodes, E, C, _dev(out, F32, "out"), _stream(),
        )
    )
    return out


def mp_edge_backward(X, vectors, r_knots, coeffs, r_width: float, r_max: float, grad_out, sender, first_occ, sender_perm,
                     sender_offsets, nnodes: int, need_gX: bool = True, need_gvec: bool = True):
    C = X.shape[-1]
    E = sender.numel()
    dev = X.device
    gX = torch.empty(nnodes, C, dtype=F32, device=dev) if need_gX else None
    gvec = torch.empty(E, 3, dtype=F32, device=dev) if need_gvec else None
    scratch = torch.empty(E, C, dtype=F32, device=dev) if need_gX else None
    _check(
        lib.cm_mp_edge_backward(
            _dev(X, F32, "X"), _dev(vectors, F32, "vectors"), _dev(r_knots, F32, "r_knots"), _dev(coeffs, F32, "coeffs"),
            r_knots.numel(), float(r_width), float(r_max), _dev(grad_out, F32, "grad_out"), _dev(sender, I32, "sender_list"),
            _dev(first_occ, I32, "first_occurences"), _dev(sender_perm, I32, "sender_perm") if need_gX else None,
            _dev(sender_offsets, I32, "sender_offsets") if need_gX else None, nnodes, E, C,
            _dev(gX, F32, "gX"), _dev(gvec, F32, "grad_vectors"), _dev(scratch, F32, "scratch"), _stream(),
        )
    )
    return gX, gvec


# ---- spherical harmonics ------------------------------------------------------------------------
def sh_forward(xyz: torch.Tensor) -> torch.Tensor:
    fn, D = _typed("cm_sh_forward", xyz)
    E = xyz.shape[0]
    Y = torch.empty(16, E, dtype=D, device=xyz.device)
    _check(fn(_dev(xyz, D, "xyz"), E, _dev(Y, D, "Y"), _stream()))
    return Y


def sh_backward(xyz: torch.Tensor, grad_Y: torch.Tensor) -> torch.Tensor:
    fn, D = _typed("cm_sh_backward", xyz)
    E = xyz.shape[0]
    g = torch.empty(E, 3, dtype=D, device=xyz.device)
    _check(fn(_dev(xyz, D, "xyz"), _dev(grad_Y, D, "grad_Y"), E, _dev(g, D, "grad_xyz"), _stream()))
    return g


# ---- edge geometry ------------------------------------------------------------------------------


def edge_geometry_forward(positions, row_a, row_b, shifts, node_rows=None):
    """node_rows int32 [N] (optional): atom n of the edge lists is row node_rows[n] of positions."""
    E = row_a.numel()
    dev = positions.device
    vec = torch.empty(E, 3, dtype=F32, device=dev)
    length = torch.empty(E, dtype=F32, device=dev)
    _check(
        lib.cm_edge_geometry_forward(
            _dev(positions, F64, "positions"), _dev(row_a, I32, "row_a"), _dev(row_b, I32, "row_b"),
            _dev(shifts, F64, "shifts"), _dev(node_rows, I32, "node_rows"), positions.shape[0], E, _dev(vec, F32, "vectors"),
            _dev(length, F32, "lengths"), _stream(),
        )
    )
    return vec, length


def edge_geometry_backward(positions, row_a, row_b, shifts, a_first_occ, b_perm, b_offsets, grad_vectors, grad_lengths,
                           need_positions: bool = True, need_shifts: bool = False, node_rows=None):
    E = row_a.numel()
    N = positions.shape[0]
    dev = positions.device
    gpos = torch.empty(N, 3, dtype=F64, device=dev) if need_positions else None
    gshift = torch.empty(E, 3, dtype=F64, device=dev) if need_shifts else None
    _check(
        lib.cm_edge_geometry_backward(
            _dev(positions, F64, "positions"), _dev(row_a, I32, "row_a"), _dev(row_b, I32, "row_b"),
            _dev(shifts, F64, "shifts"), _dev(node_rows, I32, "node_rows"), _dev(a_first_occ, I32, "a_first_occ"),
            _dev(b_perm, I32, "b_perm"),
            _dev(b_offsets, I32, "b_offsets"), _dev(grad_vectors, F32, "grad_vectors"),
            _dev(grad_lengths, F32, "grad_lengths"), N, E, _dev(gpos, F64, "grad_positions"),
            _dev(gshift, F64, "grad_shifts"), _stream(),
        )
    )
    return gpos, gshift


# ---- cubic spline ---------------------------------------------------------------------------------
def spline_forward(r, r_knots, coeffs, r_width: float, r_max: float, want_deriv: bool = False):
    fn, D = _typed("cm_spline_forward", r)
    E = r.numel()
    J = coeffs.shape[-1]
    nknots = r_knots.numel()
    if coeffs.shape[0] != nknots - 1 or coeffs.shape[1] != 4:
        raise CudaMaceError("coeffs must be [nknots-1, 4, noutputs]")
    R = torch.empty(E, J, dtype=D, device=r.device)
    dR = torch.empty(E, J, dtype=D, device=r.device) if want_deriv else None
    _check(
        fn(
            _dev(r, D, "r"), _dev(r_knots, D, "r_knots"), _dev(coeffs, D, "coeffs"), E, nknots, J,
            float(r_width), float(r_max), _dev(R, D, "R_out"), _dev(dR, D, "R_deriv"), _stream(),
        )
    )
    return (R, dR) if want_deriv else R


def spline_backward(r, r_knots, coeffs, grad_R, r_width: float, r_max: float) -> torch.Tensor:
    fn, D = _typed("cm_spline_backward", r)
    E = r.numel()
    J = coeffs.shape[-1]
    out = torch.empty(E, dtype=D, device=r.device)
    _check(
        fn(
            _dev(r, D, "r"), _dev(r_knots, D, "r_knots"), _dev(coeffs, D, "coeffs"), _dev(grad_R, D, "grad_R"),
            E, r_knots.numel(), J, float(r_width), float(r_max), _dev(out, D, "grad_r"), _stream(),
        )
    )
    return out


# ---- linears ------------------------------------------------------------------------------------------
def linear(X, W_T, node_perm=None, group_offsets=None, scale=None, zero_last_group: bool = False,
           row_scale=None, residual=None) -> torch.Tensor:
    """X [N,16,K] with W_T [(ngroups,)4,N',K], or scalar features X [N,K] with W_T [(ngroups,)N',K] (transposed weight
    blocks); scale defaults to 1/sqrt(K).  Grouped calls pass the node grouping; with zero_last_group the grouping has
    one more group than W_T, whose rows come out as zeros.  Rows of nodes in no group are left unwritten.
    row_scale [N,K]: X[n,m,k] is multiplied by row_scale[n,k] on the way in.  residual (shape of the result): added to
    the written rows."""
    scalar = X.dim() == 2
    if scalar:
        if W_T.dim() == 2:
            W_T = W_T.unsqueeze(0)
        ngroups, Nout, K = W_T.shape
        ncomp = 1
        ok = X.shape[1] == K
    else:
        if W_T.dim() == 3:
            W_T = W_T.unsqueeze(0)
        ngroups, four, Nout, K = W_T.shape
        ncomp = 16
        ok = four == 4 and X.dim() == 3 and X.shape[1] == 16 and X.shape[2] == K
    if not ok:
        raise CudaMaceError("linear: X must be [N,16,K] with W_T [(ngroups,)4,N',K], or [N,K] with W_T [(ngroups,)N',K]")
    N = X.shape[0]
    if row_scale is not None and tuple(row_scale.shape) != (N, K):
        raise CudaMaceError("linear: row_scale must be [N, K]")
    OUT = torch.empty((N, Nout) if scalar else (N, 16, Nout), dtype=F32, device=X.device)
    if residual is not None and tuple(residual.shape) != tuple(OUT.shape):
        raise CudaMaceError("linear: residual must have the shape of the result, %s" % (tuple(OUT.shape),))
    _check(
        lib.cm_linear(
            _dev(X, F32, "X"), _dev(W_T, F32, "W_T"), _dev(node_perm, I32, "node_perm"),
            _dev(group_offsets, I32, "group_offsets"), N, ngroups + (1 if zero_last_group else 0), int(zero_last_group), ncomp,
            K, Nout, float(scale) if scale is not None else 1.0 / float(K) ** 0.5, _dev(row_scale, F32, "row_scale"),
            _dev(residual, F32, "residual"), _dev(OUT, F32, "OUT"), _stream(),
        )
    )
    return OUT


def node_glue_forward(B1, prod_WT, skip_WT, up_WT, node_perm, group_offsets, skip_scale: float):
    """(h1, sc, X2) = (B1 . prod_W, skip_scale * h1 . skip_W[element], h1 . up_W) in one launch; weights transposed
    ([C out, C in], skip_WT [nelements, C, C]); the grouping has nelements + 1 groups, the last for nodes without an
    element (sc = 0 there)."""
    N, C = B1.shape
    ne = skip_WT.shape[0]
    if tuple(prod_WT.shape) != (C, C) or tuple(up_WT.shape) != (C, C) or tuple(skip_WT.shape) != (ne, C, C):
        raise CudaMaceError("node_glue_forward: weights must be [C, C], [nelements, C, C], [C, C]")
    if group_offsets.numel() != ne + 2 or node_perm.numel() != N:
        raise CudaMaceError("node_glue_forward: the grouping must list N nodes in nelements + 1 groups")
    h1, sc, X2 = (torch.empty(N, C, dtype=F32, device=B1.device) for _ in range(3))
    _check(lib.cm_node_glue_forward(_dev(B1, F32, "B1"), _dev(prod_WT, F32, "prod_WT"), _dev(skip_WT, F32, "skip_WT"),
                                    _dev(up_WT, F32, "up_WT"), _dev(node_perm, I32, "node_perm"),
                                    _dev(group_offsets, I32, "group_offsets"), N, ne + 1, C, float(skip_scale),
                                    _dev(h1, F32, "h1"), _dev(sc, F32, "sc"), _dev(X2, F32, "X2"), _stream()))
    return h1, sc, X2


def node_glue_backward(gX2, d_h2, up_W, skip_W, prod_W, w1, scale: float, node_weights, node_perm, group_offsets,
                       skip_scale: float):
    """gB1 = (gX2 . up_W^T + g1 - skip_scale * d_h2 . skip_W[element]^T) . prod_W^T with g1[n, c] = -node_weights[n] *
    scale * w1[c] (node_weights None = 1); weights plain ([C in, C out] passed as the transposes of the forward's)."""
    N, C = gX2.shape
    ne = skip_W.shape[0]
    if tuple(d_h2.shape) != (N, C) or tuple(up_W.shape) != (C, C) or tuple(prod_W.shape) != (C, C) or tuple(skip_W.shape) != (ne, C, C):
        raise CudaMaceError("node_glue_backward: operands must be [N, C] and weights [C, C], [nelements, C, C], [C, C]")
    if group_offsets.numel() != ne + 2 or node_perm.numel() != N or w1.numel() != C:
        raise CudaMaceError("node_glue_backward: the grouping must list N nodes in nelements + 1 groups, w1 holds C values")
    gB1 = torch.empty(N, C, dtype=F32, device=gX2.device)
    _check(lib.cm_node_glue_backward(_dev(gX2, F32, "gX2"), _dev(d_h2, F32, "d_h2"), _dev(up_W, F32, "up_W"),
                                     _dev(skip_W, F32, "skip_W"), _dev(prod_W, F32, "prod_W"), _dev(w1, F64, "w1"), float(scale),
                                     _dev(node_weights, F64, "node_weights"), _dev(node_perm, I32, "node_perm"),
                                     _dev(group_offsets, I32, "group_offsets"), N, ne + 1, C, float(skip_scale),
                                     _dev(gB1, F32, "gB1"), _stream()))
    return gB1


# ---- symmetric contraction -----------------------------------------------------------------------------
def symcon_tables(term3_off, term3_path, term3_val, term2_off, term2_path, term2_val, W3, W2, W1):
    fn, D = _typed("cm_symcon_tables", W3)
    ne, P3, C = W3.shape
    P2 = W2.shape[1]
    P1 = W1.shape[1]
    n3 = term3_off.numel() - 1
    n2 = term2_off.numel() - 1
    dev = W3.device
    T3 = torch.empty(ne, n3, C, dtype=D, device=dev)
    T2 = torch.empty(ne, n2, C, dtype=D, device=dev)
    T1 = torch.empty(ne, C, dtype=D, device=dev)
    _check(
        fn(
            _dev(term3_off, I32, "term3_off"), _dev(term3_path, I32, "term3_path"), _dev(term3_val, D, "term3_val"), n3,
            _dev(term2_off, I32, "term2_off"), _dev(term2_path, I32, "term2_path"), _dev(term2_val, D, "term2_val"), n2,
            _dev(W3, D, "W3"), _dev(W2, D, "W2"), _dev(W1, D, "W1"), ne, P3, P2, P1, C,
            _dev(T3, D, "T3"), _dev(T2, D, "T2"), _dev(T1, D, "T1"), _stream(),
        )
    )
    return T3, T2, T1


def symcon_builtin_structure():
    """(mono3, mono2) int32 numpy arrays of the monomial lists compiled into the library."""
    import numpy as np

    n3, n2 = ctypes.c_int(0), ctypes.c_int(0)
    _check(lib.cm_symcon_builtin_structure(None, 0, None, 0, ctypes.byref(n3), ctypes.byref(n2)))
    m3 = np.zeros(n3.value, dtype=np.int32)
    m2 = np.zeros(n2.value, dtype=np.int32)
    _check(lib.cm_symcon_builtin_structure(m3.ctypes.data, n3.value, m2.ctypes.data, n2.value, None, None))
    return m3, m2


def symcon_forward(X, node_perm, group_offsets, mono3, mono2, T3, T2, T1, want_grad: bool = True, builtin: bool = False,
                   zero_init: bool = True):
    """builtin=True: the monomial lists are the ones compiled into the library; the unrolled kernel is used.
    zero_init=False skips clearing the outputs: rows of nodes that are in no group are then undefined (every node is in
    a group when all element indices are in range)."""
    fn, D = _typed("cm_symcon_forward", X)
    N, sixteen, C = X.shape
    if sixteen != 16:
        raise CudaMaceError("symmetric contraction: X must be [N,16,C]")
    ne = T1.shape[0]
    alloc = torch.zeros if zero_init else torch.empty
    out = alloc(N, C, dtype=D, device=X.device)
    grad = alloc(N, 16, C, dtype=D, device=X.device) if want_grad else None
    _check(
        fn(
            _dev(X, D, "X"), _dev(node_perm, I32, "node_perm"), _dev(group_offsets, I32, "group_offsets"),
            None if builtin else _dev(mono3, I32, "mono3"), mono3.numel(),
            None if builtin else _dev(mono2, I32, "mono2"), mono2.numel(),
            _dev(T3, D, "T3"), _dev(T2, D, "T2"), _dev(T1, D, "T1"), N, ne, C,
            _dev(out, D, "out"), _dev(grad, D, "grad"), _stream(),
        )
    )
    return out, grad


def symcon_backward(grad, grad_out) -> torch.Tensor:
    fn, D = _typed("cm_symcon_backward", grad)
    N, _, C = grad.shape
    gX = torch.empty_like(grad)
    _check(fn(_dev(grad, D, "grad"), _dev(grad_out, D, "grad_out"), N, C, _dev(gX, D, "gX"), _stream()))
    return gX


# ---- neighbour list -------------------------------------------------------------------------------
def neighbour_list(positions, cell, pbc, cutoff: float, max_cells: int = 0):
    """(row_i int32 [E], row_j int32 [E], unit_shifts int32 [E, 3]) sorted by (i, j, S); positions fp64 [N, 3] and
    cell fp64 [3, 3] (or None) on the device, pbc three booleans.  One host synchronisation (the number of pairs)."""
    N = positions.shape[0]
    dev = positions.device
    max_cells = int(max_cells) if max_cells else max(1, min(N, 1 << 22))
    ws_bytes = lib.cm_neighbour_list_workspace(N, max_cells)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    head = torch.empty(N + 2, dtype=I32, device=dev)  # offsets [N + 1] followed by the status word
    px, py, pz = (int(bool(b)) for b in pbc)
    _check(
        lib.cm_neighbour_list_count(
            _dev(positions, F64, "positions"), _dev(cell, F64, "cell"), px, py, pz, float(cutoff), N, max_cells,
            ws.data_ptr(), ws_bytes, head.data_ptr(), head.data_ptr() + 4 * (N + 1), _stream(),
        )
    )
    E, status = (int(v) for v in head[N:].tolist())
    if status == 1:
        raise CudaMaceError("neighbour list: a periodic axis needs a non-singular cell")
    if status != 0:
        raise CudaMaceError("neighbour list: the cell is thinner than cutoff / 32 along a periodic axis")
    if E >= 2**31 // 4 - 1:
        raise CudaMaceError("neighbour list: more pairs than int32 indexing holds")
    row_i = torch.empty(E, dtype=I32, device=dev)
    row_j = torch.empty(E, dtype=I32, device=dev)
    S = torch.empty(E, 3, dtype=I32, device=dev)
    if E > 0:
        scratch = torch.empty(4 * E, dtype=I32, device=dev)
        _check(
            lib.cm_neighbour_list_fill(
                _dev(positions, F64, "positions"), float(cutoff), N, max_cells, ws.data_ptr(), head.data_ptr(), E,
                scratch.data_ptr(), row_i.data_ptr(), row_j.data_ptr(), S.data_ptr(), _stream(),
            )
        )
    return row_i, row_j, S


def max_displacement(positions, reference, out=None):
    """fp64 [1] on the device: the largest squared distance between the rows of `positions` and `reference` (fp64
    [N, 3]); nothing is read back here."""
    N = positions.shape[0]
    if reference.shape != positions.shape:
        raise CudaMaceError("max_displacement: positions and reference differ in shape")
    if out is None:
        out = torch.empty(1, dtype=F64, device=positions.device)
    _check(lib.cm_max_displacement(_dev(positions, F64, "positions"), _dev(reference, F64, "reference"), N,
                                   _dev(out, F64, "out"), _stream()))
    return out


# ---- readouts -------------------------------------------------------------------------------------
def readout_forward(h1, h2, w1, W2a, w2b, act_cst: float, scale: float, shift: float, want_feats: bool = True,
                    feats_rows=None):
    """(node_energies fp64 [N], d_h2 fp32 [N, C], node_feats fp64 [N, 2C] or None); feats_rows int32 [N] (a permutation)
    sends the features of node n to row feats_rows[n]."""
    N, C = h1.shape
    H = W2a.shape[1]
    dev = h1.device
    es = torch.empty(N, dtype=F64, device=dev)
    d2 = torch.empty(N, C, dtype=F32, device=dev)
    feats = torch.empty(N, 2 * C, dtype=F64, device=dev) if want_feats else None
    _check(
        lib.cm_readout_forward(
            _dev(h1, F32, "h1"), _dev(h2, F32, "h2"), _dev(w1, F64, "w1"), _dev(W2a, F64, "W2a"), _dev(w2b, F64, "w2b"),
            float(act_cst), float(scale), float(shift), N, C, H, _dev(es, F64, "node_energies"), _dev(d2, F32, "d_h2"),
            _dev(feats, F64, "node_feats"), _dev(feats_rows, I32, "feats_rows") if want_feats else None, _stream(),
        )
    )
    return es, d2, feats


def readout_backward(g, w1, d2, scale: float, need_h1: bool = True, need_h2: bool = True):
    N, C = d2.shape
    g1 = torch.empty_like(d2) if need_h1 else None
    g2 = torch.empty_like(d2) if need_h2 else None
    _check(
        lib.cm_readout_backward(
            _dev(g, F64, "grad_node_energies"), _dev(w1, F64, "w1"), _dev(d2, F32, "d_h2"), float(scale), N, C,
            _dev(g1, F32, "grad_h1"), _dev(g2, F32, "grad_h2"), _stream(),
        )
    )
    return g1, g2
