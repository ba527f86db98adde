#!/usr/bin/env python3
"""Headline benchmark: energy + forces steps of OptimizedInvariantMACE on a synthetic periodic box.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--atoms 25000] [--channels 128] [--no-cpu-baseline]

One "step" = one full forward (energy) + backward (forces) pass over one 25 000-atom, 128-channel,
10-element box at 0.1 atoms/A^3 (about 52 neighbours per atom within 5 A); positions, neighbour list and
weights are resident in HBM before the timed region.  Prints ONE JSON line with atoms*steps/s, the roofline
figures of the dominant kernel (measured live with events around its launches during the timed steps) and
the CPU baseline (the fp64-verified PyTorch restatement of the upstream model, timed on the host cores on a
bounded sample of the same workload).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "cuda-mace_amd"))

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published

TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic_25k_atoms_128ch.json")
KERNEL_SOURCES = os.path.join(ROOT, "cuda-mace_amd", "csrc")


# stages of cm_mace_step (include/cuda_mace_hip.h), in the order they run
STAGE_NAMES = {
    0: "00 edge geometry + live ranges", 1: "01 mp forward L0", 2: "02 channel mixing L0 [N,16,C]", 3: "03 contraction L0",
    4: "04 product linear L0 (+ skip, linear_up when chained)", 5: "05 skip connection", 6: "06 linear_up",
    7: "07 mp forward L1", 8: "08 channel mixing L1 [N,16,C]", 9: "09 contraction L1", 10: "10 product linear L1 + skip",
    11: "11 readouts", 12: "12 energy sums", 13: "13 backward seeds", 14: "14 product linear L1 backward",
    15: "15 channel mixing L1 backward (+ contraction backward)", 16: "16 mp backward L1 (edge pass + sender pass)",
    17: "17 linear_up backward (+ skip, product linear L0 backward, energy sums when chained)", 18: "18 skip backward",
    19: "19 product linear L0 backward", 20: "20 channel mixing L0 backward (+ contraction backward)",
    21: "21 mp backward L0 (edge pass, onto L1's vector gradient)", 22: "22 sum of vector gradients",
    23: "23 edge geometry backward (forces)", 24: "24 virials",
}


def kernel_sources_digest():
    """sha256 over the kernel sources (names and contents, sorted): ties a counter measurement to the code it was made on."""
    import hashlib

    h = hashlib.sha256()
    for name in sorted(os.listdir(KERNEL_SOURCES)):
        if name.endswith((".hip", ".hpp")):
            h.update(name.encode())
            with open(os.path.join(KERNEL_SOURCES, name), "rb") as f:
                h.update(f.read())
    return h.hexdigest()


def measured_traffic():
    """HBM bytes per launch at the default workload from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs (calibrated against a
    copy of known size), as recorded with the profile summaries together with the digest of the kernel sources they were
    measured on: {"in_step": {kernel: bytes}, "standalone": {kernel: bytes}} (inside the model step, where atoms are
    relabelled by spatial bin, and for the stand-alone ops on the box's random atom order).  Both are empty when the
    sources have changed since: a stale figure is not reported."""
    empty = {"in_step": {}, "standalone": {}}
    try:
        with open(TRAFFIC_FILE) as f:
            rec = json.load(f)
    except (OSError, ValueError):
        return empty
    if rec.get("kernel_sources_sha256") != kernel_sources_digest():
        return empty
    return {k: {n: int(v) for n, v in rec.get(k, {}).items()} for k in empty}


def traffic_of(table, kernels):
    """Sum over the kernels of an op ("a + b" names two); None when one of them was not measured."""
    parts = [table.get(k.strip()) for k in kernels.split("+")]
    return None if any(p is None for p in parts) else sum(parts)


def forward_kernel_name(C, N):
    """Kernel that runs the fused forward from edge vectors at this shape (csrc/mp_spline.hip: cm_mp_edge_forward; the
    benchmark's spline table has 256 knots)."""
    if 2048 <= N < 2**24 and C % 16 == 0 and N * C < 2**30:
        return "mp_edge_forward_sliced_kernel"
    return "mp_spline_forward_kernel<%d,true>" % C


def linear_kernel_name(C, N):
    """The library runs the [N,16,C] channel-mixing linear on its kernel with LDS-resident weights for 64, 96 and 128
    columns when there are at least 2 048 nodes, else on the LDS-ring kernel for 64, 96, 128, 224 and 256 columns and on
    the plain one otherwise."""
    nt = C // 32
    if nt in (2, 3, 4) and N >= 2048:
        return "linear_resident_kernel<%d,%d,false>" % (C, nt)
    return ("linear_ring_kernel<%d,false>" if nt in (2, 3, 4, 7, 8) else "linear_kernel<%d,false>") % nt


def mp_algorithmic_bytes(N, E, C):
    """Each operand touched once.  Tabulated radial weights R[E,4,C] (the reference's op): forward reads X, Y, R,
    sender, CSR and writes out; the backward edge pass without gX (first layer) reads X, Y, R, grad_out, sender, CSR and
    writes gY, gR.  Fused kernels: Y, R, gY, gR are replaced by the edge vectors / their gradient and the spline table."""
    fwd = 4 * (4 * E * C + 16 * E + 17 * N * C) + 4 * E + 8 * N
    bwd_edge = 4 * (8 * E * C + 32 * E + 17 * N * C) + 4 * E + 8 * N
    table = 255 * 16 * C * 4
    # fully fused kernels: edge vectors in (3E), out / grad_out (16NC), X (NC); the backward also writes the [E,3] gradient
    fwd_fused = 4 * (3 * E + 17 * N * C) + 4 * E + 8 * N + table
    bwd_fused = 4 * (6 * E + 17 * N * C) + 4 * E + 8 * N + table
    return fwd, bwd_edge, fwd_fused, bwd_fused


def _time_ms(torch, fn, reps):
    """Average duration of `fn` over `reps` back-to-back calls, by events on the stream the kernels are launched on
    (torch's current stream, which is what the ctypes binding hands to the library)."""
    fn()
    torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(reps):
        fn()
    e.record()
    torch.cuda.synchronize()
    return s.elapsed_time(e) / reps


def op_cases(torch, cabi, N, E, C, ne, rcv, snd, with_fused=True, with_node_ops=True, with_per_component=False):
    """(label, kernels, algorithmic bytes, callable) for every stand-alone op of the path on random operands of the given
    shape.  Bytes count each operand once.  `rcv` (sorted) and `snd` are int32 device tensors."""
    import numpy as np

    g = torch.Generator(device="cuda").manual_seed(0)
    X = torch.randn(N, C, device="cuda", generator=g)
    Y = torch.randn(16, E, device="cuda", generator=g)
    R = torch.randn(E, 4, C, device="cuda", generator=g)
    G = torch.randn(N, 16, C, device="cuda", generator=g)
    vec = torch.randn(E, 3, device="cuda", generator=g)
    vec = vec / vec.norm(dim=1, keepdim=True) * (torch.rand(E, 1, device="cuda", generator=g) * 4.0 + 0.9)
    r = vec.norm(dim=1).contiguous()
    kn, h = np.linspace(1e-12, 6.0, 256, retstep=True)
    knots = torch.tensor(kn, dtype=torch.float32, device="cuda")
    coeffs = torch.randn(255, 4, 4 * C, device="cuda", generator=g)
    fo = cabi.first_occurences(rcv, N)
    perm, off = cabi.stable_key_sort(snd, N)
    fwd_b, bwd_b, fwd_fb, bwd_fb = mp_algorithmic_bytes(N, E, C)
    bwd_full_b = 4 * (8 * E * C + 32 * E + 18 * N * C) + 8 * E
    cases = [
        ("mp_forward (tabulated R)", "mp_forward_kernel<%d>" % C, fwd_b, lambda: cabi.mp_forward(X, Y, R, snd, fo, N)),
        ("mp_backward gY,gR (tabulated R)", "mp_backward_edge_kernel<%d,true,true,false>" % C, bwd_b,
         lambda: cabi.mp_backward(X, Y, R, G, snd, fo, None, None, N, need_gX=False)),
        ("mp_backward gX,gY,gR (tabulated R): edge pass + sender pass",
         "mp_backward_edge_kernel<%d,true,true,true> + mp_backward_sender_kernel<%d,0,false>" % (C, C), bwd_full_b,
         lambda: cabi.mp_backward(X, Y, R, G, snd, fo, perm, off, N)),
    ]
    if with_per_component:
        # the same op with a radial weight per component, R [E,16,C]: four times the radial bytes
        R16 = torch.randn(E, 16, C, device="cuda", generator=g)
        cases += [
            ("mp_forward (R per component [E,16,C])", "mp_per_m_forward_kernel<%d>" % C,
             4 * (16 * E * C + 16 * E + 17 * N * C) + 8 * E, lambda: cabi.mp_forward(X, Y, R16, snd, fo, N)),
            ("mp_backward gX,gY,gR (R per component): edge pass + sender pass",
             "mp_per_m_backward_edge_kernel<%d,true,true,true> + mp_backward_sender_kernel<%d,0,false>" % (C, C),
             4 * (32 * E * C + 32 * E + 18 * N * C) + 8 * E, lambda: cabi.mp_backward(X, Y, R16, G, snd, fo, perm, off, N)),
        ]
    if with_fused:
        cases += [
            ("mp_edge_forward (fused harmonics + spline)", forward_kernel_name(C, N), fwd_fb,
             lambda: cabi.mp_edge_forward(X, vec, knots, coeffs, float(h), 5.0, snd, fo, N)),
            ("mp_edge_backward grad_vectors (fused)", "mp_spline_backward_edge_kernel<%d,true,true,true,false>" % C, bwd_fb,
             lambda: cabi.mp_edge_backward(X, vec, knots, coeffs, float(h), 5.0, G, snd, fo, None, None, N, need_gX=False)),
        ]
    if with_node_ops:
        from cuda_mace.models.upstream_like import _SymmetricContraction
        from cuda_mace.ops._autograd import monomials_from_packed
        from cuda_mace.ops.symmetric_contraction import SymmetricContraction

        WT = torch.randn(4, C, C, device="cuda", generator=g)
        gY = torch.randn(16, E, device="cuda", generator=g)
        gN = torch.randn(N, C, device="cuda", generator=g)
        mod = SymmetricContraction(_SymmetricContraction(C, ne, torch.Generator().manual_seed(0)), device="cuda")
        (m3, o3, p3, v3), (m2, o2, p2, v2) = monomials_from_packed(mod.U3_num_nonsparse, mod.U3_indices, mod.U3_values,
                                                                   mod.U2_num_nonsparse, mod.U2_indices, mod.U2_values)
        t = lambda a: torch.from_numpy(a).cuda()
        T3, T2, T1 = cabi.symcon_tables(t(o3), t(p3), t(v3), t(o2), t(p2), t(v2), mod.weights_3[0], mod.weights_2[0],
                                        mod.weights_1[0])
        types = torch.randint(0, ne, (N,), device="cuda", generator=g).int()
        eperm, eoff = cabi.stable_key_sort(types, ne)
        m3d, m2d = t(m3), t(m2)
        cases += [
            ("spherical harmonics forward", "sh_forward_kernel<float>", 76 * E, lambda: cabi.sh_forward(vec)),
            ("spherical harmonics backward", "sh_backward_kernel<float>", 88 * E, lambda: cabi.sh_backward(vec, gY)),
            ("spline forward (R only)", "spline_forward_sliced_kernel" if E >= 1 << 15 else "spline_forward_kernel<false>",
             4 * (E + 4 * E * C),
             lambda: cabi.spline_forward(r, knots, coeffs, float(h), 5.0)),
            ("spline backward", "spline_backward_sliced_kernel" if E >= 1 << 15 else "spline_backward_kernel",
             4 * (4 * E * C + 2 * E),
             lambda: cabi.spline_backward(r, knots, coeffs, R.view(E, 4 * C), float(h), 5.0)),
            ("symmetric contraction forward + gradient", "symcon_lmax3_kernel<float,true>", 4 * (33 * N * C + N),
             lambda: cabi.symcon_forward(G, eperm, eoff, m3d, m2d, T3, T2, T1, builtin=True, zero_init=False)),  # kernel alone:
            # every node is in a group, as in the model, which does not clear the outputs either
            ("symmetric contraction backward", "symcon_backward_kernel", 4 * 33 * N * C, lambda: cabi.symcon_backward(G, gN)),
            # channel-mixing linear [N,16,C] x [C,C] per l: reads X and the four weight blocks, writes OUT
            ("linear [N,16,C] x [C,C]", linear_kernel_name(C, N), 4 * (32 * N * C + 4 * C * C), lambda: cabi.linear(G, WT)),
        ]
    return cases


def box_edges(torch, make_system, N, ne):
    data = make_system(N, ne, seed=0, density=0.1)
    return data["edge_index"][0].int().cuda().contiguous(), data["edge_index"][1].int().cuda().contiguous()


def config2_edges(torch, N=4096, degree=30):
    """Benchmark configuration 2: every node receives `degree` edges, senders uniform random (torch.manual_seed(0))."""
    g = torch.Generator().manual_seed(0)
    rcv = torch.arange(N, dtype=torch.int32).repeat_interleave(degree)
    snd = torch.randint(0, N, (N * degree,), generator=g, dtype=torch.int32)
    return rcv.cuda(), snd.cuda()


def isolated_ops(args, torch, cabi, make_system, reps=3):
    """A reference copy (reads and writes `copy_bytes` each) followed by every stand-alone op of the path on random
    operands at the benchmark shape, and the message-passing op at the shape of configuration 2; prints one line per op
    with its average duration (for rocprofv3 --kernel-trace / --pmc runs)."""
    N, C = args.atoms, args.channels
    rcv, snd = box_edges(torch, make_system, N, args.elements)
    E = rcv.numel()
    copy_bytes = 1 << 30
    src = torch.empty(copy_bytes // 4, dtype=torch.float32, device="cuda").normal_()
    dst = torch.empty_like(src)
    cases = [("copy (reads %d B, writes %d B)" % (copy_bytes, copy_bytes), "copy", 2 * copy_bytes, lambda: dst.copy_(src))]
    cases += op_cases(torch, cabi, N, E, C, args.elements, rcv, snd)
    print("# isolated ops at N=%d E=%d C=%d" % (N, E, C), flush=True)
    for label, kernel, nbytes, fn in cases:
        ms = _time_ms(torch, fn, reps)
        print("%-62s %-70s %9.1f us  algorithmic %12d B  %8.1f GB/s" % (label, kernel, ms * 1e3, nbytes, nbytes / ms / 1e6), flush=True)
    rcv2, snd2 = config2_edges(torch)
    print("# configuration 2: N=4096 E=%d C=96" % rcv2.numel(), flush=True)
    for label, kernel, nbytes, fn in op_cases(torch, cabi, 4096, rcv2.numel(), 96, args.elements, rcv2, snd2, with_fused=False,
                                              with_node_ops=False, with_per_component=True):
        ms = _time_ms(torch, fn, 10 * reps)
        print("%-62s %-70s %9.1f us  algorithmic %12d B  %8.1f GB/s" % (label, kernel, ms * 1e3, nbytes, nbytes / ms / 1e6), flush=True)


def standalone_rooflines(torch, cabi, N, E, C, ne, rcv, snd, reps=10):
    """Roofline entries (HBM) of every stand-alone op at the benchmark shape and of the message-passing op at the shape of
    configuration 2, each timed on its own outside the timed steps."""
    def rows(cases, reps, **extra):
        out = []
        for label, kernel, nbytes, fn in cases:
            ms = _time_ms(torch, fn, reps)
            gbps = nbytes / (ms * 1e-3) / 1e9
            out.append(dict(op=label, kernel=kernel, bound="hbm", achieved=round(gbps, 1), peak=HBM_PEAK_GBPS, unit="GB/s",
                            frac=round(gbps / HBM_PEAK_GBPS, 4), algorithmic_bytes_per_launch=nbytes,
                            avg_launch_ms=round(ms, 4), **extra))
        return out

    at_c4 = rows(op_cases(torch, cabi, N, E, C, ne, rcv, snd, with_fused=False), reps, shape="N=%d E=%d C=%d" % (N, E, C))
    rcv2, snd2 = config2_edges(torch)
    at_c2 = rows(op_cases(torch, cabi, 4096, rcv2.numel(), 96, ne, rcv2, snd2, with_fused=False, with_node_ops=False,
                          with_per_component=True), 5 * reps,
                 shape="configuration 2: N=4096 E=%d C=96, uniform random senders" % rcv2.numel())
    fwd, full, fwd16, full16 = at_c2[0], at_c2[2], at_c2[3], at_c2[4]
    c2 = {"workload": "isolated invariant message passing forward + full backward (gX, gY, gR), 4096 nodes x 30 edges, 96 "
                      "channels, R[E,4,C] as the reference's op takes it",
          "fwd_ms": fwd["avg_launch_ms"], "bwd_ms": full["avg_launch_ms"],
          "fwd_plus_bwd_ms": round(fwd["avg_launch_ms"] + full["avg_launch_ms"], 4),
          "algorithmic_bytes": fwd["algorithmic_bytes_per_launch"] + full["algorithmic_bytes_per_launch"],
          "GB/s": round((fwd["algorithmic_bytes_per_launch"] + full["algorithmic_bytes_per_launch"])
                        / ((fwd["avg_launch_ms"] + full["avg_launch_ms"]) * 1e-3) / 1e9, 1)}
    c2["frac_of_hbm_peak"] = round(c2["GB/s"] / HBM_PEAK_GBPS, 4)
    b16 = fwd16["algorithmic_bytes_per_launch"] + full16["algorithmic_bytes_per_launch"]
    t16 = fwd16["avg_launch_ms"] + full16["avg_launch_ms"]
    c2["per_component_weights"] = {
        "workload": "the same with radial weights per component, R[E,16,C] (the shape the configuration is worded with)",
        "fwd_ms": fwd16["avg_launch_ms"], "bwd_ms": full16["avg_launch_ms"], "algorithmic_bytes": b16,
        "GB/s": round(b16 / (t16 * 1e-3) / 1e9, 1), "frac_of_hbm_peak": round(b16 / (t16 * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)}
    return at_c4 + at_c2, c2


def other_configs(torch, make_system, to_device, OptimizedInvariantMACE, SyntheticInvariantMACE):
    """Energy+forces steps of the other benchmark configurations (1: 21-atom cluster, eager and as one HIP graph;
    3: 5 000 atoms, 96 channels; 5: 100 000 atoms, 192 channels), each timed like the headline."""
    from cuda_mace.utils.graph import GraphedStep

    def run(label, data_cpu, C, numbers, warmup, steps, graph=False):
        N, E = int(data_cpu["positions"].shape[0]), int(data_cpu["edge_index"].shape[1])
        up = SyntheticInvariantMACE(channels=C, atomic_numbers=numbers, avg_num_neighbors=E / N, seed=0)
        model = OptimizedInvariantMACE(up, device="cuda")
        data = to_device(data_cpu, "cuda")

        def timed(fn):
            for _ in range(warmup):
                fn()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                fn()
            torch.cuda.synchronize()
            return 1e3 * (time.perf_counter() - t0) / steps

        ms = timed(lambda: model(dict(data)))
        out = {"workload": label, "atoms": N, "edges": E, "channels": C, "ms_per_step": round(ms, 4),
               "atoms_steps_per_s": round(N / ms * 1e3, 1), "steps": steps}
        if graph:
            step = GraphedStep(model, data)
            ms_g = timed(lambda: step(data["positions"]))
            out.update(ms_per_step_hip_graph=round(ms_g, 4), atoms_steps_per_s_hip_graph=round(N / ms_g * 1e3, 1))
        del model, data
        torch.cuda.empty_cache()
        return out

    res = {}
    res["c1"] = run("21-atom cluster in an 8 A cube, {H,C,N,O}, 64x0e (fp32 kernels; the fp64 CPU reference is the parity "
                    "oracle of this configuration)", make_system(21, 4, seed=0, density=None, cluster_box=8.0), 64,
                    (1, 6, 7, 8), 20, 200, graph=True)
    # how configuration 1 is served when throughput matters: many such structures in one batch, one library call
    from cuda_mace.utils.synthetic import collate

    nbatch = 512
    many = run("%d clusters of configuration 1 in one batch (different seeds), one step for all of them" % nbatch,
               collate([make_system(21, 4, seed=s, density=None, cluster_box=8.0) for s in range(nbatch)]), 64, (1, 6, 7, 8), 10, 50)
    many["structures"] = nbatch
    many["us_per_structure"] = round(1e3 * many["ms_per_step"] / nbatch, 3)
    res["c1"]["batched"] = many
    # the reference's own benchmark workload (tools/model_surgery.py:145-233: a cubic diamond supercell of size^3 cells with
    # 0.05 A of noise, default size 3 = 216 atoms), here with a 128-channel model
    from cuda_mace.tools.model_surgery import test_batch

    class _Table:
        atomic_numbers, r_max = (1, 6, 7, 8), 5.0

    for size in (3, 4):
        batch = {k: (v.cpu() if hasattr(v, "cpu") else v) for k, v in test_batch(_Table, size).items()}
        res["diamond_%d" % (8 * size ** 3)] = run(
            "the reference's benchmark structure: diamond supercell --size %d (%d atoms, noise 0.05 A), 128x0e" % (size, 8 * size ** 3),
            batch, 128, (1, 6, 7, 8), 50, 100, graph=True)
    res["c3"] = run("5 000-atom periodic box, 96x0e, 10 elements", make_system(5000, 10, seed=0, density=0.1), 96,
                    tuple(range(1, 11)), 10, 50)
    res["c5"] = run("100 000-atom periodic box, 192x0e, 10 elements", make_system(100000, 10, seed=0, density=0.1), 192,
                    tuple(range(1, 11)), 3, 10)
    # sixteen times the headline size on the one GPU (29 GB of its 288): the list from the device neighbour search
    from cuda_mace.utils.synthetic import make_large_system

    big = make_large_system(400000, 10, seed=0, density=0.1)
    res["c4_x16"] = run("400 000-atom periodic box (jittered lattice, 0.1 atoms/A^3), 128x0e, 10 elements",
                        {k: v for k, v in big.items()}, 128, tuple(range(1, 11)), 2, 5)
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--atoms", type=int, default=25000)
    ap.add_argument("--channels", type=int, default=128)
    ap.add_argument("--elements", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-md-loop", action="store_true",
                    help="skip the MD-like loop through the device calculator (keeps a kernel trace of this run to the "
                         "timed steps and the isolated ops)")
    ap.add_argument("--tabulated-radial", action="store_true",
                    help="keep the reference's separate spline step (R[E,4,C] in HBM) instead of the fused kernels")
    ap.add_argument("--cpu-atoms", type=int, default=1500, help="size of the box the CPU baseline is timed on")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip what is measured besides the timed steps: stand-alone op rooflines, the other configurations, "
                         "neighbour list, MD loop (keeps a profiler's trace of this run to the timed steps)")
    ap.add_argument("--isolated-ops", action="store_true",
                    help="instead of the model step, launch a plain copy of known size and each message-passing kernel a few "
                         "times at the benchmark shape (for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs)")
    args = ap.parse_args()

    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU; the hot path has no multi-GPU part (it would shard by receiver node range "
              "with one halo exchange per layer). "
              "Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(1)

    from cuda_mace import _cabi as cabi
    from cuda_mace.models import OptimizedInvariantMACE, SyntheticInvariantMACE
    from cuda_mace.utils.synthetic import make_system, to_device

    N, C, ne = args.atoms, args.channels, args.elements
    if args.isolated_ops:
        isolated_ops(args, torch, cabi, make_system)
        return
    t0 = time.time()
    data_cpu = make_system(N, ne, seed=0, density=0.1)
    E = int(data_cpu["edge_index"].shape[1])
    upstream = SyntheticInvariantMACE(channels=C, atomic_numbers=tuple(range(1, ne + 1)), avg_num_neighbors=E / N, seed=0)
    fused = not args.tabulated_radial
    model = OptimizedInvariantMACE(upstream, device="cuda", fused_radial=fused)
    data = to_device(data_cpu, "cuda")
    print("# setup %.1fs: N=%d E=%d C=%d" % (time.time() - t0, N, E, C), file=sys.stderr, flush=True)

    def step():
        out = model(dict(data))
        return out["energy"], out["forces"]

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    # Live timing of the dominant kernels inside the timed steps, by events on the launch stream.  The default model hands
    # the step to the library in one call, which brackets the chosen stages itself (message passing forward of both
    # layers, the backward edge pass of the first layer, which runs without the sender pass, and the two [N,16,C]
    # channel-mixing launches); with --tabulated-radial the step goes through the Python wrappers, which are bracketed here.
    import ctypes

    fwd_name, bwd_name = ("mp_edge_forward", "mp_edge_backward") if fused else ("mp_forward", "mp_backward")
    events = {fwd_name: [], bwd_name: [], "linear": []}
    originals = {}
    native = fused and model._native_step_of() is not None
    STAGES = {fwd_name: (1, 7), bwd_name: (21,), "linear": (2, 8)}
    if native:
        cabi._check(cabi.lib.cm_mace_step_timing(sum(1 << s for ids in STAGES.values() for s in ids)))
    else:
        originals = {fwd_name: getattr(cabi, fwd_name), bwd_name: getattr(cabi, bwd_name), "linear": cabi.linear}

        def timed(name, fn, pred):
            def wrapper(*a, **k):
                if not pred(a, k):
                    return fn(*a, **k)
                s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                s.record()
                r = fn(*a, **k)
                e.record()
                events[name].append((s, e))
                return r
            return wrapper

        setattr(cabi, bwd_name, timed(bwd_name, originals[bwd_name], lambda a, k: not k.get("need_gX", True)))
        setattr(cabi, fwd_name, timed(fwd_name, originals[fwd_name], lambda a, k: True))
        # the 16-component channel-mixing launches (forward ones: no row_scale)
        cabi.linear = timed("linear", originals["linear"], lambda a, k: a[0].dim() == 3 and k.get("row_scale") is None)

    torch.cuda.synchronize()
    t_start = time.perf_counter()
    for _ in range(args.steps):
        energy, forces = step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t_start
    for name, fn in originals.items():
        setattr(cabi, name, fn)
    stage_ms, stage_n = (ctypes.c_double * 32)(), (ctypes.c_int64 * 32)()
    if native:
        cabi._check(min(cabi.lib.cm_mace_step_timing_read(ctypes.addressof(stage_ms), ctypes.addressof(stage_n), 32), 0))
        cabi._check(cabi.lib.cm_mace_step_timing(0))

    # every stage of the step, bracketed by events in a few more steps outside the timed region (the brackets cost a
    # few microseconds of launch gaps per stage, so the sum sits slightly above ms_per_step)
    stages_us, stages_sum_ms, launches_per_step = None, None, None
    if native:
        all_ms, all_n = (ctypes.c_double * 32)(), (ctypes.c_int64 * 32)()
        cabi._check(cabi.lib.cm_mace_step_timing((1 << 25) - 1))
        nsteps_all = 10
        for _ in range(nsteps_all):
            step()
        torch.cuda.synchronize()
        cabi._check(min(cabi.lib.cm_mace_step_timing_read(ctypes.addressof(all_ms), ctypes.addressof(all_n), 32), 0))
        cabi._check(cabi.lib.cm_mace_step_timing(0))
        stages_us = {STAGE_NAMES[i]: round(1e3 * all_ms[i] / nsteps_all, 1) for i in range(25) if all_n[i]}
        stages_sum_ms = round(sum(all_ms[i] for i in range(25)) / nsteps_all, 4)

    ms_per_step = 1e3 * elapsed / args.steps
    value = N * args.steps / elapsed
    assert bool(torch.isfinite(energy).all()) and bool(torch.isfinite(forces).all())

    def launches(name):
        return int(sum(stage_n[i] for i in STAGES[name])) if native else len(events[name])

    def avg_ms(name):
        if native:
            n = launches(name)
            return sum(stage_ms[i] for i in STAGES[name]) / n if n else None
        ts = [s.elapsed_time(e) for s, e in events[name]]
        return sum(ts) / len(ts) if ts else None

    default_workload = (N, C, ne) == (25000, 128, 10)
    traffic = measured_traffic()

    def entry(kernel, nbytes, ms, **extra):
        gbps = nbytes / (ms * 1e-3) / 1e9
        d = {"kernel": kernel, "bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
             "frac": round(gbps / HBM_PEAK_GBPS, 4),
             "traffic": traffic_of(traffic["in_step"], kernel) if default_workload else None,
             "algorithmic_bytes_per_launch": nbytes, "avg_launch_ms": round(ms, 4)}
        d.update(extra)
        return d

    fwd_b, bwd_b, fwd_fb, bwd_fb = mp_algorithmic_bytes(N, E, C)
    t_bwd, t_fwd = avg_ms(bwd_name), avg_ms(fwd_name)
    if fused:
        sh_b, spline_b = 88 * E, 4 * (8 * E * C + E)  # harmonics backward, spline backward (each operand once)
        sh_f, spline_f = 76 * E, 4 * (E + 8 * E * C)  # harmonics forward, spline forward (each operand once)
        flops_fwd = 60 * E * C  # per edge and channel: the cubic of 4 degrees (12 FMA), 4 products, 16 accumulations
        roofline = entry(forward_kernel_name(C, N), fwd_fb, t_fwd, launches_timed=launches(fwd_name),
                         note="dominant kernel of the step by total time (two launches per step). Harmonics and radial "
                              "weights are evaluated in-kernel, so its own HBM operands are small; a workgroup keeps its "
                              "part of the spline table (two degrees x 16 channels, 130 KB) in LDS, so the coefficients "
                              "no longer travel through L1 (the kernel it replaces pulled 8 KB per edge from L2 and ran "
                              "at 0.37-0.46 ms): bounded by vector-instruction issue (counter summary: ~90% of the SIMDs' "
                              "four-cycle issue slots with two waves per SIMD, LDS half busy), not by HBM; see "
                              "roofline_other_kernels for the HBM-bound message passing with tabulated R[E,4,C] and for "
                              "the matrix-core linear",
                         binding_resource={
                             "resource": "fp32 vector arithmetic: per edge and channel the cubic of 4 degrees (12 FMA), 4 "
                                         "products and 16 accumulations",
                             "flops": flops_fwd, "achieved_TFLOP/s": round(flops_fwd / (t_fwd * 1e-3) / 1e12, 1),
                             "peak_TFLOP/s": 157.3, "frac": round(flops_fwd / (t_fwd * 1e-3) / 1e12 / 157.3, 4),
                             "frac_of_unpacked_rate": round(flops_fwd / (t_fwd * 1e-3) / 1e12 / 78.65, 4),
                             "meaning": "useful fp32 operations of the formulation against the vector peak (which counts "
                                        "two-wide packed fp32 instructions; this library is built without them, so one "
                                        "FMA per lane and four cycles, 78.65 TFLOP/s, is the rate its instructions can "
                                        "reach: frac_of_unpacked_rate); the kernel issues "
                                        "about 1.8 instructions per useful one (edge set-up per quad of lanes, broadcasts of "
                                        "the edge's values, addresses), and instructions with a cross-lane operand issue at "
                                        "less than half the rate of plain ones on this device"},
                         unfused_equivalent={
                             "bytes": fwd_b + sh_f + spline_f,
                             "GB/s": round((fwd_b + sh_f + spline_f) / (t_fwd * 1e-3) / 1e9, 1),
                             "meaning": "algorithmic HBM bytes of the three separate kernels this launch replaces (message "
                                        "passing with tabulated R, spline evaluation, harmonics) divided by this launch's "
                                        "duration"})
        others = [entry("mp_spline_backward_edge_kernel<%d,true,true,true,false>" % C, bwd_fb, t_bwd,
                        launches_timed=launches(bwd_name),
                        note="bounded by VALU issue (~80% of all issue slots), see the counter summary")]
        t_lin = avg_ms("linear")
        if t_lin:
            flops = 32 * N * C * C
            tf = flops / (t_lin * 1e-3) / 1e12
            lin_bytes = 4 * (32 * N * C + 4 * C * C)
            others.append(entry(linear_kernel_name(C, N), lin_bytes, t_lin, launches_timed=launches("linear"),
                                matrix_cores={"fp32_equivalent_TFLOP/s": round(tf, 1), "instruction_TFLOP/s_bf16": round(6 * tf, 1),
                                              "frac_of_bf16_peak": round(6 * tf / 2500.0, 4)},
                                note="[N,16,C] x [C,C] channel mixing: bound by its memory traffic, not by the matrix cores "
                                     "(every fp32 product is six bf16 piece products on v_mfma_f32_32x32x16_bf16, which "
                                     "keeps the pipes about a third busy)"))
            others[-1]["traffic"] = traffic_of(traffic["standalone"], linear_kernel_name(C, N)) if default_workload else None
    else:
        # The model drives the tabulated ops through the TorchScript classes, which the Python-side brackets above do not
        # see: the two message-passing kernels are then timed on their own, on the step's edge list with random operands.
        if t_bwd is None or t_fwd is None:
            alone = op_cases(torch, cabi, N, E, C, ne, data["edge_index"][0].int().contiguous(),
                             data["edge_index"][1].int().contiguous(), with_fused=False, with_node_ops=False)
            t_fwd, t_bwd = _time_ms(torch, alone[0][3], 5), _time_ms(torch, alone[1][3], 5)
        roofline = entry("mp_backward_edge_kernel<%d,true,true,false>" % C, bwd_b, t_bwd,
                         launches_timed=launches(bwd_name) or 5,
                         note="timed stand-alone on the step's edge list" if not launches(bwd_name) else "timed inside the step")
        others = [entry("mp_forward_kernel<%d>" % C, fwd_b, t_fwd)]

    # two control figures that tell boxes of the pool apart: a streaming kernel (message passing with tabulated R at the
    # step's shape, HBM-bound) and a loop of plain fp32 multiply-adds (VALU-bound)
    rcv32 = data["edge_index"][0].int().contiguous()
    snd32 = data["edge_index"][1].int().contiguous()
    probe_out = torch.zeros(1, device="cuda")
    wgs, iters = 256 * 8 * 4, 4096
    t_probe = _time_ms(torch, lambda: cabi._check(cabi.lib.cm_probe_fma(probe_out.data_ptr(), wgs, iters, cabi._stream())), 5)
    mp_case = op_cases(torch, cabi, N, E, C, ne, rcv32, snd32, with_fused=False, with_node_ops=False)[0]
    t_stream = _time_ms(torch, mp_case[3], 5)
    controls = {
        "valu_fp32_fma_TFLOP/s": round(2 * 8 * iters * 256 * wgs / (t_probe * 1e-3) / 1e12, 1),
        "valu_note": "plain v_fma_f32 loop, 8 independent chains per lane, 32 waves per compute unit, built without packed fp32 "
                     "instructions like the rest of the library",
        "hbm_stream_kernel": mp_case[1], "hbm_stream_GB/s": round(mp_case[2] / (t_stream * 1e-3) / 1e9, 1),
        "hbm_stream_ms": round(t_stream, 4),
    }
    del mp_case

    # every stand-alone op of the path (the reference's op list: message passing with tabulated R[E,4,C] incl. the full
    # backward, harmonics, spline, contraction, linear) at the same shape, and configuration 2, each timed on its own
    standalone, config2 = None, None
    if not args.no_extras:
        standalone, config2 = standalone_rooflines(torch, cabi, N, E, C, ne, rcv32, snd32)
        for row in standalone:
            row["traffic"] = traffic_of(traffic["standalone"], row["kernel"]) if default_workload else None
        others += standalone

    # the step before the path: neighbour list rebuilt on the device (excluded from the timed steps, as the reference's
    # own timing excludes it); checked against the host-built list of the generator
    from cuda_mace.utils.neighbour_list import get_neighborhood

    def build_list():
        return get_neighborhood(data["positions"].detach(), 5.0, (True, True, True), data["cell"])

    neighbour_list = None
    if not args.no_extras:
        ei_dev = build_list()[0]
        torch.cuda.synchronize()
        t_nl = time.perf_counter()
        for _ in range(5):
            build_list()
        torch.cuda.synchronize()
        neighbour_list = {"ms_per_build": round(1e3 * (time.perf_counter() - t_nl) / 5, 3), "pairs": int(ei_dev.shape[1]),
                          "identical_to_host_list": bool(torch.equal(ei_dev, data["edge_index"]))}

    # an MD-like loop through the device-side calculator: every atom moves 0.02 A per step in a random direction, the
    # Verlet list (cutoff + 0.5 A skin) is rebuilt on the device whenever an atom has moved more than half the skin
    from cuda_mace.calculators import DeviceCalculator

    calc = DeviceCalculator(model, data["node_attrs"], cutoff=5.0, skin=0.5, pbc=(True, True, True), cell=data["cell"])
    gen = torch.Generator(device="cuda").manual_seed(0)
    pos = data["positions"].detach().clone()
    md_steps = 0 if (args.no_md_loop or args.no_extras) else 60

    def md_step(p):
        d = torch.randn(p.shape, device="cuda", dtype=p.dtype, generator=gen)
        p = p + 0.02 * d / d.norm(dim=1, keepdim=True)
        calc.compute(p)
        return p

    for _ in range(5 if md_steps else 0):
        pos = md_step(pos)
    builds0 = calc.builds
    torch.cuda.synchronize()
    t_md = time.perf_counter()
    for _ in range(md_steps):
        pos = md_step(pos)
    torch.cuda.synchronize()
    t_md = time.perf_counter() - t_md
    t_move = None
    if md_steps:  # the loop's own position update (the stand-in for an integrator), timed alone
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(20):
            d = torch.randn(pos.shape, device="cuda", dtype=pos.dtype, generator=gen)
            _ = pos + 0.02 * d / d.norm(dim=1, keepdim=True)
        torch.cuda.synchronize()
        t_move = 1e3 * (time.perf_counter() - t0) / 20
    md_loop = None if not md_steps else {
               "ms_per_step": round(1e3 * t_md / md_steps, 4), "steps": md_steps,
               "of_which_position_update_ms": round(t_move, 4),
               "list_rebuilds": calc.builds - builds0, "steps_enqueued_twice": calc.dropped, "skin_A": 0.5, "move_per_step_A": 0.02,
               "hip_graph": calc.use_graph,
               "note": "energy+forces through DeviceCalculator incl. neighbour-list rebuilds on the device; the list holds "
                       "(1 + skin/cutoff)^3 = 1.33x the pairs of the exact list; the host reads the displacement test "
                       "after it has enqueued the step (a step on a list found stale is enqueued again)"}

    # the same step with virials and stress (formed from the per-edge gradients in the same library call)
    with_stress = None
    if not args.no_extras and fused:
        for _ in range(3):
            model(dict(data), compute_stress=True)
        torch.cuda.synchronize()
        t_s = time.perf_counter()
        for _ in range(20):
            out_s = model(dict(data), compute_stress=True)
        torch.cuda.synchronize()
        with_stress = {"ms_per_step": round(1e3 * (time.perf_counter() - t_s) / 20, 4), "steps": 20,
                       "stress_finite": bool(torch.isfinite(out_s["stress"]).all()),
                       "note": "energy + forces + virials + stress in one library call"}

    configs = None
    if not args.no_extras:
        del calc
        configs = other_configs(torch, make_system, to_device, OptimizedInvariantMACE, SyntheticInvariantMACE)
        configs["c2"] = config2

    cpu_baseline = None
    if not args.no_cpu_baseline:
        from oracle import mace_model as oracle_model  # the checker, timed as the reported CPU baseline

        n_cpu = min(args.cpu_atoms, N)
        sample = make_system(n_cpu, ne, seed=1, density=0.1)
        params = upstream.export_params()
        cores = torch.get_num_threads()
        oracle_model.energy_and_forces(params, sample, dtype=torch.float32)  # warm-up
        reps, t1 = 0, time.perf_counter()
        while reps < 2 or (time.perf_counter() - t1 < 10.0 and reps < 20):
            oracle_model.energy_and_forces(params, sample, dtype=torch.float32)
            reps += 1
        dt = (time.perf_counter() - t1) / reps
        cpu_baseline = {
            "value": round(n_cpu / dt, 1), "unit": "atoms*steps/s", "cores": cores, "kind": "port",
            "sample": "%d-atom periodic box of the same generator (density 0.1/A^3, %d elements, C=%d), fp32 PyTorch "
                      "restatement of the upstream model, %d energy+forces steps" % (n_cpu, ne, C, reps),
            "s_per_step": round(dt, 3),
        }

    line = {
        "metric": "atoms*steps/s (energy+forces) at 25k atoms, 128ch; msg-passing HBM GB/s",
        "value": round(value, 1), "unit": "atoms*steps/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "invariant MACE energy+forces, %d-atom periodic box at 0.1 atoms/A^3, %d edges, %dx0e, "
                               "l_max 3, correlation 3, %d elements, random-init weights (seed 0)" % (N, E, C, ne),
                   "atoms": N, "edges": E, "channels": C, "radial": "fused spline" if fused else "tabulated"},
        "roofline": roofline, "stages_us": stages_us, "stages_sum_ms": stages_sum_ms, "controls": controls,
        "roofline_other_kernels": others, "cpu_baseline": cpu_baseline,
        "neighbour_list": neighbour_list, "md_loop": md_loop, "with_stress": with_stress, "other_configs": configs,
    }
    if cpu_baseline:
        line["speedup_vs_cpu_baseline"] = round(value / cpu_baseline["value"], 1)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
