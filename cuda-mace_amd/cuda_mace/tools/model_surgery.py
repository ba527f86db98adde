"""Turn an invariant MACE model into an OptimizedInvariantMACE and save it.

    python -m cuda_mace.tools.model_surgery --model upstream.model --output optimized_model.model [--benchmark] [--accuracy]

Same job and options as the reference's tools/model_surgery.py (:19-63 parser, :254-275 main): load the pickled model,
wrap it, optionally time it and compare it with the original on a perturbed diamond supercell of `--size`^3 cubic cells,
and save the optimised model with torch.save.  Differences: the test structure and its neighbour list are built here
(device neighbour list; no ase / upstream data loader needed), and `--synthetic CHANNELS` makes a random-init model with
the upstream attribute tree when no upstream checkpoint is at hand.  Loading an upstream checkpoint needs the upstream
package importable, because the file is a pickle of its classes; `--accuracy` additionally needs that model to be callable.
"""
from __future__ import annotations

import argparse
from copy import deepcopy
from time import time

import numpy as np
import torch


def build_parser() -> argparse.ArgumentParser:
    parser = argparse.ArgumentParser(description="Optimize an invariant MACE model for MI355X inference.")
    parser.add_argument("--model", type=str, default=None, help="Path to the MACE model (a torch.save'd module).")
    parser.add_argument("--synthetic", type=int, default=0, metavar="CHANNELS",
                        help="Use a random-init model with this many channels instead of --model.")
    parser.add_argument("--output", type=str, default="optimized_model.model", help="Path to the output file.")
    parser.add_argument("--benchmark", action="store_true", default=False, help="Benchmark the optimized model.")
    parser.add_argument("--accuracy", action="store_true", default=False,
                        help="Compare energies and forces with the original model in fp64.")
    parser.add_argument("--size", type=int, default=3, help="Diamond supercell: size^3 cubic cells of 8 atoms.")
    parser.add_argument("--compare", type=int, default=0, help="Also time the original model.")
    return parser


def diamond_supercell(size: int, a: float = 3.567, noise: float = 0.05, seed: int = 0):
    """(positions [8 size^3, 3], cell [3, 3]) of cubic diamond carbon, atoms displaced by `noise` A (normal)."""
    basis = np.array([[0, 0, 0], [0, .5, .5], [.5, 0, .5], [.5, .5, 0], [.25, .25, .25], [.25, .75, .75], [.75, .25, .75],
                      [.75, .75, .25]])
    cells = np.stack(np.meshgrid(*[np.arange(size)] * 3, indexing="ij"), axis=-1).reshape(-1, 1, 3)
    pos = ((cells + basis[None]) * a).reshape(-1, 3)
    pos = pos + noise * np.random.default_rng(seed).standard_normal(pos.shape)
    return pos, np.eye(3) * a * size


def test_batch(model, size: int, device="cuda"):
    """`data` dictionary of the diamond test structure for this model's element table and cutoff."""
    from cuda_mace.utils.neighbour_list import neighbour_data

    pos, cell = diamond_supercell(size)
    numbers = [int(z) for z in model.atomic_numbers]
    column = numbers.index(6) if 6 in numbers else 0
    attrs = torch.zeros(pos.shape[0], len(numbers), dtype=torch.float64, device=device)
    attrs[:, column] = 1.0
    return neighbour_data(torch.tensor(pos, dtype=torch.float64, device=device), attrs, float(model.r_max), (True, True, True),
                          torch.tensor(cell, dtype=torch.float64, device=device))


def accuracy(model, model_opt, size: int = 4) -> None:
    batch = test_batch(model_opt, size)
    print("Number of atoms", batch["positions"].shape[0], "num edges", tuple(batch["edge_index"].shape))
    out_opt = model_opt(dict(batch), training=False, compute_force=True)
    try:
        out_org = model.double()(dict(batch), training=False, compute_force=True)
    except (NotImplementedError, TypeError) as err:  # a weight container without a forward of its own
        print("the original model cannot be evaluated here (%s); energy opt %s" % (err, out_opt["energy"]))
        return
    print("energy org", out_org["energy"], "\nenergy opt", out_opt["energy"])
    for key in ("energy", "forces"):
        err = (out_org[key] - out_opt[key]).abs()
        print("---F64:F32_Opt absolute %s error (mean, max)---\n%.5g %.5g" % (key, err.mean().item(), err.max().item()))


def benchmark(model, model_opt, size: int = 4, compare: bool = False, warmup: int = 50, niter: int = 100) -> float:
    batch = test_batch(model_opt, size)
    print("num nodes", batch["positions"].shape[0], "num edges", tuple(batch["edge_index"].shape))
    if compare:
        for _ in range(warmup):
            model(dict(batch), training=False, compute_force=True)
        torch.cuda.synchronize()
        start = time()
        for _ in range(niter):
            model(dict(batch), training=False, compute_force=True)
        torch.cuda.synchronize()
        print("original model time: %.2e (ms)" % ((time() - start) * (1000 / niter)))
    for _ in range(warmup):
        model_opt(dict(batch), training=False, compute_force=True)
    torch.cuda.synchronize()
    start = time()
    for _ in range(niter):
        model_opt(dict(batch), training=False, compute_force=True)
    torch.cuda.synchronize()
    ms = (time() - start) * (1000 / niter)
    print("optimized model time:  %.2e (ms)" % ms)
    return ms


def main(argv=None) -> None:
    from cuda_mace.models import OptimizedInvariantMACE, SyntheticInvariantMACE

    args = build_parser().parse_args(argv)
    if args.synthetic:
        model = SyntheticInvariantMACE(channels=args.synthetic, atomic_numbers=(1, 6, 7, 8), avg_num_neighbors=30.0)
    elif args.model:
        model = torch.load(args.model, weights_only=False)
    else:
        raise SystemExit("give --model PATH or --synthetic CHANNELS")
    model = model.to(torch.float64)
    opt_model = OptimizedInvariantMACE(deepcopy(model))
    print("--Optimized model")
    print(opt_model)
    if args.accuracy:
        print("--Analyzing errors")
        accuracy(model, opt_model, args.size)
    if args.benchmark:
        print("--Benchmarking")
        benchmark(model, opt_model, args.size, bool(args.compare))
    print(f"--Saving optimized model to: {args.output}")
    torch.save(opt_model, args.output)


if __name__ == "__main__":
    main()
