"""The op modules (`cuda_mace.ops.*`, i.e. the TorchScript classes over the C ABI) through torch.autograd, against the
fp64 oracle with gradients by autograd on the oracle's definitions."""
import math

import numpy as np
import pytest
import torch

from oracle import ops as O
from tests.util import close, mp_inputs, random_graph

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _leaf(t):
    return t.float().to(DEV).requires_grad_(True)


@pytest.mark.parametrize("need", [(True, True, True), (False, True, True), (True, False, False), (False, False, True)])
def test_message_passing_module_autograd(cabi, need):
    from cuda_mace.ops import InvariantMessagePassingTP

    nnodes, C = 150, 96
    snd, rcv = random_graph(nnodes, 25, 3, isolated_frac=0.1)
    E = snd.numel()
    X, v, R, G = mp_inputs(nnodes, E, C, 3)
    Y = O.spherical_harmonics(v).contiguous()
    Xa, Ya, Ra = (t.clone().requires_grad_(n) for t, n in zip((X, Y, R), need))
    (O.mp_forward(Xa, Ya, Ra, snd, rcv, nnodes) * G).sum().backward()
    xs = [t.float().to(DEV).requires_grad_(n) for t, n in zip((X, Y, R), need)]
    tp = InvariantMessagePassingTP()
    out = tp(xs[0], xs[1], xs[2], snd.to(DEV), rcv.to(DEV), nnodes)
    (out * G.float().to(DEV)).sum().backward()
    for got, want, n in zip(xs, (Xa, Ya, Ra), need):
        if n:
            close(got.grad, want.grad, 2e-5, 2e-6)
        else:
            assert got.grad is None


def test_message_passing_no_stale_index_cache(cabi):
    """Edge lists that are re-created every call (same size, possibly the same address) must never reuse derived
    index structures of an earlier list."""
    from cuda_mace.ops import InvariantMessagePassingTP

    tp = InvariantMessagePassingTP()
    nnodes, C = 64, 32
    for seed in range(4):
        snd, rcv = random_graph(nnodes, 10, 100 + seed, degree_mode="fixed")
        E = snd.numel()
        X, v, R, G = mp_inputs(nnodes, E, C, seed)
        Y = O.spherical_harmonics(v).contiguous()
        Xa = X.clone().requires_grad_(True)
        ref = O.mp_forward(Xa, Y, R, snd, rcv, nnodes)
        (ref * G).sum().backward()
        xg = _leaf(X)
        s_dev, r_dev = snd.long().to(DEV).int(), rcv.long().to(DEV).int()  # fresh int32 tensors every iteration
        out = tp(xg, Y.float().to(DEV), R.float().to(DEV), s_dev, r_dev, nnodes)
        (out * G.float().to(DEV)).sum().backward()
        close(out.detach(), ref.detach(), 2e-5, 2e-6)
        close(xg.grad, Xa.grad, 2e-5, 2e-6)
        del s_dev, r_dev


def test_spherical_harmonics_and_spline_modules(cabi):
    from cuda_mace.ops import CubicSpline
    from cuda_mace.ops.spherical_harmonics import SphericalHarmonics

    g = torch.Generator().manual_seed(0)
    xyz = torch.randn(500, 3, generator=g, dtype=torch.float64).float().double()
    gy = torch.randn(16, 500, generator=g, dtype=torch.float64)
    xa = xyz.clone().requires_grad_(True)
    (O.spherical_harmonics(xa) * gy).sum().backward()
    xg = _leaf(xyz)
    Y = SphericalHarmonics()(xg)
    (Y * gy.float().to(DEV)).sum().backward()
    close(Y.detach(), O.spherical_harmonics(xyz), 1e-5, 2e-6)
    close(xg.grad, xa.grad, 2e-5, 2e-6)

    knots_np, h = np.linspace(1e-12, 6.0, 256, retstep=True)
    knots = torch.from_numpy(knots_np)
    table = torch.cos(knots[:, None] * torch.linspace(0.2, 2.0, 256, dtype=torch.float64)[None, :])
    spline = CubicSpline(knots.float(), table.float(), float(h), 5.0).to(DEV)
    # (the coefficient solve itself is checked against scipy in fp64 on the CPU; here the module's own table is used)
    r =(torch.rand(300, generator=g, dtype=torch.float64) * 5.5 + 0.3).float().double()
    gR = torch.randn(300, 256, generator=g, dtype=torch.float64)
    ra = r.clone().requires_grad_(True)
    co = spline.coefficients.double().cpu()
    (O.spline_eval(ra, spline.r_knots.double().cpu(), co, float(np.float32(h)), 5.0) * gR).sum().backward()
    rg = _leaf(r)
    out = spline(rg)
    (out * gR.float().to(DEV)).sum().backward()
    close(out.detach(), O.spline_eval(r, spline.r_knots.double().cpu(), co, float(np.float32(h)), 5.0), 2e-5, 2e-6)
    bound = 4e-6 * (gR.abs() * O.spline_eval(r, spline.r_knots.double().cpu(), co, float(np.float32(h)), 5.0, deriv=True)[1].abs()).sum(-1) + 1e-30
    assert bool(((rg.grad.double().cpu() - ra.grad).abs() <= bound).all())


def test_linear_modules_autograd(cabi):
    from cuda_mace.models.InvariantMACE import element_linear_to_cuda
    from cuda_mace.models.upstream_like import _LinearPerL, _SkipTP
    from cuda_mace.ops import Linear

    g = torch.Generator().manual_seed(1)
    C, ne, N = 64, 5, 300
    lin = _LinearPerL(C, g)
    mod = Linear(lin).to(DEV)
    X = torch.randn(N, 16, C, generator=g, dtype=torch.float64)
    G = torch.randn(N, 16, C, generator=g, dtype=torch.float64)
    W = mod.weights.double().cpu()
    Xa = X.clone().requires_grad_(True)
    (O.linear(Xa, W) * G).sum().backward()
    xg = _leaf(X)
    out = mod(xg)
    (out * G.float().to(DEV)).sum().backward()
    close(out.detach(), O.linear(X, W), 1e-5, 2e-6)
    close(xg.grad, Xa.grad, 1e-5, 2e-6)

    el = element_linear_to_cuda(_SkipTP(C, ne, 3, g)).to(DEV)
    elem = torch.randint(0, ne + 1, (N,), generator=g)  # value ne: a row that names no element
    one_hot = torch.nn.functional.one_hot(elem, ne + 1)[:, :ne].double()
    We = el.weights.double().cpu()
    Xa = X.clone().requires_grad_(True)
    (O.elemental_linear(Xa, We, one_hot) * G).sum().backward()
    xg = _leaf(X)
    out = el(xg, one_hot.float().to(DEV))
    (out * G.float().to(DEV)).sum().backward()
    close(out.detach(), O.elemental_linear(X, We, one_hot), 1e-5, 2e-6)
    close(xg.grad, Xa.grad, 1e-5, 2e-6)
    assert float(out[(elem == ne).to(DEV)].abs().sum()) == 0.0


def test_model_pickle_round_trip(cabi, tmp_path):
    """torch.save / torch.load of the whole optimised model (the reference saves it that way,
    tools/model_surgery.py:258-261): the custom-class objects pickle with empty state."""
    from cuda_mace.models import OptimizedInvariantMACE, SyntheticInvariantMACE
    from cuda_mace.utils.synthetic import make_system, to_device

    data = make_system(30, 4, seed=2, density=None, cluster_box=8.0)
    avg = data["edge_index"].shape[1] / 30
    model = OptimizedInvariantMACE(SyntheticInvariantMACE(channels=32, avg_num_neighbors=avg, seed=2), device=DEV)
    out = model(to_device(data, DEV))
    path = tmp_path / "model.pt"
    torch.save(model, path)
    back = torch.load(path, weights_only=False)
    out2 = back(to_device(data, DEV))
    assert torch.equal(out["energy"], out2["energy"]) and torch.equal(out["forces"], out2["forces"])


def test_model_surgery_tool(cabi, tmp_path, capsys):
    """The conversion tool end to end on a random-init model: optimise, time on the diamond test structure, save, reload."""
    from cuda_mace.tools import model_surgery

    path = tmp_path / "optimized.model"
    model_surgery.main(["--synthetic", "32", "--size", "2", "--benchmark", "--accuracy", "--output", str(path)])
    printed = capsys.readouterr().out
    assert "optimized model time" in printed and "Saving optimized model" in printed
    back = torch.load(path, weights_only=False)
    batch = model_surgery.test_batch(back, 2)
    assert batch["positions"].shape[0] == 64 and batch["edge_index"].shape[1] > 64 * 30
    out = back(batch)
    assert bool(torch.isfinite(out["energy"]).all()) and out["forces"].shape == (64, 3)
    assert float(out["forces"].sum(0).abs().max()) < 1e-4 * max(1.0, float(out["forces"].abs().max()))


def test_model_surgery_tool_against_a_callable_source_model(cabi, tmp_path, capsys):
    """The tool's own accuracy check (the reference's tools/model_surgery.py:66-143 compares the optimised model with
    the original one in fp64) on a saved source model that can be evaluated: here its forward is the fp64 reference
    model.  The errors the tool prints must meet the parity bar; the diamond cell of size 2 is narrower than two
    cutoffs, so pairs interact through several periodic images."""
    import re

    from tests.util import oracle_backed_model

    from cuda_mace.tools import model_surgery

    src = tmp_path / "source.model"
    torch.save(oracle_backed_model(channels=32, atomic_numbers=(1, 6, 7, 8), avg_num_neighbors=60.0, seed=3), src)
    out_path = tmp_path / "optimized.model"
    model_surgery.main(["--model", str(src), "--size", "2", "--accuracy", "--output", str(out_path)])
    printed = capsys.readouterr().out
    errs = {m.group(1): (float(m.group(2)), float(m.group(3)))
            for m in re.finditer(r"absolute (\w+) error \(mean, max\)---\n(\S+) (\S+)", printed)}
    energy = float(re.search(r"energy org tensor\(\[([-0-9.e]+)", printed).group(1))
    assert set(errs) == {"energy", "forces"}, printed
    assert errs["energy"][1] <= 1e-5 * abs(energy), printed
    assert errs["forces"][1] <= 1e-4, printed
    assert torch.load(out_path, weights_only=False).orig_model is not None
