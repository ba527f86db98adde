"""DeviceCalculator: Verlet list on the GPU + graph replays reproduce the model on an exact, freshly built list."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("use_graph", [True, False], ids=["graph", "eager"])
def test_md_like_walk(cabi, use_graph):
    from cuda_mace.calculators import DeviceCalculator
    from cuda_mace.models import OptimizedInvariantMACE, SyntheticInvariantMACE
    from cuda_mace.utils.neighbour_list import neighbour_data
    from cuda_mace.utils.synthetic import make_system, to_device

    n = 400
    data = to_device(make_system(n, 10, seed=11, density=0.1), "cuda")
    avg = data["edge_index"].shape[1] / n
    model = OptimizedInvariantMACE(SyntheticInvariantMACE(channels=64, atomic_numbers=tuple(range(1, 11)),
                                                          avg_num_neighbors=avg, seed=12), device="cuda")
    calc = DeviceCalculator(model, data["node_attrs"], cutoff=5.0, skin=0.4, pbc=(True, True, True), cell=data["cell"],
                            use_graph=use_graph)
    g = torch.Generator(device="cuda").manual_seed(1)
    pos = data["positions"].clone()
    for it in range(25):
        pos = pos + 0.03 * torch.randn(pos.shape, device="cuda", dtype=pos.dtype, generator=g)
        got = calc.compute(pos)
        exact = model(neighbour_data(pos.clone(), data["node_attrs"], 5.0, (True, True, True), data["cell"]))
        scale = float(exact["forces"].abs().max())
        torch.testing.assert_close(got["energy"], exact["energy"].detach(), rtol=1e-7, atol=1e-7)
        torch.testing.assert_close(got["forces"], exact["forces"].detach(), rtol=0, atol=2e-6 * scale)
    assert 1 < calc.builds < 25 and calc.steps == 25
