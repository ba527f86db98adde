"""The whole energy+forces step captured as one HIP graph: every replay must reproduce the eager step."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("natoms,channels,periodic,relabel", [(21, 64, False, False), (600, 128, True, False), (600, 64, True, True)])
def test_graph_replays_equal_eager(cabi, natoms, channels, periodic, relabel):
    from cuda_mace.models import OptimizedInvariantMACE, SyntheticInvariantMACE
    from cuda_mace.utils.graph import GraphedStep
    from cuda_mace.utils.synthetic import make_system, to_device

    if periodic:
        data = make_system(natoms, 10, seed=3, density=0.1)
        numbers = tuple(range(1, 11))
    else:
        data = make_system(natoms, 4, seed=3, density=None, cluster_box=8.0)
        numbers = (1, 6, 7, 8)
    avg = data["edge_index"].shape[1] / natoms
    model = OptimizedInvariantMACE(SyntheticInvariantMACE(channels=channels, atomic_numbers=numbers, avg_num_neighbors=avg,
                                                          seed=4), device="cuda",
                                   spatial_order_min_atoms=0 if relabel else None)  # relabel: the spatially re-ordered graph
    dev = to_device(data, "cuda")
    step = GraphedStep(model, dev)
    g = torch.Generator(device="cuda").manual_seed(0)
    base = dev["positions"].clone()
    for it in range(5):
        # small displacements keep the neighbour list valid; eager work and synchronisations between the replays
        pos = base + 0.02 * it * torch.randn(base.shape, device="cuda", dtype=base.dtype, generator=g)
        eager_in = dict(dev)
        eager_in["positions"] = pos.clone()
        eager = model(eager_in)
        torch.cuda.synchronize()
        out = step(pos)
        torch.cuda.synchronize()
        assert torch.equal(out["energy"], eager["energy"].detach()), "replay %d" % it
        assert torch.equal(out["forces"], eager["forces"].detach()), "replay %d" % it
        assert torch.equal(out["node_energy"], eager["node_energy"].detach())
    # replay without new positions repeats the last result
    again = {k: v.clone() for k, v in step().items()}
    assert torch.equal(again["forces"], eager["forces"].detach())
