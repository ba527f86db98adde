"""Seeded synthetic inputs shared by the tests (shapes of benchmark configuration 2, the isolated message-passing op at 4096 nodes, and smaller)."""
import numpy as np
import torch


def random_graph(nnodes, avg_degree, seed, degree_mode="poisson", isolated_frac=0.0):
    """Receiver-sorted edge list with uniformly random senders (any directed multigraph)."""
    rng = np.random.default_rng(seed)
    if degree_mode == "fixed":
        deg = np.full(nnodes, avg_degree, dtype=np.int64)
    else:
        deg = rng.poisson(avg_degree, nnodes).astype(np.int64)
    if isolated_frac > 0:
        deg[rng.random(nnodes) < isolated_frac] = 0
    receiver = np.repeat(np.arange(nnodes), deg).astype(np.int32)
    sender = rng.integers(0, max(nnodes, 1), receiver.shape[0]).astype(np.int32)
    return torch.from_numpy(sender), torch.from_numpy(receiver)


def mp_inputs(nnodes, nedges, channels, seed, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    X = torch.randn(nnodes, channels, generator=g, dtype=dtype)
    v = torch.randn(nedges, 3, generator=g, dtype=dtype)
    R = torch.randn(nedges, 4, channels, generator=g, dtype=dtype)
    G = torch.randn(nnodes, 16, channels, generator=g, dtype=dtype)
    return X, v, R, G


def close(actual, expected, rtol, atol_scale):
    """assert_close with an absolute tolerance proportional to the magnitude of the expected data."""
    expected = expected.double()
    actual = actual.double().cpu()
    scale = float(expected.abs().max()) if expected.numel() else 1.0
    torch.testing.assert_close(actual, expected, rtol=rtol, atol=atol_scale * max(scale, 1e-30))
