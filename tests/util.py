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


def carve_cluster(data, centre, r_atoms, r_receivers, cutoff=5.0):
    """The neighbourhood of atom `centre` of a periodic cubic box as a non-periodic cluster for the fp64 reference.

    A two-layer model with cutoff rc is local: the energy of node n depends on atoms within 2 rc of n, so the force on
    atom i depends on atoms within 4 rc of i.  The cluster holds every periodic image within r_atoms of the centre,
    unwrapped, and every pair within the cutoff whose receiving end lies within r_receivers of the centre.  With
    r_atoms = 4 rc and r_receivers = 3 rc the features of layer 1 are exact within 3 rc, node energies within 2 rc, and
    the derivative of the cluster's energy with respect to the centre's position is the force of the full system
    (nodes beyond 2 rc have wrong energies that do not depend on the centre).  Returns (cluster data, original index
    of every cluster atom, distance of every cluster atom from the centre)."""
    from scipy.spatial import cKDTree

    pos = data["positions"].numpy()
    box = float(data["cell"][0, 0])
    assert box > 2 * r_atoms, "images must be unique inside the cluster"
    d = pos - pos[centre]
    d -= box * np.round(d / box)
    dist = np.linalg.norm(d, axis=1)
    keep = np.flatnonzero(dist < r_atoms)
    cpos, cdist = d[keep], dist[keep]
    pairs = cKDTree(cpos).query_pairs(cutoff, output_type="ndarray")
    snd = np.concatenate([pairs[:, 0], pairs[:, 1]])
    rcv = np.concatenate([pairs[:, 1], pairs[:, 0]])
    live = cdist[rcv] < r_receivers
    snd, rcv = snd[live], rcv[live]
    order = np.lexsort((rcv, snd))
    cluster = {
        "positions": torch.from_numpy(cpos.copy()),
        "node_attrs": data["node_attrs"][keep],
        "edge_index": torch.from_numpy(np.stack([snd[order], rcv[order]]).astype(np.int64)),
        "shifts": torch.zeros(int(live.sum()), 3, dtype=torch.float64),
    }
    return cluster, keep, cdist


def reference_on_fresh_list(params, positions, node_attrs, box, cutoff=5.0, strain=None, compute_forces=True):
    """The fp64 reference model on a neighbour list built on the host (scipy) for these positions in a cubic periodic
    box; `strain` (3x3, symmetric) deforms positions and cell together, for finite-difference virials."""
    from cuda_mace.utils.synthetic import neighbour_list
    from oracle import mace_model as M

    pos = np.asarray(positions, dtype=np.float64)
    ei, S = neighbour_list(pos, cutoff, box)
    cell = np.eye(3) * box
    if strain is not None:
        pos = pos + pos @ strain
        cell = cell + cell @ strain
    data = {"positions": torch.from_numpy(pos), "node_attrs": node_attrs.detach().cpu().double(),
            "edge_index": torch.from_numpy(ei), "shifts": torch.from_numpy(S @ cell)}
    return M.energy_and_forces(params, data, compute_forces=compute_forces)


def oracle_backed_model(**kwargs):
    """A source model for the conversion tool that can also be called, like an upstream model: the random-init weight
    container of the package with a forward that evaluates the fp64 reference (oracle) on the host."""
    from cuda_mace.models import SyntheticInvariantMACE

    return OracleBackedMACE(**kwargs)


def _oracle_forward(self, data, training=False, compute_force=True, **unused):
    from oracle import mace_model as M

    cpu = {k: v.detach().cpu() for k, v in data.items()}
    out = M.energy_and_forces(self.export_params(), cpu, compute_forces=compute_force)
    dev = data["positions"].device
    return {k: (v.to(dev) if v is not None else None) for k, v in out.items()}


try:
    from cuda_mace.models import SyntheticInvariantMACE as _Synthetic

    class OracleBackedMACE(_Synthetic):
        forward = _oracle_forward
except ImportError:  # the package needs its built library; tests that use this class fail loudly on their own
    OracleBackedMACE = None


def spatial_order_reference(positions, batch, edge_index, shifts, r_max, bins=64):
    """Host restatement (numpy, library sorts) of the relabelling that cm_graph_prepare performs on the device:
    (perm new -> old, inverse, receiver, sender, edge_perm new -> old) with atoms sorted by (graph, grid cell, index) and
    every receiver's pairs ordered by (beyond the cutoff?, sender label | length, position in the list)."""
    import numpy as np

    pos = positions.double().cpu().numpy()
    ei = edge_index.cpu().numpy()
    sh = shifts.double().cpu().numpy()
    n = pos.shape[0]
    lo = pos.min(axis=0) if n else np.zeros(3)
    extent = float((pos.max(axis=0) - lo).max()) if n else 0.0
    width = max(extent / bins * (1.0 + 1e-12), 0.5 * r_max)
    b = np.clip(np.floor((pos - lo) / width), 0, bins - 1).astype(np.int64)
    key = ((batch.cpu().numpy().astype(np.int64) * bins + b[:, 0]) * bins + b[:, 1]) * bins + b[:, 2]
    perm = np.argsort(key, kind="stable")
    inverse = np.empty(n, dtype=np.int64)
    inverse[perm] = np.arange(n)
    v = (pos[ei[1]] - pos[ei[0]]) + sh
    length = np.sqrt((v[:, 0] * v[:, 0] + v[:, 1] * v[:, 1]) + v[:, 2] * v[:, 2])
    shell = length > r_max
    row0, row1 = inverse[ei[0]], inverse[ei[1]]
    second = np.where(shell, length, row1.astype(np.float64))  # labels are exact in fp64
    order = np.lexsort((np.arange(ei.shape[1]), second, shell, row0))  # last key is the most significant
    return perm, inverse, row0[order], row1[order], order
