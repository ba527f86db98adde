"""The sort entry point that allocates nothing (cm_stable_key_sort_static) against cm_stable_key_sort, through the C
ABI: index work, so the results must be identical.  Two calls in a row share the built-in scratch buffer, the second
with a smaller input, so stale counters or bucket entries of the first call would show."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _pair(n, nkeys, seed, device):
    g = torch.Generator().manual_seed(seed)
    keys = torch.randint(0, max(nkeys, 1), (n,), generator=g, dtype=torch.int32).to(device)
    return keys


def test_static_sort_matches_workspace_sort_on_two_calls_in_a_row():
    from cuda_mace import _cabi

    dev = torch.device("cuda:0")
    # outputs pre-allocated up front: the calls under test allocate nothing
    cases = [(1_301_200, 25_000, 0), (4_097, 300, 1), (100_000, 11, 2), (0, 5, 3), (33, 1, 4), (5_000, 64, 5)]
    keys = [_pair(n, k, s, dev) for n, k, s in cases]
    perms = [torch.full((n,), -7, dtype=torch.int32, device=dev) for n, _, _ in cases]
    offs = [torch.full((k + 1,), -7, dtype=torch.int32, device=dev) for _, k, _ in cases]
    want = [_cabi.stable_key_sort(kk, k) for kk, (_, k, _) in zip(keys, cases)]
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    for kk, (n, k, _), p, o in zip(keys, cases, perms, offs):
        _cabi.stable_key_sort_static(kk, k, p, o)
    assert torch.cuda.memory_allocated() == before
    torch.cuda.synchronize()
    for (n, k, _), p, o, (wp, wo), kk in zip(cases, perms, offs, want, keys):
        assert torch.equal(p, wp), (n, k)
        assert torch.equal(o, wo), (n, k)
        if n:
            # independent check: stable order by key
            ref = torch.sort(kk.long() * n + torch.arange(n, device=dev)).indices.int()
            assert torch.equal(p, ref)
    # a repeat of the large case after the small ones
    _cabi.stable_key_sort_static(keys[0], cases[0][1], perms[0].fill_(-1), offs[0].fill_(-1))
    assert torch.equal(perms[0], want[0][0]) and torch.equal(offs[0], want[0][1])


def test_static_sort_rejects_sizes_beyond_its_buffer():
    from cuda_mace import _cabi

    cap = _cabi.lib.cm_stable_key_sort_static_capacity()
    assert cap == 32 << 20
    dev = torch.device("cuda:0")
    n = cap // 4 + 1
    keys = torch.zeros(n, dtype=torch.int32, device=dev)
    perm = torch.empty(n, dtype=torch.int32, device=dev)
    offsets = torch.empty(2, dtype=torch.int32, device=dev)
    with pytest.raises(_cabi.CudaMaceError, match="built-in"):
        _cabi.stable_key_sort_static(keys, 1, perm, offsets)


def test_static_sort_inside_a_captured_graph():
    """After the set-up call the entry point only enqueues kernels: recorded into a HIP graph, every replay sorts the
    keys that are in the input buffer at that time."""
    from cuda_mace import _cabi

    dev = torch.device("cuda:0")
    assert _cabi.lib.cm_stable_key_sort_static_capacity() == 32 << 20  # looks the buffer up for this device
    n, nkeys = 20_000, 700
    keys = _pair(n, nkeys, 11, dev)
    perm = torch.empty(n, dtype=torch.int32, device=dev)
    offsets = torch.empty(nkeys + 1, dtype=torch.int32, device=dev)
    _cabi.stable_key_sort_static(keys, nkeys, perm, offsets)  # warm call outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _cabi.stable_key_sort_static(keys, nkeys, perm, offsets)
    for seed in (12, 13, 14):
        keys.copy_(_pair(n, nkeys, seed, dev))
        perm.fill_(-1), offsets.fill_(-1)
        graph.replay()
        torch.cuda.synchronize()
        want_perm, want_off = _cabi.stable_key_sort(keys, nkeys)
        assert torch.equal(perm, want_perm) and torch.equal(offsets, want_off), seed
