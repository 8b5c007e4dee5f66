"""expt::lbs_workcreate through the C ABI (counts read from an array) against
the CPU checker: sizes, new segment starts and the (item, segment, rank) each
new segment comes from are all integers and must match exactly.  Then a
breadth-first search whose frontier is rebuilt by the GPU engine level by
level, against scipy's shortest path lengths."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _segments(rng, count, nseg):
    s = np.zeros(nseg, dtype=np.int32)
    if nseg > 1:
        s[1:] = np.sort(rng.integers(0, count + 1, size=nseg - 1))
    return s


def _check(oracle, dev, created, segments):
    import moderngpu_amd as m
    got = m.workcreate(torch.from_numpy(created).to(dev), torch.from_numpy(segments).to(dev))
    torch.cuda.synchronize()
    want = oracle.workcreate(created, segments)
    assert got[0] == want[0]
    for name, g, w in zip(("starts", "index", "seg", "rank"), got[1:], want[1:]):
        assert np.array_equal(g.cpu().numpy(), w), name


@pytest.mark.parametrize("count,nseg,keep", [
    (0, 0, 0.5), (0, 9, 0.5), (1, 1, 1.0), (77, 5, 0.5), (3071, 1, 1.0), (3072, 2, 0.0),
    (3073, 3000, 0.5), (100003, 1000, 0.01), (100003, 90000, 0.99),
    ((1 << 22) + 5, 1 << 18, 0.3), (1 << 22, 3, 0.001)])
def test_workcreate_matches_oracle(oracle, dev, count, nseg, keep):
    rng = np.random.default_rng(count + nseg)
    segments = _segments(rng, count, nseg) if nseg else np.zeros(0, np.int32)
    if count and not nseg:
        pytest.skip("items need a segment")
    created = rng.integers(1, 12, size=count).astype(np.int32)
    created[rng.random(count) >= keep] = 0
    created[rng.random(count) < 0.02] = -1
    _check(oracle, dev, created, segments)


def test_workcreate_every_item_creates_long_segments(oracle, dev):
    count = 500000
    segments = np.array([0, 10, 10, 400000], dtype=np.int32)
    _check(oracle, dev, np.full(count, 4000, dtype=np.int32), segments)   # sums to 2e9 < 2^31


def test_bfs_frontier_rebuilt_on_gpu_vs_scipy(dev):
    import scipy.sparse as sp
    from scipy.sparse.csgraph import shortest_path
    import moderngpu_amd as m
    rng = np.random.default_rng(9)
    n, live = 60000, 54000
    rows = np.concatenate([np.arange(live), rng.integers(0, live, live // 2),
                           np.zeros(2000, dtype=np.int64)])
    cols = np.concatenate([(np.arange(live) + 1) % live, rng.integers(0, live, live // 2),
                           rng.integers(0, live, 2000)])
    a = sp.coo_matrix((np.ones(rows.size), (rows, cols)), shape=(n, n))
    a = ((a + a.T) > 0).astype(np.int8).tocsr()
    source = 23
    want = shortest_path(a, unweighted=True, indices=source)
    want = np.where(np.isinf(want), -1, want).astype(np.int64)

    indptr = torch.from_numpy(a.indptr.astype(np.int64)).to(dev)
    indices = torch.from_numpy(a.indices.astype(np.int64)).to(dev)
    level = torch.full((n,), -1, dtype=torch.int64, device=dev)
    level[source] = 0
    segments = torch.zeros(1, dtype=torch.int32, device=dev)
    first_edge = indptr[source:source + 1].clone()
    count, depth = int(indptr[source + 1] - indptr[source]), 0
    while segments.numel():
        seg, rank = m.transform_lbs(count, segments)
        w = indices[first_edge[seg.long()] + rank.long()]
        # "first edge to reach an undiscovered vertex creates its out-edges":
        # the first occurrence of each new vertex in item order.
        fresh = level[w] == -1
        order = torch.arange(count, device=dev)
        first_hit = torch.full((n,), count, dtype=torch.int64, device=dev)
        first_hit.scatter_reduce_(0, w[fresh], order[fresh], reduce="amin")
        creates = fresh & (first_hit[w] == order)
        level[w[creates]] = depth + 1
        created = torch.where(creates, indptr[w + 1] - indptr[w], 0).to(torch.int32)
        new_count, new_segments, src, src_seg, src_rank = m.workcreate(created, segments)
        nw = indices[first_edge[src_seg.long()] + src_rank.long()]
        assert torch.equal(nw, w[src.long()])
        segments, first_edge, count = new_segments, indptr[nw], new_count
        depth += 1
    assert np.array_equal(level.cpu().numpy(), want)
