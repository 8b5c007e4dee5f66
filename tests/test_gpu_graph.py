"""The entry points only launch kernels on the caller's stream (no allocation,
no memset, no synchronisation), so a caller may record them into a HIP graph.
One graph with segreduce, load_balance_search, interval_expand and scan is
captured on the small configuration (where three launches cost more than the
work) and replayed several times with new input values in the same buffers
and the program's own eager work between the replays; every replay is checked
against the CPU checker."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_calls_recorded_in_a_graph_replay_correctly(oracle, dev):
    import moderngpu_amd as m
    rng = np.random.default_rng(21)
    count, nseg = 1_000_000, 10_000
    segs = np.sort(rng.integers(0, count, nseg)).astype(np.int32)
    segs[0] = 0
    values = torch.zeros(count, dtype=torch.int32, device=dev)
    per_seg = torch.zeros(nseg, dtype=torch.int32, device=dev)
    segments = torch.from_numpy(segs).to(dev)

    reduced = torch.empty(nseg, dtype=torch.int32, device=dev)
    owners = torch.empty(count, dtype=torch.int32, device=dev)
    expanded = torch.empty(count, dtype=torch.int32, device=dev)
    scanned = torch.empty(count, dtype=torch.int32, device=dev)
    total = torch.empty(1, dtype=torch.int32, device=dev)

    def calls():
        m.segreduce(values, segments, "plus", -1, out=reduced)
        m.load_balance_search(count, segments, out=owners)
        m.interval_expand(per_seg, count, segments, out=expanded)
        m.scan(values, "plus", out=scanned, reduction=total)

    # Workspaces are made per stream on first use: warm them up on the stream
    # the capture uses, then record.
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        calls()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        calls()

    for replay in range(4):
        v = rng.integers(-1000, 1000, count).astype(np.int32)
        p = rng.integers(-1000, 1000, nseg).astype(np.int32)
        values.copy_(torch.from_numpy(v).to(dev))
        per_seg.copy_(torch.from_numpy(p).to(dev))
        for t in (reduced, owners, expanded, scanned, total):
            t.fill_(-7)
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(reduced.cpu().numpy(), oracle.segreduce(v, segs, "plus", -1)), replay
        assert np.array_equal(owners.cpu().numpy(), oracle.load_balance_search(count, segs)), replay
        assert np.array_equal(expanded.cpu().numpy(), oracle.interval_expand(p, count, segs)), replay
        want, want_total = oracle.scan(v, "plus", 0)
        assert np.array_equal(scanned.cpu().numpy(), want), replay
        assert int(total.item()) == int(want_total), replay
        # eager work of the program between replays
        eager = m.segreduce(values, segments, "maximum", 0)
        assert np.array_equal(eager.cpu().numpy(), oracle.segreduce(v, segs, "maximum", 0))


def test_large_call_recorded_in_a_graph_takes_new_segments(oracle, dev):
    """A call of more than 4,096 tiles has a partition kernel in front of its
    tile kernel (smaller ones let the tiles search their own splits).  The
    replays here get new segment starts in the same buffer each time: the
    partition has to run again in every replay, splits left by an earlier one
    would give wrong sums."""
    import moderngpu_amd as m
    rng = np.random.default_rng(22)
    nv = m.segreduce_tile_size(0)
    count, nseg = 4200 * nv, 150_000
    values = torch.zeros(count, dtype=torch.int32, device=dev)
    segments = torch.zeros(nseg, dtype=torch.int32, device=dev)
    reduced = torch.empty(nseg, dtype=torch.int32, device=dev)
    owners = torch.empty(count, dtype=torch.int32, device=dev)

    def calls():
        m.segreduce(values, segments, "plus", -1, out=reduced)
        m.load_balance_search(count, segments, out=owners)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        calls()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        calls()

    for replay in range(3):
        v = rng.integers(-1000, 1000, count).astype(np.int32)
        segs = np.sort(rng.integers(0, count, nseg)).astype(np.int32)
        segs[0] = 0
        values.copy_(torch.from_numpy(v).to(dev))
        segments.copy_(torch.from_numpy(segs).to(dev))
        reduced.fill_(-7)
        owners.fill_(-7)
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(reduced.cpu().numpy(), oracle.segreduce(v, segs, "plus", -1)), replay
        assert np.array_equal(owners.cpu().numpy(), oracle.load_balance_search(count, segs)), replay
        # the same call run eagerly between the replays
        eager = m.segreduce(values, segments, "plus", -1)
        assert torch.equal(eager, reduced), replay
