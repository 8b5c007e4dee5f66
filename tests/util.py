"""Helpers shared by the GPU parity tests."""
import numpy as np


def lengths_of(segments, count):
    return np.diff(np.append(np.asarray(segments, dtype=np.int64), count))


def random_segments(rng, count, nseg, dup=0.3, closed=True):
    """0 followed by sorted uniform starts in [0, count] (closed: a start may
    equal count), with runs of equal starts forced in (empty segments)."""
    s = np.zeros(nseg, dtype=np.int32)
    if nseg > 1:
        draws = rng.integers(0, count + (1 if closed else 0), size=nseg - 1)
        if dup > 0 and nseg > 4:
            k = max(1, int(dup * (nseg - 1)))
            draws[rng.integers(0, nseg - 1, size=k)] = draws[rng.integers(0, nseg - 1, size=k)]
        s[1:] = np.sort(draws)
    return s


def segment_layouts(rng, nv):
    """(name, count, segments) cases aimed at tile and spine boundaries for a
    tile of nv merged elements."""
    cases = []
    cases.append(("single_item", 1, np.array([0], np.int32)))
    cases.append(("one_segment_small", 100, np.array([0], np.int32)))
    cases.append(("one_segment_many_tiles", 5 * nv + 17, np.array([0], np.int32)))
    cases.append(("all_empty_but_last", 50, np.zeros(40, np.int32)))
    cases.append(("all_trailing_empty", 3 * nv, np.concatenate(
        [[0], np.full(2 * nv + 5, 3 * nv)]).astype(np.int32)))
    cases.append(("unit_segments", 3 * nv + 1, np.arange(3 * nv + 1, dtype=np.int32)))
    # a segment boundary exactly where a tile ends: tile 0 holds nv - k items
    # and k starts; put the k-th start right at item nv - k.
    for k in (1, 2, 7):
        starts = np.concatenate([[0], np.full(k - 1, 0), [nv - k]]).astype(np.int32) if k > 1 \
            else np.array([0, nv - 1], np.int32)
        cases.append(("boundary_on_tile_edge_%d" % k, 4 * nv, starts))
    # starts clustered on one item in the middle of a long run of items
    cases.append(("burst_of_empties", 6 * nv, np.concatenate(
        [[0], np.full(nv + nv // 2, 2 * nv + 3), [5 * nv]]).astype(np.int32)))
    # many segments, few items
    cases.append(("segments_dominate", 37, random_segments(rng, 37, 3 * nv)))
    # zero items
    cases.append(("no_items", 0, np.zeros(5, np.int32)))
    # skew: a few giant segments among unit/empty ones
    lens = (rng.random(4000) < 0.5).astype(np.int64)
    lens[[500, 1500, 2500, 3500]] = [3 * nv + 1, 7 * nv, nv, 2 * nv - 1]
    starts = np.concatenate([[0], np.cumsum(lens)[:-1]]).astype(np.int32)
    cases.append(("giants_among_units", int(lens.sum()), starts))
    # tiles with more starts than threads: short segments of one length, of
    # mixed lengths below and around the 32 items a thread folds by itself,
    # and short ones with a long one in the middle of a tile
    for length in (3, 8):
        n = 3 * nv + 5
        cases.append(("dense_len%d" % length, n, np.arange(0, n, length, dtype=np.int32)))
    for top in (12, 33, 70):
        lens = rng.integers(0, top + 1, size=nv)
        starts = np.concatenate([[0], np.cumsum(lens)[:-1]]).astype(np.int32)
        cases.append(("dense_mixed_to_%d" % top, int(lens.sum()), starts))
    lens = rng.integers(0, 4, size=2 * nv)
    lens[nv // 3] = nv // 2 + 3
    lens[nv] = 33
    starts = np.concatenate([[0], np.cumsum(lens)[:-1]]).astype(np.int32)
    cases.append(("dense_with_long", int(lens.sum()), starts))
    for i in range(4):
        count = int(rng.integers(1, 6 * nv))
        nseg = int(rng.integers(1, 2 * nv))
        cases.append(("random_%d" % i, count, random_segments(rng, count, nseg)))
    return cases
