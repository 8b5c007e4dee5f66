"""Seeded synthetic inputs for the five benchmark configurations.

Everything is generated on the host with numpy's PCG64 so that a (config,
seed, scale) triple always yields the same arrays.  ``scale`` divides the item
and segment counts of a configuration (power of two) so the tests can run the
same shapes at sizes a CPU checker finishes in seconds.

Segment descriptors follow moderngpu's convention: ``segments[s]`` is the index
of the first item of segment ``s``; ascending; ``segments[0] == 0``; no
trailing ``count`` entry; equal consecutive starts are empty segments.
"""
import functools
import os

import numpy as np


def _disk_cached(fn):
    """With MGPU_WORKLOAD_CACHE naming a directory, a configuration's arrays are
    kept there as .npz and loaded instead of being generated again (several
    profiler runs of one workload in a row)."""
    @functools.wraps(fn)
    def wrapper(*args, **kwargs):
        folder = os.environ.get("MGPU_WORKLOAD_CACHE")
        if not folder:
            return fn(*args, **kwargs)
        tag = "_".join([fn.__name__] + [str(a) for a in args] +
                       ["%s-%s" % kv for kv in sorted(kwargs.items())])
        path = os.path.join(folder, tag + ".npz")
        if os.path.exists(path):
            with np.load(path, allow_pickle=False) as z:
                return {k: (z[k].item() if z[k].ndim == 0 else z[k]) for k in z.files}
        out = fn(*args, **kwargs)
        os.makedirs(folder, exist_ok=True)
        np.savez(path + ".tmp.npz", **out)
        os.replace(path + ".tmp.npz", path)
        return out
    return wrapper


def _starts(lengths):
    s = np.zeros(lengths.size, dtype=np.int64)
    np.cumsum(lengths[:-1], out=s[1:])
    assert s[-1] + lengths[-1] < 2 ** 31
    return s.astype(np.int32)


def _stochastic_round(x, rng):
    lo = np.floor(x)
    return (lo + (rng.random(x.size) < (x - lo))).astype(np.int64)


def _fix_total(lengths, total, rng, floor=0):
    """Adds/removes single items on random segments until sum == total."""
    diff = int(total - lengths.sum())
    while diff != 0:
        step = 1 if diff > 0 else -1
        pool = np.flatnonzero(lengths > floor) if step < 0 else np.arange(lengths.size)
        pick = rng.choice(pool, size=min(abs(diff), pool.size), replace=False)
        lengths[pick] += step
        diff = int(total - lengths.sum())
    return lengths


def _bounded_zipf(s, cap, size, rng):
    """Zipf(s) on {1..cap} by inverse CDF (numpy's zipf is unbounded)."""
    k = np.arange(1, cap + 1, dtype=np.float64)
    cdf = np.cumsum(k ** (-s))
    cdf /= cdf[-1]
    return (np.searchsorted(cdf, rng.random(size), side="left") + 1).astype(np.int64)


def config1(seed=42, count=1_000_000, num_segments=10_000):
    """C1: int32 sum, values uniform in [0,100); starts = 0 followed by
    num_segments-1 sorted uniform offsets in [0,count), duplicates kept."""
    rng = np.random.Generator(np.random.PCG64(seed))
    values = rng.integers(0, 100, size=count, dtype=np.int32)
    starts = np.zeros(num_segments, dtype=np.int32)
    starts[1:] = np.sort(rng.integers(0, count, size=num_segments - 1, dtype=np.int32))
    return {"values": values, "segments": starts, "op": "plus", "init": 0}


def config2_segments(seed=42, scale=1):
    count, num_segments = (1 << 26) // scale, (1 << 20) // scale
    rng = np.random.Generator(np.random.PCG64(seed))
    lengths = rng.geometric(1.0 / 64.0, size=num_segments).astype(np.int64)
    lengths[rng.random(num_segments) < 0.05] = 0
    lengths = _stochastic_round(lengths * (count / lengths.sum()), rng)
    lengths = _fix_total(lengths, count, rng)
    return count, _starts(lengths)


@_disk_cached
def config2(seed=42, scale=1):
    """C2: fp32 sum, 2^26 values uniform [0,1), 2^20 segments with geometric
    lengths (mean 64), ~5% forced empty, total exactly 2^26."""
    count, starts = config2_segments(seed, scale)
    rng = np.random.Generator(np.random.PCG64(seed + 1))
    values = rng.random(count, dtype=np.float32)
    return {"values": values, "segments": starts, "op": "plus", "init": 0.0}


@_disk_cached
def config3(seed=42, scale=1):
    """C3: load-balancing search / interval_expand.  2^24 segments whose
    lengths are Zipf(1.2) on [1, 2^16], scaled (stochastic rounding, so many
    short draws become empty segments) to a total of 2^28 work items; one
    int32 value per segment uniform in [0, 2^31)."""
    num_segments = (1 << 24) // scale
    count = (1 << 28) // scale
    rng = np.random.Generator(np.random.PCG64(seed))
    lengths = _bounded_zipf(1.2, 1 << 16, num_segments, rng)
    lengths = _stochastic_round(lengths * (count / lengths.sum()), rng)
    lengths = _fix_total(lengths, count, rng)
    values = rng.integers(0, 2 ** 31, size=num_segments, dtype=np.int64).astype(np.int32)
    return {"count": count, "segments": _starts(lengths), "values": values}


@_disk_cached
def config4(seed=42, scale=1):
    """C4: CSR spmv, 2^22 rows, nnz/row = 1 + scaled Zipf(1.5) on [1,4096]
    (mean ~16, at least 1, at most 4096), columns uniform and sorted inside
    each row, fp32 matrix and x uniform in [-1,1)."""
    rows = (1 << 22) // scale
    rng = np.random.Generator(np.random.PCG64(seed))
    z = _bounded_zipf(1.5, 4096, rows, rng)
    extra = _stochastic_round((z - 1) * (15.0 / max((z - 1).mean(), 1e-9)), rng)
    lengths = np.minimum(1 + extra, 4096)
    nnz = int(lengths.sum())
    starts = _starts(lengths)
    cols = rng.integers(0, rows, size=nnz, dtype=np.int64)
    # sort columns inside each row: sort by (row, col) with one key.
    row_of = np.repeat(np.arange(rows, dtype=np.int64), lengths)
    order = np.argsort(row_of * rows + cols, kind="stable")
    cols = cols[order].astype(np.int32)
    matrix = (rng.random(nnz, dtype=np.float32) * 2 - 1).astype(np.float32)
    vector = (rng.random(rows, dtype=np.float32) * 2 - 1).astype(np.float32)
    return {"matrix": matrix, "columns": cols, "vector": vector,
            "segments": starts, "nnz": nnz}


def config5_segments(seed=42, scale=1):
    count, num_segments = (1 << 27) // scale, (1 << 18) // scale
    rng = np.random.Generator(np.random.PCG64(seed))
    lengths = (rng.random(num_segments) < 0.5).astype(np.int64)
    big = [num_segments // 8, 3 * num_segments // 8, 5 * num_segments // 8,
           7 * num_segments // 8]
    lengths[big] = 0
    rest = count - int(lengths.sum())
    share = rest // 4
    for i, b in enumerate(big):
        lengths[b] = share + (rest - 4 * share if i == 3 else 0)
    return count, _starts(lengths)


@_disk_cached
def config5(seed=42, scale=1, kind="f64max"):
    """C5: extreme skew.  2^27 values, 2^18 segments: four hold ~2^25 items
    each, every other one is empty or has one item.  kind = 'f64max' (normal
    (0,1) doubles, max) or 'i64sum' (int64 uniform in [-2^40, 2^40), sum)."""
    count, starts = config5_segments(seed, scale)
    rng = np.random.Generator(np.random.PCG64(seed + 1))
    if kind == "f64max":
        values = rng.standard_normal(count)
        return {"values": values, "segments": starts, "op": "maximum",
                "init": float("-inf")}
    values = rng.integers(-(1 << 40), 1 << 40, size=count, dtype=np.int64)
    return {"values": values, "segments": starts, "op": "plus", "init": 0}


def reference_test_segments(count, num_segments, seed):
    """Segment starts shaped like the reference's own segreduce test
    (tests/test_segreduce.cu:16-22): 0 followed by sorted uniform draws from
    the closed range [0, count] -- a start may equal count (trailing empty
    segments).  numpy's generator replaces std::mt19937, so the draws differ
    from the reference's but the distribution is the same; fixtures made with
    std::mt19937 itself are under tests/golden/."""
    rng = np.random.Generator(np.random.PCG64(seed))
    starts = np.zeros(num_segments, dtype=np.int32)
    starts[1:] = np.sort(rng.integers(0, count + 1, size=num_segments - 1))
    return starts
