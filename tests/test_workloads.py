"""The synthetic inputs have the shapes BASELINE's configurations describe."""
import numpy as np

from moderngpu_amd import workloads as w


def _lengths(segments, count):
    return np.diff(np.append(segments.astype(np.int64), count))


def _valid(segments, count):
    ln = _lengths(segments, count)
    return segments[0] == 0 and (ln >= 0).all() and segments.dtype == np.int32


def test_config1():
    d = w.config1()
    assert d["values"].size == 1_000_000 and d["segments"].size == 10_000
    assert d["values"].min() >= 0 and d["values"].max() < 100
    assert _valid(d["segments"], 1_000_000)
    assert np.array_equal(w.config1()["segments"], d["segments"])     # seeded


def test_config2_small():
    d = w.config2(scale=64)
    n, s = (1 << 26) // 64, (1 << 20) // 64
    assert d["values"].size == n and d["segments"].size == s and d["values"].dtype == np.float32
    ln = _lengths(d["segments"], n)
    assert _valid(d["segments"], n) and ln.sum() == n
    assert 0.03 < (ln == 0).mean() < 0.08 and abs(ln.mean() - 64) < 1e-9


def test_config3_small():
    d = w.config3(scale=256)
    ln = _lengths(d["segments"], d["count"])
    assert d["count"] == (1 << 28) // 256 and ln.sum() == d["count"]
    assert _valid(d["segments"], d["count"]) and ln.max() > 20 * ln.mean()
    assert d["values"].min() >= 0


def test_config4_small():
    d = w.config4(scale=256)
    ln = _lengths(d["segments"], d["nnz"])
    assert ln.min() >= 1 and ln.max() <= 4096 and 12 < ln.mean() < 20
    rows = d["segments"].size
    assert d["columns"].min() >= 0 and d["columns"].max() < rows
    # sorted inside every row
    row_of = np.repeat(np.arange(rows), ln)
    same = row_of[1:] == row_of[:-1]
    assert (np.diff(d["columns"].astype(np.int64))[same] >= 0).all()


def test_config5_small():
    for kind in ("f64max", "i64sum"):
        d = w.config5(scale=64, kind=kind)
        n = (1 << 27) // 64
        ln = _lengths(d["segments"], n)
        assert ln.sum() == n and _valid(d["segments"], n)
        assert (ln > n // 8).sum() == 4 and set(np.unique(ln[ln <= n // 8])) <= {0, 1}


def test_disk_cache_returns_the_same_arrays(tmp_path, monkeypatch):
    """With MGPU_WORKLOAD_CACHE set a configuration is generated once, kept as
    .npz, and read back with the same values and types (profiler runs use
    this to start several runs of one workload quickly)."""
    monkeypatch.setenv("MGPU_WORKLOAD_CACHE", str(tmp_path))
    first = w.config5(scale=256, kind="i64sum")
    assert any(p.suffix == ".npz" for p in tmp_path.iterdir())
    again = w.config5(scale=256, kind="i64sum")
    assert set(first) == set(again)
    for key in first:
        if isinstance(first[key], np.ndarray):
            assert first[key].dtype == again[key].dtype
            assert np.array_equal(first[key], again[key])
        else:
            assert first[key] == again[key] and type(first[key]) is type(again[key])
    monkeypatch.delenv("MGPU_WORKLOAD_CACHE")
    plain = w.config5(scale=256, kind="i64sum")
    assert np.array_equal(plain["values"], first["values"])
