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


def test_bench_line_fits_the_record():
    """The one JSON line of a default bench run, with every workload present
    and every number at full width, stays under bench.LINE_LIMIT characters, so
    that a record keeping the last 8,000 characters of the output holds the
    whole line -- and BASELINE's configurations come last in it."""
    import json
    import os
    import sys
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    import bench

    def result(key):
        return {"workload": key, "description": "d" * 90, "dtype": "f32",
                "ms_per_step": 0.123456789, "median_ms_per_step": 0.123456789,
                "sustained_ms_per_step": 0.123456789, "GBps": 5555.123456789,
                "items_per_s": 1.23456789e12, "pct_hbm_peak": 69.123456789,
                "algorithmic_bytes": 1207959552,
                "roofline": {"bound": "hbm", "kernel": "k" * 56, "achieved": 5555.123456789,
                             "peak": 8000.0, "unit": "GB/s", "frac": 0.70123456789,
                             "kernel_ms": 0.123456789, "traffic": 1207959552},
                "cpu_baseline": {"value": 11.123456789, "unit": "GB/s", "cores": 16,
                                 "kind": "port", "items_per_s": 1.23456789e9,
                                 "single_thread_value": 10.123456789, "sample": "s" * 160}}
    keys = [k for k in bench.DEFAULT_EXTRA.split(",")]
    assert set(bench.BASELINE_EXTRA) <= set(keys)
    others = {k: result(k) for k in keys}
    yard = {k: 0.123456789 for k in ("read_nt_256MiB", "store_1GiB_runs",
                                     "store_1GiB_runs_read2KB", "store_1GiB_runs_read4KB",
                                     "store_1GiB_eighths",
                                     "read_64MiB_behind_store_1GiB")}
    device = {"name": "AMD Instinct MI355X", "compute_units": 256, "hbm_peak_used_GBps": 8000.0,
              "memory_clock_khz": 2000000, "memory_bus_width_bits": 8192}
    line = bench.format_line(result("c2_segreduce_f32"), others, yard, device, 20, 5, 4)
    assert len(line) < bench.LINE_LIMIT, len(line)
    parsed = json.loads(line)
    for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step",
              "higher_is_better", "scaling", "vs_baseline", "dtype", "data", "config",
              "roofline", "cpu_baseline"):
        assert k in parsed
    assert list(parsed["others"])[-len(bench.BASELINE_EXTRA):] == list(bench.BASELINE_EXTRA)
    assert parsed["others"]["c3_load_balance_search"]["frac_of_yardstick"] == 1.0
    assert bench.sig(0.123456789) == 0.12346 and bench.sig(7) == 7 and bench.sig(None) is None
