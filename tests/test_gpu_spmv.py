"""CSR spmv through the C ABI.  Tolerance: |y_gpu - y_exact| <= tol * sum_k
|a_k x_k| per row with tol = 1e-5 (fp32) / 1e-12 (fp64); y_exact is a float64
evaluation (scipy / the oracle's float64 loop)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _check(w, dtype, tol, oracle):
    import moderngpu_amd as m
    mat, x = w["matrix"].astype(dtype), w["vector"].astype(dtype)
    got = m.spmv(_dev(mat), _dev(w["columns"]), _dev(x), _dev(w["segments"])).cpu().numpy()
    exact = oracle.spmv(mat.astype(np.float64), w["columns"], x.astype(np.float64), w["segments"])
    norm = oracle.spmv_abs(mat, w["columns"], x, w["segments"])
    assert got.dtype == dtype
    assert np.all(np.abs(got - exact) <= tol * norm + 1e-300)
    serial = oracle.spmv(mat, w["columns"], x, w["segments"])
    assert np.all(np.abs(got.astype(np.float64) - serial) <= 2 * tol * norm + 1e-300)
    return got


@pytest.mark.parametrize("dtype,tol", [(np.float32, 1e-5), (np.float64, 1e-12)])
def test_spmv_config4_scaled(dev, oracle, dtype, tol):
    from moderngpu_amd import workloads
    _check(workloads.config4(scale=64), dtype, tol, oracle)


def test_spmv_empty_rows_and_small(dev, oracle):
    import moderngpu_amd as m
    mat = np.array([2.0, 3.0], dtype=np.float32)
    col = np.array([1, 0], dtype=np.int32)
    x = np.array([10.0, 100.0], dtype=np.float32)
    segs = np.array([0, 0, 1, 2, 2], dtype=np.int32)
    got = m.spmv(_dev(mat), _dev(col), _dev(x), _dev(segs)).cpu().numpy()
    assert list(got) == [0.0, 200.0, 30.0, 0.0, 0.0]


def test_spmv_identity_and_scipy(dev):
    import scipy.sparse as sp
    import moderngpu_amd as m
    rng = np.random.default_rng(31)
    n = 20000
    eye = sp.identity(n, dtype=np.float64, format="csr")
    x = rng.standard_normal(n)
    got = m.spmv(_dev(eye.data), _dev(eye.indices.astype(np.int32)), _dev(x),
                 _dev(eye.indptr[:-1].astype(np.int32))).cpu().numpy()
    assert np.array_equal(got, x)
    a = sp.random(n, n, density=0.002, format="csr", random_state=5, dtype=np.float64)
    got = m.spmv(_dev(a.data), _dev(a.indices.astype(np.int32)), _dev(x),
                 _dev(a.indptr[:-1].astype(np.int32))).cpu().numpy()
    want = a @ x
    norm = abs(a) @ np.abs(x)
    assert np.all(np.abs(got - want) <= 1e-12 * norm + 1e-300)


def test_spmv_full_size_config4(dev):
    """2^22 rows / ~2^26 nonzeros, checked on the device against torch's own
    CSR product in float64."""
    import torch
    import moderngpu_amd as m
    from moderngpu_amd import workloads
    w = workloads.config4()
    mat, col, x, segs = (_dev(w[k]) for k in ("matrix", "columns", "vector", "segments"))
    got = m.spmv(mat, col, x, segs)
    rows = segs.numel()
    lens = torch.diff(torch.cat([segs.long(), torch.tensor([w["nnz"]], device=dev)]))
    prod = mat.double() * x.double()[col.long()]
    want = torch.segment_reduce(prod, "sum", lengths=lens, unsafe=True)
    norm = torch.segment_reduce(prod.abs(), "sum", lengths=lens, unsafe=True)
    assert torch.all((got.double() - want).abs() <= 1e-5 * norm + 1e-30)
