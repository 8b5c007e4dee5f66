"""Wave64 CTA primitives (cta_scan_t, cta_reduce_t, cta_segscan_t, shuffles)
against serial host scans, for every CTA size and for partial counts."""
import ctypes
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
NTS = [64, 128, 256, 512, 1024]


@pytest.fixture(scope="module")
def tk(dev):
    path = os.path.join(HERE, "csrc", "libmgpu_test_kernels.so")
    assert os.path.exists(path), "build tests/csrc first (make -C tests/csrc)"
    return ctypes.CDLL(path)


def _dev(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _p(t):
    return ctypes.c_void_p(t.data_ptr())


def _fold(op, a, b):
    if op == 0:
        return a + b
    if op == 1:
        return b if a < b else a
    if op == 2:
        return b if b < a else a
    return a        # left projection: associative, not commutative


def _wrap32(x):
    return ((int(x) + 2 ** 31) % 2 ** 32) - 2 ** 31


@pytest.mark.parametrize("nt", NTS)
@pytest.mark.parametrize("op", [0, 1, 2, 3])
def test_cta_scan_i32(tk, dev, nt, op):
    import torch
    rng = np.random.default_rng(nt * 10 + op)
    for count in sorted({nt, nt - 1, 1, nt // 2 + 3, 65 if nt > 64 else 33}):
        x = rng.integers(-9, 9, size=nt).astype(np.int32)
        dx = _dev(torch, x)
        for inclusive in (0, 1):
            out = torch.zeros(nt, dtype=torch.int32, device=dev)
            red = torch.zeros(1, dtype=torch.int32, device=dev)
            assert tk.tk_scan_i32(nt, _p(dx), count, _p(out), _p(red), op, 77, inclusive) == 0
            got, gred = out.cpu().numpy(), int(red.item())
            acc = None
            want = []
            for i in range(count):
                inc = int(x[i]) if acc is None else _wrap32(_fold(op, acc, int(x[i])))
                want.append(inc if inclusive else (77 if i == 0 else acc))
                acc = inc
            assert list(got[:count]) == want, (nt, op, count, inclusive)
            assert gred == acc
            assert all(g == acc for g in got[count:])   # out-of-range threads get the total


@pytest.mark.parametrize("nt", [64, 256, 1024])
def test_cta_scan_wide_types(tk, dev, nt):
    import torch
    rng = np.random.default_rng(nt)
    x = rng.integers(-2 ** 40, 2 ** 40, size=nt).astype(np.int64)
    out = torch.zeros(nt, dtype=torch.int64, device=dev)
    red = torch.zeros(1, dtype=torch.int64, device=dev)
    assert tk.tk_scan_i64(nt, _p(_dev(torch, x)), nt, _p(out), _p(red), 0,
                          ctypes.c_longlong(5), 1) == 0
    assert np.array_equal(out.cpu().numpy(), np.cumsum(x))
    xf = rng.standard_normal(nt)
    outf = torch.zeros(nt, dtype=torch.float64, device=dev)
    redf = torch.zeros(1, dtype=torch.float64, device=dev)
    tk.tk_scan_f64.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p,
                               ctypes.c_void_p, ctypes.c_int, ctypes.c_double, ctypes.c_int]
    assert tk.tk_scan_f64(nt, _p(_dev(torch, xf)), nt, _p(outf), _p(redf), 1, 0.0, 1) == 0
    assert np.array_equal(outf.cpu().numpy(), np.maximum.accumulate(xf))


@pytest.mark.parametrize("nt,vt", [(128, 7), (256, 4), (64, 3)])
def test_cta_scan_vectorized(tk, dev, nt, vt, oracle):
    import torch
    rng = np.random.default_rng(vt)
    nv = nt * vt
    for count in (nv, nv - 5, vt + 1, 1):
        x = rng.integers(-9, 9, size=nv).astype(np.int32)
        for inclusive in (0, 1):
            for use_carry in (0, 1):
                out = torch.zeros(nv, dtype=torch.int32, device=dev)
                red = torch.zeros(1, dtype=torch.int32, device=dev)
                assert tk.tk_scan_vt_i32(nt, vt, _p(_dev(torch, x)), count, _p(out), _p(red),
                                         0, 0, inclusive, 1000, use_carry) == 0
                base = 1000 if use_carry else 0
                want, wred = oracle.scan(x[:count], "plus", 0, inclusive=bool(inclusive))
                got = out.cpu().numpy()[:count]
                assert np.array_equal(got, want + base), (nt, vt, count, inclusive, use_carry)
                assert int(red.item()) == wred + base


@pytest.mark.parametrize("nt", NTS)
def test_cta_reduce(tk, dev, nt):
    import torch
    rng = np.random.default_rng(nt + 1)
    x = rng.integers(-9, 9, size=nt).astype(np.int32)
    dx = _dev(torch, x)
    for count in sorted({nt, nt - 1, 1, 63, 64, 65} & set(range(1, nt + 1))):
        for op in (0, 1, 2, 3):
            acc = int(x[0])
            for i in range(1, count):
                acc = _wrap32(_fold(op, acc, int(x[i])))
            for all_return in (0, 1):
                out = torch.zeros(nt, dtype=torch.int32, device=dev)
                assert tk.tk_reduce_i32(nt, _p(dx), count, _p(out), op, all_return) == 0
                got = out.cpu().numpy()
                assert got[0] == acc, (nt, count, op)
                if all_return:
                    assert (got == acc).all()
    xf = rng.standard_normal(nt)
    outf = torch.zeros(nt, dtype=torch.float64, device=dev)
    assert tk.tk_reduce_f64(nt, _p(_dev(torch, xf)), nt, _p(outf), 2, 1) == 0
    assert (outf.cpu().numpy() == xf.min()).all()


def _serial_segscan(x, heads, carries, op, init, wrap=_wrap32):
    """Host statement of the cta_segscan_t contract: a run of partials starts
    at a thread with a head flag or right after a thread without carry-out;
    thread t receives the fold of its run up to t - 1 when t - 1 carries out."""
    scan, cin, left, has_left = [], [], [], []
    inc = None          # inclusive value of the thread below
    run_start = -1
    for t in range(len(x)):
        has_cin = t > 0 and bool(carries[t - 1])
        starts = bool(heads[t]) or (t > 0 and not carries[t - 1])
        scan.append(inc if has_cin else init)
        cin.append(int(has_cin))
        if starts:
            run_start = t
        if starts or inc is None:
            inc = int(x[t])
        else:
            inc = wrap(_fold(op, inc, int(x[t])))
        left.append(max(run_start, 0))
        has_left.append(int(run_start >= 0))
    return scan, cin, left, has_left


@pytest.mark.parametrize("nt", NTS)
@pytest.mark.parametrize("density", [0.0, 0.02, 0.3, 1.0])
def test_cta_segscan(tk, dev, nt, density):
    import torch
    rng = np.random.default_rng(int(nt * 100 + density * 50))
    for trial in range(3):
        x = rng.integers(-9, 9, size=nt).astype(np.int32)
        heads = (rng.random(nt) < density).astype(np.int32)
        carries = (rng.random(nt) < (0.9 if trial else 1.0)).astype(np.int32)
        for op in (0, 3):
            want_scan, want_cin, want_left, want_has = _serial_segscan(x, heads, carries, op, -5)
            scan = torch.zeros(nt, dtype=torch.int32, device=dev)
            cin = torch.zeros(nt, dtype=torch.int32, device=dev)
            left = torch.zeros(nt, dtype=torch.int32, device=dev)
            has = torch.zeros(nt, dtype=torch.int32, device=dev)
            red = torch.zeros(1, dtype=torch.int32, device=dev)
            assert tk.tk_segscan_i32(nt, _p(_dev(torch, x)), _p(_dev(torch, heads)),
                                     _p(_dev(torch, carries)), _p(scan), _p(cin), _p(left),
                                     _p(has), _p(red), op, -5) == 0
            gcin = cin.cpu().numpy()
            assert list(gcin) == want_cin
            gscan = scan.cpu().numpy()
            for t in range(nt):
                if want_cin[t]:
                    assert int(gscan[t]) == want_scan[t], (nt, density, op, t)
                else:
                    assert int(gscan[t]) == -5
            assert list(has.cpu().numpy()) == want_has
            gl = left.cpu().numpy()
            for t in range(nt):
                if want_has[t]:
                    assert gl[t] == want_left[t], (t, gl[t], want_left[t])


def test_cta_segscan_i64(tk, dev):
    import torch
    nt = 256
    rng = np.random.default_rng(5)
    x = rng.integers(-2 ** 40, 2 ** 40, size=nt).astype(np.int64)
    heads = (rng.random(nt) < 0.05).astype(np.int32)
    carries = np.ones(nt, dtype=np.int32)
    want_scan, want_cin, _, _ = _serial_segscan(x, heads, carries, 0, 0, wrap=int)
    scan = torch.zeros(nt, dtype=torch.int64, device=dev)
    ints = [torch.zeros(nt, dtype=torch.int32, device=dev) for _ in range(3)]
    red = torch.zeros(1, dtype=torch.int64, device=dev)
    assert tk.tk_segscan_i64(nt, _p(_dev(torch, x)), _p(_dev(torch, heads)),
                             _p(_dev(torch, carries)), _p(scan), _p(ints[0]), _p(ints[1]),
                             _p(ints[2]), _p(red), 0, ctypes.c_longlong(0)) == 0
    g = scan.cpu().numpy()
    for t in range(1, nt):
        assert int(g[t]) == want_scan[t]


@pytest.mark.parametrize("nt", NTS)
def test_cta_scan_bool(tk, dev, nt):
    import torch
    rng = np.random.default_rng(nt + 7)
    x = (rng.random(nt) < 0.4).astype(np.int32)
    out = torch.zeros(nt, dtype=torch.int32, device=dev)
    red = torch.zeros(1, dtype=torch.int32, device=dev)
    assert tk.tk_scan_bool(nt, _p(_dev(torch, x)), _p(out), _p(red)) == 0
    assert np.array_equal(out.cpu().numpy(), np.cumsum(x) - x)
    assert int(red.item()) == x.sum()


def test_shuffles_and_lane_queries(tk, dev):
    import torch
    x = np.arange(64, dtype=np.int32) * 3 + 1
    dx = _dev(torch, x)
    out = torch.zeros(64, dtype=torch.int32, device=dev)

    def run(mode, offset=0, width=64):
        assert tk.tk_shfl(_p(dx), _p(out), mode, offset, width) == 0
        return out.cpu().numpy().copy()

    lane = np.arange(64)
    for width in (64, 32, 16):
        for offset in (1, 2, 5, 16):
            if offset >= width:
                continue
            inside = (lane % width) >= offset
            up = np.where(inside, x[np.maximum(lane - offset, 0)], x)
            assert np.array_equal(run(0, offset, width), up)
            inside_d = (lane % width) + offset < width
            down = np.where(inside_d, x[np.minimum(lane + offset, 63)], x)
            assert np.array_equal(run(1, offset, width), down)
            assert np.array_equal(run(2, offset, width), np.where(inside, x + up, x))
            assert np.array_equal(run(3, offset, width), np.where(inside_d, x + down, x))
    assert (run(4) == int(x[0])).all()      # all-reduce with left projection
    assert np.array_equal(run(5), lane)
    assert (run(6) == int((x & 1).sum())).all()


@pytest.mark.parametrize("nt,vt", [(64, 3), (128, 7), (128, 11), (256, 4), (256, 16), (512, 12)])
def test_cta_load_balance_placement_and_merge_flags(tk, dev, oracle, nt, vt):
    """cta_load_balance_t::load_balance (placement, merge bits, strided
    index/segment/rank) and cta_load_balance_fill against the thread-by-thread
    CPU restatement, tile by tile."""
    import torch
    rng = np.random.default_rng(nt * 100 + vt)
    nv = nt * vt
    cases = [(5 * nv + 17, 40), (3 * nv, 2 * nv + 5), (nv // 2, 7), (4 * nv + 1, 900)]
    for count, nseg in cases:
        segs = np.zeros(nseg, dtype=np.int32)
        segs[1:] = np.sort(rng.integers(0, count + 1, size=nseg - 1))
        tiles = (count + nseg + nv - 1) // nv
        d_segs = _dev(torch, segs)
        parts = torch.zeros(tiles + 1, dtype=torch.int32, device="cuda")
        outs = {k: torch.full((tiles * nt,), -7, dtype=torch.int32, device="cuda")
                for k in ("a_index", "b_index", "merge_flags")}
        big = {k: torch.full((tiles * nt * vt,), -7, dtype=torch.int32, device="cuda")
               for k in ("indices", "segments", "ranks")}
        ranges = torch.zeros(4 * tiles, dtype=torch.int32, device="cuda")
        for fill_mode in (0, 1):
            rc = tk.tk_load_balance(nt, vt, count, _p(d_segs), nseg, _p(parts),
                                    _p(outs["a_index"]), _p(outs["b_index"]),
                                    _p(outs["merge_flags"]), _p(big["indices"]),
                                    _p(big["segments"]), _p(big["ranks"]), _p(ranges),
                                    fill_mode)
            assert rc == 0
            got = {k: v.cpu().numpy().reshape(tiles, nt) for k, v in outs.items()}
            gbig = {k: v.cpu().numpy().reshape(tiles, nt, vt) for k, v in big.items()}
            grange = ranges.cpu().numpy().reshape(tiles, 4)
            for cta in range(tiles):
                want = oracle.cta_load_balance(count, segs, nt, vt, cta)
                for k in ("indices", "segments", "ranks"):
                    assert np.array_equal(gbig[k][cta], want[k]), (count, nseg, cta, k, fill_mode)
                if not fill_mode:
                    for k in ("a_index", "b_index", "merge_flags"):
                        assert np.array_equal(got[k][cta], want[k]), (count, nseg, cta, k)
                    assert np.array_equal(grange[cta], want["range"]), (count, nseg, cta)
