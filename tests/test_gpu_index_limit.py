"""The largest inputs the 32-bit index space allows: count + num_segments =
2^31 - 1.  Expected results are computed on the device with independent torch
operations (searchsorted, cumsum) in chunks; everything is integer and must
match exactly.  These catch index arithmetic that passes 2^31 on the way
(tile ends, rounded-up divisions)."""
import pytest
import torch

pytestmark = pytest.mark.gpu

TOTAL = (1 << 31) - 1
CHUNK = 1 << 27


def _starts(count, nseg, dev, seed):
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    s = torch.randint(0, count + 1, (nseg,), dtype=torch.int64, device=dev, generator=g)
    s[0] = 0
    s[-3:] = count                      # empty segments at the very end
    return torch.sort(s).values.to(torch.int32)


def _segment_of(segs, lo, hi):
    idx = torch.arange(lo, hi, dtype=torch.int64, device=segs.device)
    return torch.searchsorted(segs.long(), idx, right=True) - 1


def test_load_balance_search_and_expand_at_the_index_limit(dev):
    import moderngpu_amd as m
    nseg = 1 << 20
    count = TOTAL - nseg
    segs = _starts(count, nseg, dev, 1)
    out = m.load_balance_search(count, segs)
    torch.cuda.synchronize()
    for lo in range(0, count, CHUNK):
        hi = min(lo + CHUNK, count)
        assert torch.equal(out[lo:hi].long(), _segment_of(segs, lo, hi)), lo
    vals = torch.arange(nseg, dtype=torch.int32, device=dev) * 7 + 3
    out = m.interval_expand(vals, count, segs, out=out)
    torch.cuda.synchronize()
    for lo in range(0, count, CHUNK):
        hi = min(lo + CHUNK, count)
        assert torch.equal(out[lo:hi].long(), _segment_of(segs, lo, hi) * 7 + 3), lo


def test_segreduce_at_the_index_limit(dev):
    import moderngpu_amd as m
    nseg = 1 << 16
    count = TOTAL - nseg
    segs = _starts(count, nseg, dev, 2)
    values = torch.empty(count, dtype=torch.int32, device=dev)
    for lo in range(0, count, CHUNK):                  # fill in pieces
        hi = min(lo + CHUNK, count)
        values[lo:hi] = (torch.arange(lo, hi, dtype=torch.int64, device=dev) * 2654435761 >> 7
                         ).to(torch.int32)
    got = m.segreduce(values, segs, "plus", -5)
    torch.cuda.synchronize()
    # Inclusive prefix sums in int64, a chunk at a time, sampled at the ends.
    ends = torch.cat([segs[1:].long(), torch.tensor([count], device=dev)])
    begins = segs.long()
    before_end = torch.zeros(nseg, dtype=torch.int64, device=dev)     # sum of values[:end]
    before_begin = torch.zeros(nseg, dtype=torch.int64, device=dev)
    carry = torch.zeros((), dtype=torch.int64, device=dev)
    for lo in range(0, count, CHUNK):
        hi = min(lo + CHUNK, count)
        cs = torch.cumsum(values[lo:hi].long(), 0) + carry
        for at, dst in ((ends, before_end), (begins, before_begin)):
            sel = (at > lo) & (at <= hi)
            dst[sel] = cs[at[sel] - lo - 1]
        carry = cs[-1].clone()
        del cs
    want = (before_end - before_begin).to(torch.int32)                # wraps like int32 '+'
    want[ends == begins] = -5
    assert torch.equal(got, want)


def test_scan_at_the_index_limit(dev):
    import moderngpu_amd as m
    count = TOTAL
    values = torch.empty(count, dtype=torch.int32, device=dev)
    for lo in range(0, count, CHUNK):
        hi = min(lo + CHUNK, count)
        values[lo:hi] = (torch.arange(lo, hi, dtype=torch.int64, device=dev) % 5).to(torch.int32)
    red = torch.zeros(1, dtype=torch.int32, device=dev)
    out, _ = m.scan(values, "plus", inclusive=False, reduction=red)
    torch.cuda.synchronize()
    carry = torch.zeros((), dtype=torch.int64, device=dev)
    for lo in range(0, count, CHUNK):
        hi = min(lo + CHUNK, count)
        v = values[lo:hi].long()
        cs = torch.cumsum(v, 0) + carry
        assert torch.equal(out[lo:hi], (cs - v).to(torch.int32)), lo
        carry = cs[-1].clone()
        del cs, v
    assert int(red.item()) == int(carry.to(torch.int32).item())
