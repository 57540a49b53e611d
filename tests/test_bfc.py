"""BFC arena bookkeeping (host only): the reference's own test sequence
(cuda/bfc_test.go:47-120) plus differential runs against a literal Python
restatement of cuda/bfc.go on random alloc/free traffic."""
import random

import pytest

from gorgonia_amd.engine import BFC
from oracle.bfc_oracle import OOM, BFCOracle


def both(align=32, start=0, size=1024):
    a, b = BFC(align), BFCOracle(align)
    a.reserve(start, size)
    b.reserve(start, size)
    return a, b


@pytest.mark.parametrize("impl", ["product", "oracle"])
def test_reference_sequence(impl):
    """TestBFC: free-list lengths 2, 2, 3, 4, 3 and reuse of the freed address."""
    if impl == "product":
        bfc = BFC(32)
        bfc.reserve(0, 1024)
        flen, flist = bfc.freelist_len, bfc.freelist
    else:
        bfc = BFCOracle(32)
        bfc.reserve(0, 1024)
        flen, flist = (lambda: bfc.freelist.l), bfc.freelist.blocks
    with pytest.raises(ValueError):
        bfc.alloc(0)
    addr0 = bfc.alloc(21)
    assert addr0 % 32 == 0 and flen() == 2
    assert flist() == [(21, 11), (32, 992)]
    addr1 = bfc.alloc(32)
    assert addr1 % 32 == 0 and flen() == 2
    assert flist() == [(21, 11), (64, 960)]
    addr2 = bfc.alloc(69)
    assert addr2 % 32 == 0 and flen() == 3
    assert flist() == [(21, 11), (133, 27), (160, 864)]
    bfc.free(addr1)
    assert flen() == 4
    addr3 = bfc.alloc(32)
    assert addr3 == addr1 and flen() == 3
    bfc.free(addr3)
    bfc.free(addr2)  # third free of four allocs: 0.75 -> coalesce
    assert flist() == [(21, 11), (32, 992)]
    bfc.coalesce()
    assert flist() == [(21, 11), (32, 992)]
    bfc.free(addr0)
    assert flist() == [(0, 1024)]


def test_align():
    b = BFC(32)
    assert [b.align(s) for s in (1, 31, 32, 33, 64, 69)] == [32, 32, 32, 64, 64, 96]


def test_unknown_free_is_ignored_and_oom_reports():
    b = BFC(32)
    b.reserve(4096, 256)
    b.free(12345)  # silently ignored (cuda/bfc.go:394-401)
    a = b.alloc(200)
    assert a == 4096
    with pytest.raises(MemoryError) as ei:
        b.alloc(100)
    assert "allocated/reserved: 200/256" in str(ei.value)  # cuda/errors.go:13
    b.free(a)
    assert b.alloc(256) == 4096


def test_oom_retries_after_coalesce():
    """Fragmented but sufficient space: alloc coalesces and succeeds (cuda/bfc.go:363-372)."""
    a, o = both(32, 0, 1024)
    pa = [a.alloc(64) for _ in range(16)]
    po = [o.alloc(64) for _ in range(16)]
    assert pa == po
    for p in pa[:8]:
        a.free(p)
        o.free(p)
    assert a.alloc(512) == o.alloc(512) == 0


@pytest.mark.parametrize("seed", range(12))
def test_differential_random_traffic(seed):
    rng = random.Random(seed)
    align = rng.choice([32, 64, 256])
    start = rng.choice([0, 4096, 1 << 32])
    size = rng.choice([4096, 65536, 1 << 20])
    a, o = both(align, start, size)
    live = []
    for step in range(600):
        if live and rng.random() < 0.45:
            p = live.pop(rng.randrange(len(live)))
            a.free(p)
            o.free(p)
        else:
            sz = rng.choice([1, 7, 21, 32, 69, 100, 256, 1000, 4097]) * rng.choice([1, 1, 3])
            try:
                want = o.alloc(sz)
            except OOM:
                with pytest.raises(MemoryError):
                    a.alloc(sz)
                assert a.freelist() == o.freelist.blocks(), f"step {step} (after OOM)"
                continue
            got = a.alloc(sz)
            assert got == want, f"step {step}: alloc({sz})"
            live.append(got)
        assert a.freelist() == o.freelist.blocks(), f"step {step}"
        assert a.allocated() == o.allocated
    a.reset_allocator()
    o.reset_allocator()
    assert a.freelist() == o.freelist.blocks() == [(0, size)]
    assert a.used_count() == 0


def test_deterministic_addresses_after_reset():
    """The same alloc/free order after ResetAllocator gives the same addresses
    (what makes a tape segment's pointer set stable across runs)."""
    b = BFC(32)
    b.reserve(1 << 20, 1 << 16)
    def run():
        ps = [b.alloc(s) for s in (100, 3000, 64, 7)]
        b.free(ps[1])
        ps.append(b.alloc(2000))
        return ps
    first = run()
    b.reset_allocator()
    assert run() == first
