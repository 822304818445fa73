"""CPU tests of the device plugin's sub-allocator (plugin/arena_allocator.h) over a host-memory raw
allocator: alignment, no overlap, exact accounting, coalescing, region growth, limits, failure of the
raw allocator, and a seeded random workload."""
import ctypes as C
import os
import random

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "mock_tf", "libarena_test.so")
KB, MB = 1 << 10, 1 << 20
NAMES = ("num_allocs", "bytes_in_use", "peak_bytes_in_use", "largest_alloc_size", "bytes_reserved",
         "peak_bytes_reserved", "bytes_limit", "largest_free_block_bytes", "num_regions")


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(LIB):
        import importlib.util
        spec = importlib.util.spec_from_file_location("mock_tf_build", os.path.join(HERE, "mock_tf", "build.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        mod.build()
    l = C.CDLL(LIB)
    l.arena_new.restype = C.c_void_p
    l.arena_new.argtypes = [C.c_uint64] * 3
    l.arena_alloc.restype = C.c_void_p
    l.arena_alloc.argtypes = [C.c_void_p, C.c_uint64]
    l.arena_free.argtypes = [C.c_void_p, C.c_void_p]
    l.arena_allocated_size.restype = C.c_uint64
    l.arena_allocated_size.argtypes = [C.c_void_p, C.c_void_p]
    l.arena_stats.argtypes = [C.c_void_p, C.POINTER(C.c_int64)]
    l.arena_raw_counts.argtypes = [C.c_void_p, C.POINTER(C.c_int64)]
    l.arena_delete.argtypes = [C.c_void_p]
    return l


def stats(lib, h):
    out = (C.c_int64 * 9)()
    lib.arena_stats(h, out)
    return dict(zip(NAMES, out))


def raw(lib, h):
    out = (C.c_int64 * 3)()
    lib.arena_raw_counts(h, out)
    return tuple(out)


def test_alignment_rounding_and_split(lib):
    h = lib.arena_new(0, 1 * MB, 0)
    a = lib.arena_alloc(h, 1)
    b = lib.arena_alloc(h, 257)
    c = lib.arena_alloc(h, 0)  # a zero-byte request still gets a distinct, aligned chunk
    assert a % 256 == 0 and b % 256 == 0 and c % 256 == 0 and len({a, b, c}) == 3
    assert lib.arena_allocated_size(h, a) == 256 and lib.arena_allocated_size(h, b) == 512
    assert b == a + 256 and c == b + 512  # carved front to back out of one region
    s = stats(lib, h)
    assert s["num_allocs"] == 3 and s["bytes_in_use"] == 256 + 512 + 256 and s["num_regions"] == 1
    assert s["bytes_reserved"] == 1 * MB and s["largest_free_block_bytes"] == 1 * MB - 1024
    assert raw(lib, h)[0] == 1
    assert lib.arena_delete(h) == 0


def test_free_coalesces_with_both_neighbours(lib):
    h = lib.arena_new(0, 1 * MB, 0)
    p = [lib.arena_alloc(h, 64 * KB) for _ in range(16)]  # fills the region exactly
    assert stats(lib, h)["largest_free_block_bytes"] == 0
    for i in (3, 5):
        assert lib.arena_free(h, p[i]) == 0
    assert stats(lib, h)["largest_free_block_bytes"] == 64 * KB
    assert lib.arena_free(h, p[4]) == 0  # joins its left and right neighbours
    assert stats(lib, h)["largest_free_block_bytes"] == 3 * 64 * KB
    big = lib.arena_alloc(h, 3 * 64 * KB)  # fits without growing
    assert big == p[3] and stats(lib, h)["num_regions"] == 1
    for q in p[:3] + p[6:] + [big]:
        assert lib.arena_free(h, q) == 0
    s = stats(lib, h)
    assert s["bytes_in_use"] == 0 and s["largest_free_block_bytes"] == s["bytes_reserved"] == 1 * MB
    assert lib.arena_delete(h) == 0


def test_double_free_and_foreign_pointer_are_refused(lib):
    h = lib.arena_new(0, 1 * MB, 0)
    a = lib.arena_alloc(h, 1000)
    assert lib.arena_free(h, a + 256) == 1   # inside an allocation, not its start
    assert lib.arena_free(h, a) == 0
    assert lib.arena_free(h, a) == 1         # already free
    assert lib.arena_free(h, 0) == 0         # null is a no-op
    assert stats(lib, h)["bytes_in_use"] == 0
    assert lib.arena_delete(h) == 0


def test_regions_grow_geometrically_and_best_fit_reuses_them(lib):
    h = lib.arena_new(0, 1 * MB, 0)
    a = lib.arena_alloc(h, 1 * MB)        # region 1: 1 MB
    b = lib.arena_alloc(h, 1 * MB)        # region 2: 2 MB
    c = lib.arena_alloc(h, 3 * MB)        # region 3: 4 MB
    s = stats(lib, h)
    assert s["num_regions"] == 3 and s["bytes_reserved"] == 7 * MB
    d = lib.arena_alloc(h, 10 * MB)       # larger than the next step (8 MB): region of its own size
    s = stats(lib, h)
    assert s["num_regions"] == 4 and s["bytes_reserved"] == 17 * MB and s["largest_alloc_size"] == 10 * MB
    # best fit: a 512 KB request takes the 1 MB hole of region 2 rather than the 1 MB... both are 1 MB; free `a` too
    lib.arena_free(h, a)
    e = lib.arena_alloc(h, 900 * KB)
    assert stats(lib, h)["num_regions"] == 4
    for q in (b, c, d, e):
        assert lib.arena_free(h, q) == 0
    # chunks of different regions never merge
    assert stats(lib, h)["largest_free_block_bytes"] == 10 * MB
    assert lib.arena_delete(h) == 0


def test_limit_and_raw_allocator_failure(lib):
    h = lib.arena_new(3 * MB, 1 * MB, 0)  # total limit 3 MB
    a = lib.arena_alloc(h, 1 * MB)
    b = lib.arena_alloc(h, 1 * MB + 1)    # wants a 2 MB region: exactly the rest of the limit
    assert a and b and stats(lib, h)["bytes_reserved"] == 3 * MB
    assert lib.arena_alloc(h, 1 * MB) is None  # 768 KB - 256 B are free, 1 MB is not, and the limit forbids growing
    assert lib.arena_alloc(h, 512 * KB)
    assert lib.arena_delete(h) == 0
    # a raw allocator that only has 5 MB: the 4 MB region request backs off to what is needed
    h = lib.arena_new(0, 4 * MB, 5 * MB)
    a = lib.arena_alloc(h, 3 * MB)        # region of 4 MB
    b = lib.arena_alloc(h, 1 * MB + 256)  # does not fit the 1 MB tail; 8 MB, 4 MB, 2 MB regions fail; exact size fails too
    assert a and b is None
    c = lib.arena_alloc(h, 1 * MB)        # the tail of region 1
    assert c == a + 3 * MB
    d = lib.arena_alloc(h, 512 * KB)      # backs off 8 -> 4 -> 2 -> 1 MB
    assert d and stats(lib, h)["bytes_reserved"] == 5 * MB
    assert lib.arena_delete(h) == 0


def test_random_workload_invariants(lib):
    rng = random.Random(1234)
    h = lib.arena_new(0, 4 * MB, 0)
    live = {}
    in_use = 0
    peak = 0
    for step in range(4000):
        if live and (rng.random() < 0.45 or len(live) > 300):
            p = rng.choice(list(live))
            in_use -= live.pop(p)
            assert lib.arena_free(h, p) == 0
        else:
            n = rng.choice([1, 100, 255, 256, 4000, 70000, 1 << 20, 3 << 20]) + rng.randrange(0, 50)
            p = lib.arena_alloc(h, n)
            assert p and p % 256 == 0
            size = lib.arena_allocated_size(h, p)
            assert n <= size < n + 512  # rounded to 256, never split below one granule
            live[p] = size
            in_use += size
            peak = max(peak, in_use)
        if step % 97 == 0:
            spans = sorted((p, p + s) for p, s in live.items())
            assert all(a[1] <= b[0] for a, b in zip(spans, spans[1:]))  # no two live allocations overlap
            s = stats(lib, h)
            assert s["bytes_in_use"] == in_use and s["peak_bytes_in_use"] == peak
            assert s["bytes_in_use"] + s["largest_free_block_bytes"] <= s["bytes_reserved"]
    for p in list(live):
        assert lib.arena_free(h, p) == 0
    s = stats(lib, h)
    assert s["bytes_in_use"] == 0
    allocs, frees, live_bytes = raw(lib, h)
    assert allocs == s["num_regions"] and frees == 0 and live_bytes == s["bytes_reserved"]
    assert lib.arena_delete(h) == 0  # every region went back to the raw allocator
