"""The freed-block cache behind the component's mem_alloc / mem_free
(xccl_amd/csrc/mc_pool.c), exercised on the host: the C library's allocator
stands in for the device's (tests/pool_harness.c)."""
import ctypes
import os
import random
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "xccl_amd", "csrc")
KiB, MiB, GiB = 1 << 10, 1 << 20, 1 << 30


class Stats(ctypes.Structure):
    _fields_ = [("hits", ctypes.c_uint64), ("misses", ctypes.c_uint64), ("backing_frees", ctypes.c_uint64),
                ("cached_bytes", ctypes.c_size_t), ("live_blocks", ctypes.c_size_t), ("free_blocks", ctypes.c_size_t)]


@pytest.fixture()
def pool(tmp_path):
    """A fresh copy of the library per test: the cache is process-global state."""
    out = str(tmp_path / "libpool_harness.so")
    subprocess.run(["gcc", "-shared", "-fPIC", "-O1", "-g", "-Wall", "-Wextra", "-Werror", "-I", CSRC, "-o", out,
                    os.path.join(ROOT, "tests", "pool_harness.c"), os.path.join(CSRC, "mc_pool.c"), "-lpthread",
                    "-Wl,-Bsymbolic"],      # bind the harness to ITS copy of the cache, whatever else the process loaded
                   check=True)
    lib = ctypes.CDLL(out)
    lib.mc_pool_size_class.restype = ctypes.c_size_t
    lib.mc_pool_size_class.argtypes = [ctypes.c_size_t]
    lib.mc_pool_alloc.argtypes = [ctypes.c_int, ctypes.POINTER(ctypes.c_void_p), ctypes.c_size_t]
    lib.mc_pool_free.argtypes = [ctypes.c_void_p]
    lib.mc_pool_set_limit.argtypes = [ctypes.c_size_t]
    lib.mc_pool_trim.argtypes = [ctypes.c_int]
    lib.mc_pool_get_stats.argtypes = [ctypes.POINTER(Stats)]
    lib.harness_configure.argtypes = [ctypes.c_size_t]
    lib.harness_backing_allocs.restype = ctypes.c_long
    lib.harness_backing_frees.restype = ctypes.c_long
    lib.harness_stress.restype = ctypes.c_long
    lib.harness_configure(64 * MiB)
    return lib


def alloc(lib, n, dev=0):
    p = ctypes.c_void_p()
    rc = lib.mc_pool_alloc(dev, ctypes.byref(p), n)
    return rc, p.value


def stats(lib):
    s = Stats()
    lib.mc_pool_get_stats(ctypes.byref(s))
    return s


def test_size_class_properties(pool):
    assert pool.mc_pool_size_class(0) == 0
    assert pool.mc_pool_size_class(1) == 4096 and pool.mc_pool_size_class(4096) == 4096
    assert pool.mc_pool_size_class((1 << 62) + 1) == 0            # too large to round: not cached
    rng = random.Random(7)
    lens = [rng.randrange(1, 1 << rng.randrange(1, 41)) for _ in range(4000)]
    lens += [(1 << k) + d for k in range(12, 40) for d in (-1, 0, 1)]
    prev = None
    for n in sorted(lens):
        c = pool.mc_pool_size_class(n)
        assert c >= n and c >= 4096
        if n >= 4096:
            assert c <= n + n // 8 + 1, (n, c)                    # at most 12.5 % over
        assert pool.mc_pool_size_class(c) == c                    # a class is its own class
        assert prev is None or c >= prev                          # monotone
        prev = c
    # headline scratch: 7 vectors of 256 MiB stays exact
    assert pool.mc_pool_size_class(7 * 256 * MiB) == 7 * 256 * MiB


def test_freed_block_is_handed_out_again(pool):
    rc, a = alloc(pool, 100 * KiB)
    assert rc == 0 and a
    assert pool.mc_pool_free(a) == 0
    assert stats(pool).free_blocks == 1 and stats(pool).cached_bytes == pool.mc_pool_size_class(100 * KiB)
    rc, b = alloc(pool, 99 * KiB)               # same class
    assert rc == 0 and b == a
    s = stats(pool)
    assert (s.hits, s.misses, s.free_blocks, s.live_blocks, s.cached_bytes) == (1, 1, 0, 1, 0)
    rc, c = alloc(pool, 100 * KiB)              # the only block of that class is live
    assert rc == 0 and c != a
    assert pool.mc_pool_free(b) == 0 and pool.mc_pool_free(c) == 0
    rc, d = alloc(pool, 100 * KiB, dev=1)       # another device never gets device 0's block
    assert rc == 0 and d not in (a, c)
    rc, e = alloc(pool, 300 * KiB)              # another class neither
    assert rc == 0 and e not in (a, c, d)
    assert pool.mc_pool_free(d) == 0 and pool.mc_pool_free(e) == 0
    pool.mc_pool_trim(-1)
    s = stats(pool)
    assert s.free_blocks == 0 and s.cached_bytes == 0 and s.live_blocks == 0
    assert pool.harness_backing_allocs() == pool.harness_backing_frees() == 4


def test_limit_evicts_least_recently_freed(pool):
    pool.mc_pool_set_limit(3 * MiB)
    blocks = [alloc(pool, MiB)[1] for _ in range(4)]
    for b in blocks:
        assert pool.mc_pool_free(b) == 0
        assert stats(pool).cached_bytes <= 3 * MiB
    s = stats(pool)
    assert s.free_blocks == 3 and s.backing_frees == 1
    got = {alloc(pool, MiB)[1] for _ in range(3)}
    assert got == set(blocks[1:])               # blocks[0] was freed first, so it is the one that left
    assert stats(pool).hits == 3
    for b in got:
        pool.mc_pool_free(b)
    rc, big = alloc(pool, 8 * MiB)              # larger than the whole limit: never cached
    assert rc == 0
    before = pool.harness_backing_frees()
    assert pool.mc_pool_free(big) == 0
    assert pool.harness_backing_frees() == before + 1 and stats(pool).free_blocks == 3
    pool.mc_pool_set_limit(MiB)                 # shrinking releases at once
    assert stats(pool).free_blocks == 1 and stats(pool).cached_bytes == MiB


def test_limit_zero_is_a_pass_through(pool):
    pool.mc_pool_set_limit(0)
    rc, a = alloc(pool, 64 * KiB)
    assert rc == 0 and pool.mc_pool_free(a) == 0
    s = stats(pool)
    assert (s.hits, s.free_blocks, s.live_blocks, s.cached_bytes) == (0, 0, 0, 0)
    assert pool.harness_backing_allocs() == pool.harness_backing_frees() == 1
    # a block that was live when caching was switched off is still released properly
    pool.mc_pool_set_limit(MiB)
    rc, b = alloc(pool, 64 * KiB)
    pool.mc_pool_set_limit(0)
    assert pool.mc_pool_free(b) == 0
    assert pool.harness_backing_allocs() == pool.harness_backing_frees() == 2 and stats(pool).live_blocks == 0


def test_double_free_and_null(pool):
    assert pool.mc_pool_free(None) == 0
    rc, a = alloc(pool, 5000)
    assert pool.mc_pool_free(a) == 0
    assert pool.mc_pool_free(a) == -1           # reported, and the cached block is untouched
    assert stats(pool).free_blocks == 1
    assert alloc(pool, 5000)[1] == a
    assert alloc(pool, 0)[0] == 0               # zero bytes go straight to the backing allocator


def test_more_live_blocks_than_the_table_holds(pool):
    ptrs = [alloc(pool, 4096)[1] for _ in range(300)]
    assert len(set(ptrs)) == 300
    assert stats(pool).live_blocks == 256
    for p in ptrs:
        assert pool.mc_pool_free(p) == 0
    s = stats(pool)
    assert s.live_blocks == 0 and s.free_blocks == 256
    pool.mc_pool_trim(-1)
    assert pool.harness_backing_allocs() == pool.harness_backing_frees() == 300


def test_backing_failure_empties_the_cache_and_retries(pool):
    rc, a = alloc(pool, MiB)
    pool.mc_pool_free(a)
    assert stats(pool).free_blocks == 1
    pool.harness_fail_next(1)
    rc, b = alloc(pool, 2 * MiB)
    assert rc == 0 and b
    assert stats(pool).free_blocks == 0         # the cached block was given back before the second attempt
    pool.harness_fail_next(2)
    rc, c = alloc(pool, 4 * MiB)
    assert rc != 0                              # both attempts failed: the error comes back
    assert pool.mc_pool_free(b) == 0


def test_random_sequence_never_hands_out_a_live_block(pool):
    rng = random.Random(11)
    pool.mc_pool_set_limit(2 * MiB)
    live = {}
    sizes = [3000, 4096, 10000, 70000, 70001, 300000, MiB]
    for _ in range(4000):
        if live and rng.random() < 0.5:
            p = rng.choice(list(live))
            assert pool.mc_pool_free(p) == 0
            del live[p]
        else:
            n, dev = rng.choice(sizes), rng.randrange(2)
            rc, p = alloc(pool, n, dev)
            assert rc == 0 and p not in live
            live[p] = (n, dev)
        s = stats(pool)
        assert s.cached_bytes <= 2 * MiB and s.live_blocks == len(live)
    for p in live:
        assert pool.mc_pool_free(p) == 0
    pool.mc_pool_trim(0)
    pool.mc_pool_trim(1)
    s = stats(pool)
    assert s.free_blocks == 0 and s.cached_bytes == 0
    assert pool.harness_backing_allocs() == pool.harness_backing_frees()


def test_four_threads(pool):
    assert pool.harness_stress(4, 20000) == 0
    pool.mc_pool_trim(-1)
    s = stats(pool)
    assert s.live_blocks == 0 and s.free_blocks == 0
    assert pool.harness_backing_allocs() == pool.harness_backing_frees()
    assert s.hits > 0
