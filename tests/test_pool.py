"""Allocator policy on the CPU: the real ``Pool`` (l2_torch_alloc_amd/csrc/pool.cpp) over a fake
backing store.

What the reference promises and this pool must keep (sideaware.cu:1199-1273, 1320-1352):
exact-size LIFO reuse of large blocks, 2 MiB rounding and alignment, blocks stay cached on free,
cached bytes above the start threshold are trimmed to the end threshold on a miss, a four-step
ladder before giving up with a null pointer, free(null) is a no-op, unknown pointers are
forwarded to the runtime.  Added here: pooled size classes for small requests, double-free
detection, stream hand-over syncs.
"""
import ctypes
import os
import random
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
SRC = os.path.join(HERE, "native", "pool_harness.cpp")
POOL = os.path.join(ROOT, "l2_torch_alloc_amd", "csrc", "pool.cpp")
LIB = os.path.join(HERE, "native", "libpool_harness.so")

MiB = 1 << 20
GiB = 1 << 30
FIELDS = ("large_hits", "large_misses", "small_hits", "small_carves", "slabs_acquired", "backing_acquires",
          "backing_releases", "stream_syncs", "device_syncs", "trims", "ladder_retries", "failures",
          "foreign_frees", "bytes_live", "bytes_cached_large", "bytes_cached_small", "bytes_reserved",
          "peak_reserved", "large_carves", "arenas_acquired", "bytes_free_arena", "bytes_free_slab_arena",
          "cache_folds", "refused_frees", "canonical_placements")


def build_harness():
    csrc = os.path.dirname(POOL)
    newest = max(os.path.getmtime(p) for p in (SRC, POOL, POOL[:-4] + ".h", os.path.join(csrc, "launch_plan.h"),
                                               os.path.join(csrc, "side_map.h")))
    if not os.path.exists(LIB) or os.path.getmtime(LIB) < newest:
        subprocess.run(["g++", "-std=c++17", "-O1", "-g", "-fPIC", "-shared", "-Wall", SRC, POOL, "-o", LIB],
                       check=True)
    return LIB


@pytest.fixture(scope="module")
def ph():
    L = ctypes.CDLL(build_harness())
    u, sz, vp = ctypes.c_uint64, ctypes.c_size_t, ctypes.c_void_p
    L.ph_create.restype, L.ph_create.argtypes = vp, [sz]
    L.ph_destroy.argtypes = [vp]
    L.ph_alloc.restype, L.ph_alloc.argtypes = u, [vp, sz, u, ctypes.c_int]
    L.ph_free.restype, L.ph_free.argtypes = ctypes.c_int, [vp, u, u]
    L.ph_release_unused.restype, L.ph_release_unused.argtypes = sz, [vp]
    L.ph_set_threshold.argtypes = [vp, sz]
    L.ph_set_trim.argtypes = [vp, sz, sz]
    L.ph_set_limit.argtypes = [vp, sz]
    L.ph_set_arena.argtypes = [vp, sz]
    L.ph_owns.restype, L.ph_owns.argtypes = ctypes.c_int, [vp, u]
    L.ph_block_bytes.restype, L.ph_block_bytes.argtypes = sz, [vp, u]
    L.ph_stats.restype, L.ph_stats.argtypes = ctypes.c_int, [vp, ctypes.POINTER(u), ctypes.c_int]
    L.ph_backing_used.restype, L.ph_backing_used.argtypes = sz, [vp]
    L.ph_backing_live_blocks.restype, L.ph_backing_live_blocks.argtypes = sz, [vp]
    L.ph_set_capacity.argtypes = [vp, sz]
    L.ph_set_foreign_result.argtypes = [vp, ctypes.c_int]
    L.ph_log.restype, L.ph_log.argtypes = ctypes.c_char_p, [vp]
    L.ph_clear_log.argtypes = [vp]
    L.ph_set_side_rule.argtypes = [vp, ctypes.c_int]
    L.ph_side_of.restype, L.ph_side_of.argtypes = ctypes.c_int, [vp, u]
    L.ph_round_large.restype, L.ph_round_large.argtypes = sz, [sz]
    L.ph_small_class_size.restype, L.ph_small_class_size.argtypes = sz, [sz]
    L.ph_small_class_index.restype, L.ph_small_class_index.argtypes = ctypes.c_int, [sz]
    return L


class P:
    def __init__(self, L, capacity=64 * GiB, arena=0):
        # arena=0: every large region is its own backing allocation (the reference's shape, and
        # what the policy tests below reason about); the arena tests pass a size.
        self.L, self.h = L, L.ph_create(capacity)
        L.ph_set_arena(self.h, arena)

    def close(self):
        self.L.ph_destroy(self.h)

    def alloc(self, n, stream=0, large=False):
        return self.L.ph_alloc(self.h, n, stream, int(large))

    def free(self, p, stream=0):
        return self.L.ph_free(self.h, p, stream)

    def stats(self):
        buf = (ctypes.c_uint64 * len(FIELDS))()
        n = self.L.ph_stats(self.h, buf, len(FIELDS))
        assert n == len(FIELDS)
        return dict(zip(FIELDS, buf))

    def log(self):
        return self.L.ph_log(self.h).decode().splitlines()

    def clear_log(self):
        self.L.ph_clear_log(self.h)


@pytest.fixture
def pool(ph):
    p = P(ph)
    yield p
    p.close()


# ------------------------------------------------------------------------------ rounding rules

def test_round_large(ph):
    assert ph.ph_round_large(1) == 2 * MiB
    assert ph.ph_round_large(2 * MiB) == 2 * MiB
    assert ph.ph_round_large(2 * MiB + 1) == 4 * MiB
    assert ph.ph_round_large(512 * MiB) == 512 * MiB


def test_small_classes_monotone_tight_and_aligned(ph):
    prev_size, prev_idx = 0, -1
    for n in list(range(1, 70000, 37)) + [2 ** k + d for k in range(9, 33) for d in (-1, 0, 1)]:
        c = ph.ph_small_class_size(n)
        assert c >= n and c % 512 == 0
        assert c - n <= max(511, n // 8 + 1), (n, c)      # at most 12.5 % slack above 4 KiB
        assert ph.ph_small_class_size(c) == c              # a class size is its own class
        assert ph.ph_small_class_index(n) == ph.ph_small_class_index(c)
    sizes = sorted({ph.ph_small_class_size(n) for n in range(1, 1 << 20, 101)})
    idx = [ph.ph_small_class_index(s) for s in sizes]
    assert idx == sorted(idx) and len(set(idx)) == len(idx)   # distinct sizes, distinct slots, same order


# ------------------------------------------------------------------------------ large path

def test_large_is_2mib_aligned_rounded_and_reused_lifo(pool):
    a = pool.alloc(9 * MiB)
    b = pool.alloc(9 * MiB + 5)          # rounds to the same 10 MiB
    assert a % (2 * MiB) == 0 and b % (2 * MiB) == 0 and a != b
    assert pool.stats()["bytes_live"] == 20 * MiB
    pool.free(a)
    pool.free(b)
    s = pool.stats()
    assert s["bytes_live"] == 0 and s["bytes_cached_large"] == 20 * MiB
    assert s["backing_releases"] == 0                        # freed blocks stay cached
    assert pool.alloc(10 * MiB) == b                         # newest first
    assert pool.alloc(9 * MiB + 1) == a
    assert pool.stats()["large_hits"] == 2
    c = pool.alloc(12 * MiB)                                 # another size: no reuse
    assert c not in (a, b) and pool.stats()["large_misses"] == 3


def test_near_fit_reuses_a_slightly_larger_region(pool):
    a = pool.alloc(64 * MiB)
    b = pool.alloc(72 * MiB)
    c = pool.alloc(80 * MiB)
    for p in (a, b, c):
        pool.free(p)
    # 66 MiB: no exact match; 72 MiB is within one eighth (66 + 8.25), and smaller than 80
    got = pool.alloc(66 * MiB)
    assert got == b and pool.L.ph_block_bytes(pool.h, got) == 72 * MiB
    assert pool.stats()["large_hits"] == 1 and pool.stats()["bytes_live"] == 72 * MiB
    # 40 MiB: the smallest cached region (64 MiB) is more than one eighth larger: a miss
    misses = pool.stats()["large_misses"]
    d = pool.alloc(40 * MiB)
    assert d not in (a, b, c) and pool.stats()["large_misses"] == misses + 1
    pool.free(got)
    assert pool.stats()["bytes_cached_large"] == (64 + 72 + 80) * MiB   # goes back under its own size
    assert pool.alloc(72 * MiB) == b


def test_direct_entry_points_are_always_large(pool):
    p = pool.alloc(100, large=True)
    assert p % (2 * MiB) == 0 and pool.stats()["bytes_live"] == 2 * MiB


def test_threshold_moves_the_boundary(pool):
    pool.L.ph_set_threshold(pool.h, 1 * MiB)
    p = pool.alloc(1 * MiB)
    assert p % (2 * MiB) == 0 and pool.stats()["large_misses"] == 1
    q = pool.alloc(1 * MiB - 1)
    assert pool.stats()["small_carves"] == 1 and q != p


def test_stream_handover_orders_the_new_stream_after_the_old(pool):
    a = pool.alloc(16 * MiB, stream=11)
    pool.free(a, stream=11)
    pool.clear_log()
    assert pool.alloc(16 * MiB, stream=11) == a
    assert pool.log() == []                                  # same stream: reuse is stream-ordered
    pool.free(a, stream=11)
    assert pool.alloc(16 * MiB, stream=22) == a
    assert pool.log() == ["order 11 -> 22"]            # stream 22 waits for what 11 had queued
    s = pool.alloc(4096, stream=5)
    pool.free(s, stream=5)
    pool.clear_log()
    assert pool.alloc(4096, stream=6) == s
    assert pool.log() == ["order 5 -> 6"]


def test_trim_thresholds(pool):
    pool.L.ph_set_trim(pool.h, 64 * MiB, 16 * MiB)
    blocks = [pool.alloc((8 + 2 * i) * MiB) for i in range(8)]     # 8..22 MiB, 120 MiB total
    for b in blocks:
        pool.free(b)
    assert pool.stats()["bytes_cached_large"] == 120 * MiB
    pool.clear_log()
    p = pool.alloc(100 * MiB)                                      # a miss with the cache over budget
    assert p
    s = pool.stats()
    assert s["trims"] == 1 and s["bytes_cached_large"] <= 16 * MiB
    log = pool.log()
    assert log[0] == "sync_device"                                 # drained before memory goes back
    assert log[-1] == "acquire %d" % (100 * MiB)
    # a hit never trims, whatever the cache holds
    pool.free(p)
    before = pool.stats()["backing_releases"]
    assert pool.alloc(100 * MiB) == p
    assert pool.stats()["backing_releases"] == before


def test_oom_ladder_and_null(ph):
    pool = P(ph, capacity=64 * MiB)
    try:
        a = pool.alloc(20 * MiB)
        b = pool.alloc(20 * MiB)
        small = pool.alloc(4096)                 # a 2 MiB slab
        pool.free(a)
        pool.free(b)
        pool.free(small)
        # 40 MiB cached + 2 MiB slab held; 44 MiB only fits once the caches are given back
        pool.clear_log()
        c = pool.alloc(44 * MiB)
        assert c
        log = pool.log()
        assert log[0] == "acquire_failed %d" % (44 * MiB)          # step 2
        assert "release %d" % (20 * MiB) in log                    # step 3 gives the cache back
        s = pool.stats()
        assert s["ladder_retries"] >= 1 and s["failures"] == 0
        # nothing can make 128 MiB fit: every step is walked, then null
        pool.clear_log()
        assert pool.alloc(128 * MiB) == 0
        s = pool.stats()
        assert s["failures"] == 1
        assert pool.log().count("acquire_failed %d" % (128 * MiB)) == 3
        # the pool is still usable afterwards
        pool.free(c)
        assert pool.alloc(44 * MiB) == c
    finally:
        pool.close()


def test_reserve_limit_acts_like_a_full_device(pool):
    pool.L.ph_set_limit(pool.h, 100 * MiB)
    a = pool.alloc(60 * MiB)
    assert a and pool.alloc(60 * MiB) == 0            # would hold 120 MiB
    assert pool.stats()["failures"] == 1
    pool.free(a)
    b = pool.alloc(80 * MiB)                          # fits once the cached 60 MiB is given back
    assert b and pool.stats()["bytes_reserved"] == 80 * MiB
    pool.L.ph_set_limit(pool.h, 0)
    assert pool.alloc(60 * MiB)


def test_release_unused_returns_everything_cached(pool):
    a = pool.alloc(32 * MiB)
    smalls = [pool.alloc(1000) for _ in range(10)]
    keep = pool.alloc(3000)
    pool.free(a)
    for s in smalls:
        pool.free(s)
    released = pool.L.ph_release_unused(pool.h)
    assert released == 32 * MiB + 2 * MiB             # the large block and the now-empty 1 KiB-class slab
    st = pool.stats()
    assert st["bytes_cached_large"] == 0
    assert pool.L.ph_backing_live_blocks(pool.h) == 1  # only the slab that holds `keep`
    assert pool.L.ph_owns(pool.h, keep)
    # and the classes still work after their slabs were taken away
    again = pool.alloc(1000)
    assert again and pool.L.ph_owns(pool.h, again)


# ------------------------------------------------------------------------------ arenas

def test_regions_are_carved_from_one_arena_and_coalesce(ph):
    pool = P(ph, arena=64 * MiB)
    try:
        a, b, c = pool.alloc(16 * MiB), pool.alloc(16 * MiB), pool.alloc(16 * MiB)
        assert pool.log() == ["acquire %d" % (64 * MiB)]               # one driver call for all three
        assert b == a + 16 * MiB and c == b + 16 * MiB
        assert all(p % (2 * MiB) == 0 for p in (a, b, c))
        st = pool.stats()
        # the first request needed the driver (a miss); the next two were carved from what it brought
        assert st["large_misses"] == 1 and st["large_carves"] == 2
        assert st["arenas_acquired"] == 1 and st["bytes_free_arena"] == 16 * MiB
        # a freed region comes back exactly while it is cached (LIFO, as in the reference) ...
        pool.free(b)
        assert pool.stats()["bytes_cached_large"] == 16 * MiB
        assert pool.alloc(16 * MiB) == b and pool.stats()["large_hits"] == 1
        # ... and a request of a size that is not cached folds the cache back into the arena first and
        # is carved, best fit, from what is free then: here from the hole b leaves, not from the
        # 16 MiB tail, and not from the driver
        pool.free(b)
        d = pool.alloc(10 * MiB)
        st = pool.stats()
        assert d == b and st["backing_acquires"] == 1 and st["cache_folds"] == 1 and st["bytes_cached_large"] == 0
        assert st["bytes_free_arena"] == 6 * MiB + 16 * MiB
        e = pool.alloc(16 * MiB)
        assert e == c + 16 * MiB
        b = e
        # everything freed and folded back: the extents merge into the whole arena, which goes home
        for p in (a, b, c, d):
            pool.free(p)
        assert pool.L.ph_release_unused(pool.h) == 64 * MiB
        assert pool.L.ph_backing_used(pool.h) == 0 and pool.stats()["bytes_free_arena"] == 0
        assert "release %d" % (64 * MiB) in pool.log()
    finally:
        pool.close()


def test_request_larger_than_an_arena_gets_its_own(ph):
    pool = P(ph, arena=64 * MiB)
    try:
        p = pool.alloc(200 * MiB)
        # plus two pages of slack: a region of 32 MiB or more may have to start one page into its arena
        assert p and pool.log() == ["acquire %d" % (204 * MiB)]
    finally:
        pool.close()


def test_arena_falls_back_to_the_request_size_when_memory_is_short(ph):
    pool = P(ph, capacity=100 * MiB, arena=64 * MiB)
    try:
        a = pool.alloc(40 * MiB)                      # arena 1: 64 MiB
        b = pool.alloc(30 * MiB)                      # does not fit the 24 MiB left; 64 MiB more would pass 100
        assert a and b
        assert pool.log() == ["acquire %d" % (64 * MiB), "acquire_failed %d" % (64 * MiB), "acquire %d" % (30 * MiB)]
    finally:
        pool.close()


def test_trim_folds_the_cache_back_and_releases_whole_arenas(ph):
    pool = P(ph, arena=64 * MiB)
    try:
        pool.L.ph_set_trim(pool.h, 100 * MiB, 0)
        blocks = [pool.alloc(32 * MiB) for _ in range(6)]         # three arenas
        keep = blocks[0]
        for b in blocks[1:]:
            pool.free(b)
        assert pool.stats()["bytes_cached_large"] == 160 * MiB
        pool.clear_log()
        big = pool.alloc(48 * MiB)                                # a miss with 160 MiB cached > 100 MiB
        assert big
        st = pool.stats()
        assert st["trims"] == 1 and st["bytes_cached_large"] == 0
        log = pool.log()
        assert log[0] == "sync_device" and log.count("release %d" % (64 * MiB)) == 2   # two wholly free arenas
        assert pool.L.ph_owns(pool.h, keep)                       # the arena with a live region stays
    finally:
        pool.close()


def test_carved_pages_wait_for_the_stream_that_freed_them(ph):
    pool = P(ph, arena=64 * MiB)
    try:
        a = pool.alloc(32 * MiB, stream=7)
        b = pool.alloc(32 * MiB, stream=8)
        pool.free(a, stream=7)
        pool.free(b, stream=8)
        pool.clear_log()
        c = pool.alloc(20 * MiB, stream=7)                        # the cache is folded back; carved from pages freed on 7 and on 8
        assert c and pool.log() == ["order 8 -> 7"]               # stream 7 waits for 8, not the host for the device
        # the rest of the extent remembers both streams
        pool.clear_log()
        d = pool.alloc(10 * MiB, stream=9)
        assert d and sorted(pool.log()) == ["order 7 -> 9", "order 8 -> 9"]
        # pages freed on the null stream are waited for like any others; never-used pages are not
        fresh = P(ph, arena=64 * MiB)
        a0 = fresh.alloc(16 * MiB, stream=0)
        fresh.free(a0, stream=0)
        fresh.clear_log()
        b0 = fresh.alloc(60 * MiB, stream=5)                      # the 16 MiB freed on stream 0 + never-used pages
        assert b0 == a0 and fresh.log() == ["order 0 -> 5"]
        fresh.close()
        # more distinct streams than an extent keeps track of: the device is drained instead
        many = P(ph, arena=64 * MiB)
        blocks = [many.alloc(8 * MiB, stream=20 + i) for i in range(6)]
        for i, blk in enumerate(blocks):
            many.free(blk, stream=20 + i)
        many.clear_log()
        assert many.alloc(44 * MiB, stream=1) and many.log() == ["sync_device"]
        many.close()
    finally:
        pool.close()


def test_cached_regions_are_folded_back_before_the_driver_is_asked(ph):
    pool = P(ph, arena=64 * MiB)
    try:
        a, b, c = pool.alloc(16 * MiB), pool.alloc(16 * MiB), pool.alloc(16 * MiB)
        pool.free(a)
        pool.free(b)
        assert pool.stats()["bytes_cached_large"] == 32 * MiB
        pool.clear_log()
        # 30 MiB: not cached, larger than the 16 MiB free tail, no cached region within one eighth.
        # The two cached neighbours are folded back, merge, and serve it: no driver call.
        d = pool.alloc(30 * MiB, stream=3)
        st = pool.stats()
        assert d == a and pool.log() == ["order 0 -> 3"]          # no driver call; freed on stream 0, taken by 3
        assert st["cache_folds"] == 1 and st["backing_acquires"] == 1 and st["bytes_cached_large"] == 0
        assert st["large_misses"] == 1 and st["large_carves"] == 3          # only the very first request was a miss
        assert st["bytes_free_arena"] == 64 * MiB - 30 * MiB - 16 * MiB
        # with one backing allocation per region (arena size 0) regions are never split: a miss stays a miss
        solo = P(ph, arena=0)
        x = solo.alloc(32 * MiB)
        solo.free(x)
        y = solo.alloc(20 * MiB)
        assert y != x and solo.stats()["cache_folds"] == 0 and solo.stats()["backing_acquires"] == 2
        solo.close()
        # pages freed on another stream are waited for when they are carved
        pool.free(d, stream=3)
        pool.free(c, stream=4)
        pool.clear_log()
        e = pool.alloc(60 * MiB, stream=5)                                    # folds again: 30 (stream 3) + 2 + 16 (stream 4) + tail
        # (the 2 MiB left over from the first fold still carry stream 0, on which they were freed)
        assert e == a and sorted(pool.log()) == ["order 0 -> 5", "order 3 -> 5", "order 4 -> 5"]
    finally:
        pool.close()


def test_slabs_are_carved_from_their_own_arenas(ph):
    pool = P(ph, arena=64 * MiB)
    try:
        big = pool.alloc(16 * MiB)
        smalls = [pool.alloc(n) for n in (1000, 5000, 70000, 300000, 3 * MiB)]   # five classes, five slabs
        assert all(smalls)
        st = pool.stats()
        assert st["slabs_acquired"] == 5
        # one arena for the large region, one for all five slabs: two driver calls, not six
        assert pool.log() == ["acquire %d" % (64 * MiB), "acquire %d" % (64 * MiB)]
        assert st["arenas_acquired"] == 2 and st["backing_acquires"] == 2
        # slabs never share an arena with large regions: all five sit in one 64 MiB window, `big` outside it
        lo = min(smalls)
        assert all(lo <= s < lo + 64 * MiB for s in smalls) and not (lo <= big < lo + 64 * MiB)
        # 2 + 2 + 2 + 6 + 48 MiB of slabs (16 blocks each, at least 2 MiB, at most 64 MiB): 60 MiB carved
        assert st["bytes_free_slab_arena"] == 64 * MiB - 60 * MiB
        # emptied slabs go back to their arena; the arena goes home once all of it is free
        for s in smalls[:-1]:
            pool.free(s)
        assert pool.L.ph_release_unused(pool.h) == 0               # the 3 MiB block still pins the arena
        assert pool.stats()["bytes_free_slab_arena"] == 64 * MiB - 48 * MiB
        again = pool.alloc(1000)                                   # carved from the arena again: no driver call
        assert again and pool.stats()["backing_acquires"] == 2
        pool.free(again)
        pool.free(smalls[-1])
        assert pool.L.ph_release_unused(pool.h) == 64 * MiB
        assert pool.stats()["bytes_free_slab_arena"] == 0
        assert pool.L.ph_backing_live_blocks(pool.h) == 1          # only the large region's arena
        assert pool.L.ph_owns(pool.h, big)
    finally:
        pool.close()


def test_slab_arena_size_is_capped(ph):
    pool = P(ph, capacity=16 * GiB, arena=4 * GiB)
    try:
        assert pool.alloc(4096)
        assert pool.log() == ["acquire %d" % (1 * GiB)]            # not the 4 GiB of a large-region arena
    finally:
        pool.close()


def test_slab_falls_back_when_the_backing_is_short(ph):
    pool = P(ph, capacity=40 * MiB, arena=64 * MiB)
    try:
        a = pool.alloc(4096)                                        # no 64 MiB arena fits: a 2 MiB one
        assert a and pool.log() == ["acquire_failed %d" % (64 * MiB), "acquire %d" % (2 * MiB)]
        big = pool.alloc(30 * MiB)
        assert big
        pool.free(big)
        pool.clear_log()
        b = pool.alloc(5 * MiB)         # its class wants a 64 MiB slab, more than the device has left
        # the cache is given back first; when 64 MiB still does not fit, a slab of one block does
        assert b and pool.stats()["failures"] == 0
        log = pool.log()
        assert "release %d" % (30 * MiB) in log and log[-1] == "acquire %d" % (6 * MiB)
        assert pool.L.ph_block_bytes(pool.h, b) == 5 * MiB
    finally:
        pool.close()


def test_large_regions_share_one_side_pattern(ph):
    """With a backing store that knows which half of the device holds which 8 KiB granule (the HIP
    one measures it), regions of 32 MiB and more are placed so that the granule at offset o is on
    side parity(o & bits 13, 21, 28) in every one of them, whatever arena they come from and
    whatever lies around them: an elementwise kernel that follows the sides of one of its arrays then finds
    the others on the same side."""
    SIDE_BITS = (1 << 13) | (1 << 21) | (1 << 28)
    p = P(ph, capacity=256 * GiB, arena=4 * GiB)
    ph.ph_set_side_rule(p.h, 1)
    rng = random.Random(3)
    live = []
    checked = fresh = placed = 0
    for step in range(600):
        if live and rng.random() < 0.45:
            ptr, n = live.pop(rng.randrange(len(live)))
            assert p.free(ptr) == 0
            continue
        n = rng.choice([8, 10, 32, 34, 64, 100, 256, 300, 1024, 1536]) * MiB
        before = p.stats()
        ptr = p.alloc(n)
        after = p.stats()
        assert ptr and ptr % (2 * MiB) == 0
        live.append((ptr, n))
        if n < 32 * MiB or after["large_hits"] > before["large_hits"]:
            continue                                       # below the size the rule applies to, or a reused region
        fresh += 1
        if after["canonical_placements"] == before["canonical_placements"]:
            # no free run could hold it that way without a large hole in front: the best fit (on the
            # right starting page when the run has a page to spare)
            continue
        placed += 1
        # up to an eighth of a region may lie past a line where the pattern flips
        hits = total = 0
        for _ in range(200):
            o = rng.randrange(0, n) & ~0x1fff
            hits += ph.ph_side_of(p.h, ptr + o) == bin(o & SIDE_BITS).count("1") & 1
            total += 1
        assert hits >= 0.85 * total, (hex(ptr), n // MiB, hits, total)
        assert ph.ph_side_of(p.h, ptr) == 0 and ph.ph_side_of(p.h, ptr + 8192) == 1
        checked += total
    assert placed >= 0.8 * fresh and placed > 50 and checked > 2000, (placed, fresh, checked)
    # blocks stay disjoint and inside what the backing store handed out
    spans = sorted(live)
    for (a, n), (b, _) in zip(spans, spans[1:]):
        assert a + n <= b
    for ptr, n in live:
        assert p.free(ptr) == 0
    assert p.stats()["bytes_live"] == 0
    # without the rule nothing changes: the best fit's front is taken
    ph.ph_set_side_rule(p.h, 0)
    before = p.stats()["canonical_placements"]
    q = p.alloc(64 * MiB)
    assert q and p.stats()["canonical_placements"] == before
    p.close()


# ------------------------------------------------------------------------------ small path

def test_small_blocks_are_pooled_and_512_aligned(pool):
    ptrs = [pool.alloc(n) for n in (1, 511, 512, 513, 4096, 4097, 100000, 7 * MiB)]
    assert all(p and p % 512 == 0 for p in ptrs)
    assert len(set(ptrs)) == len(ptrs)
    s = pool.stats()
    assert s["small_carves"] == len(ptrs) and s["large_misses"] == 0
    pool.free(ptrs[2])
    assert pool.alloc(400) == ptrs[2]                 # same class (512 B) comes straight back
    assert pool.stats()["small_hits"] == 1


def test_many_small_allocs_reach_the_backing_rarely(pool):
    ptrs = [pool.alloc(4096) for _ in range(1000)]
    assert pool.stats()["slabs_acquired"] <= 2        # 64 KiB-per-16 rule => 2 MiB slabs of 512 blocks
    for p in ptrs:
        pool.free(p)
    for _ in range(1000):
        assert pool.alloc(4096) in ptrs
    assert pool.stats()["slabs_acquired"] <= 2


def test_double_free_and_interior_pointer_are_refused(pool):
    p = pool.alloc(2048)
    assert pool.free(p) == 0
    assert pool.free(p) != 0                          # second free of the same block
    q = pool.alloc(2048)
    assert pool.free(q + 512) != 0                    # not a block start
    assert pool.L.ph_owns(pool.h, q)


@pytest.mark.parametrize("arena", [0, 4 * GiB])
def test_stale_pointers_into_the_pools_own_arenas_never_reach_the_runtime(ph, arena):
    # A second free of a large region, the base of an arena whose first region was freed, an interior
    # pointer of a live region and a pointer into free pages are all addresses the runtime's own
    # free must never see: its free of an arena's base would take the arena away from under the
    # blocks carved from it.  They are refused and counted; nothing is forwarded.
    pool = P(ph, capacity=64 * GiB, arena=arena)
    try:
        a = pool.alloc(64 * MiB)
        b = pool.alloc(32 * MiB)
        assert pool.free(a) == 0
        pool.clear_log()
        assert pool.free(a) != 0                      # double free (with arenas: a is the arena's base)
        assert pool.free(b + 2 * MiB) != 0            # interior pointer of a live region
        assert pool.free(a + 4 * MiB) != 0            # inside a cached region
        if arena:
            assert pool.free(b + 512 * MiB) != 0      # free pages of the arena, never handed out
        assert not any(l.startswith("foreign") for l in pool.log()), pool.log()
        st = pool.stats()
        assert st["foreign_frees"] == 0 and st["refused_frees"] == (4 if arena else 3)
        # the pool is intact: the cached region comes back, the live one is still live
        assert pool.alloc(64 * MiB) == a
        assert pool.L.ph_owns(pool.h, b)
        # after the cache went back to the driver the old address is foreign again, as it should be
        assert pool.free(a) == 0 and pool.free(b) == 0
        pool.L.ph_release_unused(pool.h)
        pool.clear_log()
        assert pool.free(a) == 0
        assert pool.log() == ["foreign %d" % a]
    finally:
        pool.close()


def test_free_null_and_foreign(pool):
    assert pool.free(0) == 0
    assert pool.log() == []
    pool.L.ph_set_foreign_result(pool.h, 0)
    assert pool.free(0x123456000) == 0
    assert pool.log() == ["foreign %d" % 0x123456000]
    assert pool.stats()["foreign_frees"] == 1


# ------------------------------------------------------------------------------ churn invariants

@pytest.mark.parametrize("arena", [0, 256 * MiB, 4 * GiB])
def test_random_churn_keeps_blocks_disjoint_and_accounts_balance(ph, arena):
    pool = P(ph, capacity=16 * GiB, arena=arena)
    rng = random.Random(4)
    live = {}                                         # ptr -> rounded size
    try:
        for step in range(6000):
            if live and (rng.random() < 0.45 or sum(live.values()) > 4 * GiB):
                p = rng.choice(list(live))
                assert pool.free(p) == 0
                del live[p]
            else:
                n = int(4096 * 2 ** (rng.random() * 17))        # log-uniform 4 KiB .. 512 MiB
                p = pool.alloc(n)
                if p == 0:
                    continue
                rounded = (ph.ph_round_large(n) if n >= 8 * MiB else ph.ph_small_class_size(n))
                assert p % (2 * MiB if n >= 8 * MiB else 512) == 0
                assert p not in live
                held = ph.ph_block_bytes(pool.h, p)
                assert rounded <= held <= rounded + rounded // 8      # exact, or a near fit handed out whole
                live[p] = held
            if step % 500 == 0:
                spans = sorted((p, p + n) for p, n in live.items())
                assert all(a[1] <= b[0] for a, b in zip(spans, spans[1:])), "live blocks overlap"
                st = pool.stats()
                assert st["bytes_live"] == sum(live.values())
                assert st["bytes_reserved"] == pool.L.ph_backing_used(pool.h)
                assert (st["bytes_live"] + st["bytes_cached_large"] + st["bytes_cached_small"]
                        + st["bytes_free_arena"] + st["bytes_free_slab_arena"]) <= st["bytes_reserved"]
        for p in list(live):
            assert pool.free(p) == 0
        st = pool.stats()
        assert st["bytes_live"] == 0
        pool.L.ph_release_unused(pool.h)
        assert pool.L.ph_backing_used(pool.h) == 0 and pool.stats()["bytes_reserved"] == 0
    finally:
        pool.close()


def test_concurrent_callers_keep_the_pool_consistent(ph):
    # PyTorch may call the allocator from several threads (the reference has no lock at all):
    # eight threads churn one pool; ctypes drops the GIL during each call.
    import threading
    pool = P(ph, capacity=32 * GiB, arena=1 * GiB)
    errors = []
    live_per_thread = [dict() for _ in range(8)]

    def worker(tid):
        rng = random.Random(100 + tid)
        live = live_per_thread[tid]
        try:
            for _ in range(3000):
                if live and rng.random() < 0.5:
                    p = rng.choice(list(live))
                    if pool.free(p, stream=tid) != 0:
                        errors.append("free failed")
                    del live[p]
                else:
                    n = int(4096 * 2 ** (rng.random() * 15))
                    p = pool.alloc(n, stream=tid)
                    if p == 0 or p in live:
                        errors.append("bad pointer")
                        continue
                    live[p] = ph.ph_block_bytes(pool.h, p)
        except Exception as e:  # pragma: no cover
            errors.append(repr(e))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    try:
        assert not errors, errors[:3]
        everything = {}
        for live in live_per_thread:
            for p, n in live.items():
                assert p not in everything, "one block handed to two threads"
                everything[p] = n
        spans = sorted((p, p + n) for p, n in everything.items())
        assert all(a[1] <= b[0] for a, b in zip(spans, spans[1:])), "live blocks overlap"
        st = pool.stats()
        assert st["bytes_live"] == sum(everything.values())
        assert st["bytes_reserved"] == pool.L.ph_backing_used(pool.h)
        for p in everything:
            assert pool.free(p) == 0
        pool.L.ph_release_unused(pool.h)
        assert pool.L.ph_backing_used(pool.h) == 0
    finally:
        pool.close()
