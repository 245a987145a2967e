"""The pooled allocator's policy (the reference's CUDADeviceAllocator, code/source/base/alloc_cu.cpp:7-119)
driven through the C ABI with an injected backing allocator, so no GPU is involved."""
import ctypes

import pytest

from llminfer_amd import _binding as B

MiB = 1024 * 1024


class FakeBacking:
    """Hands out fake, increasing addresses and records every call."""

    def __init__(self, fail_after=None):
        self.next = 0x10000000
        self.live = {}
        self.allocs = []
        self.frees = []
        self.fail_after = fail_after

        def alloc(pp, nbytes, user):
            if self.fail_after is not None and len(self.allocs) >= self.fail_after:
                return -12
            addr = self.next
            self.next += (nbytes + 0xFFF) & ~0xFFF
            pp[0] = addr
            self.live[addr] = nbytes
            self.allocs.append(nbytes)
            return 0

        def free(p, user):
            self.frees.append(p)
            del self.live[p]
            return 0

        self.alloc_cb = B.BACKING_ALLOC_FN(alloc)
        self.free_cb = B.BACKING_FREE_FN(free)
        self.pool = B.lib().llmi_pool_create(self.alloc_cb, self.free_cb, None)
        assert self.pool

    def alloc(self, n):
        return B.lib().llmi_pool_alloc(self.pool, n)

    def free(self, p):
        return B.lib().llmi_pool_free(self.pool, p)

    def stats(self):
        s = B.PoolStats()
        assert B.lib().llmi_pool_get_stats(self.pool, ctypes.byref(s)) == 0
        return s

    def destroy(self):
        B.lib().llmi_pool_destroy(self.pool)
        self.pool = None


@pytest.fixture
def fb():
    f = FakeBacking()
    yield f
    if f.pool:
        f.destroy()


def test_zero_bytes_and_null(fb):
    assert fb.alloc(0) is None            # alloc_cu.cpp:8-10
    assert fb.free(None) == 0             # alloc_cu.cpp:82-84
    assert fb.allocs == []


def test_reuse_returns_the_same_pointer(fb):
    p = fb.alloc(4)
    assert fb.free(p) == 0
    assert fb.alloc(4) == p               # the per-token id tensor pattern: alloc/free/alloc of 4 bytes
    assert len(fb.allocs) == 1 and fb.stats().reuses == 1 and fb.frees == []  # released blocks are kept


def test_class_boundary_is_strictly_above_one_mib(fb):
    small = fb.alloc(MiB)                 # exactly 1 MiB is still the small class (alloc_cu.cpp:21: '>')
    big = fb.alloc(MiB + 1)
    s = fb.stats()
    assert (s.small_busy_blocks, s.big_busy_blocks) == (1, 1)
    fb.free(small)
    fb.free(big)
    s = fb.stats()
    assert (s.small_free_blocks, s.big_free_blocks) == (1, 1)
    assert s.small_free_bytes == MiB and s.big_free_bytes == MiB + 1
    # a big request never takes the small block and vice versa
    assert fb.alloc(MiB + 1) == big
    assert fb.alloc(100) == small


def test_big_blocks_need_less_than_one_mib_of_slack(fb):
    p = fb.alloc(10 * MiB)
    fb.free(p)
    assert fb.alloc(9 * MiB) != p         # slack exactly 1 MiB: not "< 1 MiB" (alloc_cu.cpp:23-24) -> new block
    q = fb.alloc(9 * MiB + 1)             # slack 1 MiB - 1: reuse
    assert q == p
    assert len(fb.allocs) == 2


def test_best_fit_among_several_free_blocks(fb):
    sizes = [300, 100, 200, 1000]
    ptrs = {n: fb.alloc(n) for n in sizes}
    for p in ptrs.values():
        fb.free(p)
    assert fb.alloc(150) == ptrs[200]     # smallest block that fits (alloc_cu.cpp:52-61)
    assert fb.alloc(150) == ptrs[300]     # next smallest
    assert fb.alloc(50) == ptrs[100]
    assert fb.alloc(1) == ptrs[1000]      # small class: any slack is accepted
    assert len(fb.allocs) == 4
    big = {n: fb.alloc(n * MiB) for n in (8, 4, 6)}
    for p in big.values():
        fb.free(p)
    assert fb.alloc(4 * MiB - 5) == big[4]
    assert fb.alloc(6 * MiB - 5) == big[6]
    assert fb.alloc(2 * MiB) not in big.values()  # 8 MiB block is too loose a fit


def test_equal_sizes_are_distinct_blocks(fb):
    a, b = fb.alloc(64), fb.alloc(64)
    assert a != b
    fb.free(a)
    fb.free(b)
    assert {fb.alloc(64), fb.alloc(64)} == {a, b}


def test_unknown_and_double_free_are_rejected(fb):
    p = fb.alloc(128)
    assert fb.free(0xdead0000) == B.STATUS["UNKNOWN_POINTER"]   # the reference CHECK-fails (alloc_cu.cpp:86-87)
    assert fb.free(p) == 0
    assert fb.free(p) == B.STATUS["UNKNOWN_POINTER"]
    assert fb.stats().small_free_blocks == 1


def test_backing_failure_returns_null():
    f = FakeBacking(fail_after=1)
    assert f.alloc(10)
    assert f.alloc(20) is None            # alloc_cu.cpp:65-72
    assert f.alloc(2 * MiB) is None       # alloc_cu.cpp:35-42
    s = f.stats()
    assert s.backing_allocs == 1 and s.small_busy_blocks == 1 and s.big_busy_blocks == 0
    f.destroy()


def test_trim_and_destroy_hand_memory_back():
    f = FakeBacking()
    a, b, c = f.alloc(100), f.alloc(3 * MiB), f.alloc(200)
    f.free(a)
    f.free(b)
    assert B.lib().llmi_pool_trim(f.pool) == 100 + 3 * MiB
    assert sorted(f.frees) == sorted([a, b]) and f.stats().small_free_blocks == 0
    f.destroy()                           # the still-busy block goes back too
    assert c in f.frees and f.live == {}


def test_kv_cache_sized_requests_land_in_the_big_class(fb):
    kv = 36 * 4096 * 1024 * 2             # one Qwen3-4B K cache at 4K context
    p = fb.alloc(kv)
    s = fb.stats()
    assert s.big_busy_bytes == kv and s.small_busy_bytes == 0
    fb.free(p)
    assert fb.alloc(kv) == p


def test_create_rejects_missing_callbacks():
    assert B.lib().llmi_pool_create(B.BACKING_ALLOC_FN(0), B.BACKING_FREE_FN(0), None) is None
    assert B.lib().llmi_pool_alloc(None, 10) is None
    assert B.lib().llmi_pool_free(None, None) == B.STATUS["NULL_POINTER"]
