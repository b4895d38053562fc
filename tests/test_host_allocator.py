"""The symmetric-heap allocator of the library against the reference's unit-test
expectations and the oracle's model of the same strategy."""
import ctypes as C

import numpy as np

import oracle
from roc_shmem_amd import _lib

NONE = C.c_size_t(-1).value


class HostAlloc:
    def __init__(self, heap):
        self.lib = _lib.load()
        self.h = self.lib.rsm_host_alloc_create(heap)

    def alloc(self, n):
        return self.lib.rsm_host_alloc_alloc(self.h, n)

    def free(self, off):
        return self.lib.rsm_host_alloc_free(self.h, off)

    def in_use(self):
        return self.lib.rsm_host_alloc_in_use(self.h)

    def close(self):
        self.lib.rsm_host_alloc_destroy(self.h)


def both(heap):
    return HostAlloc(heap), oracle.Allocator(heap)


def test_reference_unit_test_expectations():
    # clients/unit_tests/single_heap_gtest.cpp:26-142, pow2_bins_gtest.cpp:26-157
    for a in both(1 << 30):
        assert a.alloc(0) == NONE                      # alloc(0) yields nothing
        first = a.alloc(1)
        assert first == 0 and a.in_use() == 128        # 128-byte floor
        assert a.alloc(4097) % 8192 == 0 and a.in_use() == 128 + 8192
    for a in both(1 << 30):
        assert a.alloc(1 << 30) == 0                   # a fresh heap satisfies one heap-sized request
        assert a.alloc(1) == NONE                      # and is then exhausted
    for a in both(1 << 30):
        assert a.alloc(1 << 29) == 0
        assert a.alloc(1 << 29) == 1 << 29             # two half-heap objects fill the heap
        assert a.alloc(128) == NONE


def test_split_order_and_lifo_reuse():
    for a in both(1 << 20):
        offs = [a.alloc(100) for _ in range(5)]
        assert offs == [0, 128, 256, 384, 512]         # lower half first, ascending
        assert a.free(offs[1]) == 0 and a.free(offs[3]) == 0
        assert a.alloc(128) == 384                     # most recently freed block first
        assert a.alloc(128) == 128
        assert a.free(12345) != 0                      # not an outstanding allocation
        # freed blocks are never merged: two adjacent free 128-byte blocks cannot serve 256 bytes
        assert a.free(0) == 0 and a.free(128) == 0
        assert a.alloc(256) == 768


def test_random_sequences_agree_with_the_model():
    rng = np.random.default_rng(9)
    lib, model = both(1 << 24)
    live = []
    for step in range(4000):
        if live and rng.random() < 0.45:
            off = live.pop(int(rng.integers(0, len(live))))
            assert lib.free(off) == model.free(off) == 0
        else:
            n = int(rng.choice([1, 64, 128, 129, 1000, 4096, 70000, 1 << 20]))
            a, b = lib.alloc(n), model.alloc(n)
            assert a == b, "step %d" % step
            if a != NONE:
                live.append(a)
        assert lib.in_use() == model.in_use()
    lib.close()
