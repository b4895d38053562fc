"""Pins the oracle's data-movement and AMO models with the patterns the reference's tests use."""
import numpy as np

import oracle


def test_put_get_fill_patterns():
    # clients/functional_tests/primitive_tester.cpp:97-129: sender filled '0', receiver '1',
    # after the put the receiver reads '0' over the message and '1' beyond it
    h = oracle.Heap(2, 4096)
    h.view(0, 0, 1024, np.uint8)[:] = ord("0")
    h.view(1, 2048, 1024, np.uint8)[:] = ord("1")
    oracle.put(h, 2048, 0, 512, 0, 1)
    r = h.view(1, 2048, 1024, np.uint8)
    assert (r[:512] == ord("0")).all() and (r[512:] == ord("1")).all()
    # clients/sos_tests/bigput.cpp:202-263: Source[i] = i + 1 arrives unchanged; get is the mirror image
    src = np.arange(1, 257, dtype=np.int32)
    h = oracle.Heap(3, 4096)
    h.view(2, 0, 256, np.int32)[:] = src
    oracle.put(h, 1024, 0, 1024, 2, 0)
    assert np.array_equal(h.view(0, 1024, 256, np.int32), src)
    oracle.get(h, 2048, 0, 1024, 1, 2)
    assert np.array_equal(h.view(1, 2048, 256, np.int32), src)
    before = h.buf.copy()
    oracle.put(h, 0, 0, 0, 0, 1)                        # zero length: nothing moves
    assert np.array_equal(before, h.buf)


def test_broadcast_leaves_the_root_dest_alone():
    # clients/functional_tests/tester.cpp:236-271 (source 1, dest 2) and
    # clients/sos_tests/broadcast_active_set.cpp:84-128 (shrinking set, changing root)
    npes, n = 6, 16
    h = oracle.Heap(npes, 1024)
    for p in range(npes):
        h.view(p, 0, n, np.int64)[:] = 1
        h.view(p, 512, n, np.int64)[:] = 2
    oracle.broadcast(h, 512, 0, n * 8, 0)
    assert (h.view(0, 512, n, np.int64) == 2).all()
    for p in range(1, npes):
        assert (h.view(p, 512, n, np.int64) == 1).all()
    h = oracle.Heap(npes, 1024)
    for p in range(npes):
        h.view(p, 0, n, np.int64)[:] = p
        h.view(p, 512, n, np.int64)[:] = -1
    for i in range(npes):          # active set i..npes-1, root = its first member
        oracle.broadcast(h, 512, 0, n * 8, 0, pe_start=i, log_stride=0, pe_size=npes - i)
        for me in range(npes):
            if me < i:
                continue
            expected = i - 1 if me == i else i
            assert (h.view(me, 512, n, np.int64) == expected).all(), (i, me)


def test_alltoall_and_fcollect_patterns():
    # clients/functional_tests/tester.cpp:310-334: (src_pe << 16) + dst_pe; :336-355: value = source rank
    npes, n = 4, 8
    h = oracle.Heap(npes, 4096)
    for i in range(npes):
        h.view(i, 0, n * npes, np.int64)[:] = np.repeat([(i << 16) + j for j in range(npes)], n)
    oracle.alltoall(h, 2048, 0, n * 8)
    for j in range(npes):
        assert np.array_equal(h.view(j, 2048, n * npes, np.int64),
                              np.repeat([(i << 16) + j for i in range(npes)], n))
    h = oracle.Heap(npes, 4096)
    for i in range(npes):
        h.view(i, 0, n, np.int64)[:] = i
    oracle.fcollect(h, 2048, 0, n * 8)
    for j in range(npes):
        assert np.array_equal(h.view(j, 2048, n * npes, np.int64), np.repeat(np.arange(npes), n))
    # a strided sub-team leaves everybody else untouched
    h = oracle.Heap(6, 4096, fill=0xEE)
    for i in (0, 2, 4):
        h.view(i, 0, 3, np.int32)[:] = 100 + i
    oracle.fcollect(h, 1024, 0, 12, pe_start=0, log_stride=1, pe_size=3)
    for p in range(6):
        got = h.view(p, 1024, 9, np.int32)
        if p % 2 == 0:
            assert np.array_equal(got, np.repeat([100, 102, 104], 3))
        else:
            assert (got.view(np.uint8) == 0xEE).all()


def ops_array(rows):
    ops = np.zeros(len(rows), oracle.SMALL_OP_DTYPE)
    for i, r in enumerate(rows):
        ops[i] = r
    return ops


def test_amo_closed_forms():
    # clients/functional_tests/amo_standard_tester.cpp:76-117
    n = 50
    K = dict(P64=0, FADD=1, ADD=2, FINC=3, INC=4, CSWAP=5, FETCH=6, SET=7, SWAP=8, P32=9, FADD32=10)
    h = oracle.Heap(2, 256)
    ops = ops_array([(K["FADD"], 1, 0, 2, 0)] * n + [(K["FINC"], 1, 8, 0, 0)] * n +
                    [(K["ADD"], 1, 16, 2, 0)] * n + [(K["INC"], 1, 24, 0, 0)] * n)
    f = oracle.small_ops(h, ops, np.zeros(len(ops), np.uint32))
    w = h.view(1, 0, 4, np.int64)
    assert f[n - 1] == 2 * (n - 1) and w[0] == 2 * n          # fetch_add
    assert f[2 * n - 1] == n - 1 and w[1] == n                # fetch_inc: lfinc.cpp:90-111 returns j
    assert np.array_equal(f[n:2 * n], np.arange(n))
    assert w[2] == 2 * n and w[3] == n                        # add, inc
    assert not h.view(0, 0, 32, np.int64).any()               # neighbours untouched
    # cxx_test_shmem_atomic_add.cpp:85-144: every PE adds me+1 to every PE -> npes(npes+1)/2
    npes = 5
    h = oracle.Heap(npes, 64)
    rows, issuers = [], []
    for me in range(npes):
        for pe in range(npes):
            rows.append((K["ADD"], pe, 0, me + 1, 0))
            issuers.append(me)
    oracle.small_ops(h, ops_array(rows), np.array(issuers, np.uint32))
    for pe in range(npes):
        assert h.view(pe, 0, 1, np.int64)[0] == npes * (npes + 1) // 2
    # compare_swap stores only on a match and always returns the old value; swap/set/fetch
    h = oracle.Heap(1, 64)
    h.view(0, 0, 1, np.int64)[:] = 7
    f = oracle.small_ops(h, ops_array([(K["CSWAP"], 0, 0, 9, 3), (K["CSWAP"], 0, 0, 9, 7),
                                       (K["FETCH"], 0, 0, 0, 0), (K["SWAP"], 0, 0, -4, 0),
                                       (K["SET"], 0, 0, 11, 0), (K["FETCH"], 0, 0, 0, 0)]),
                         np.zeros(6, np.uint32))
    assert list(f[:4]) == [7, 7, 9, 9] and f[5] == 11
    # 32-bit operands leave the other half of the word alone
    h = oracle.Heap(1, 64)
    h.view(0, 0, 2, np.int32)[:] = [5, 6]
    f = oracle.small_ops(h, ops_array([(K["FADD32"], 0, 4, -10, 0), (K["P32"], 0, 0, 77, 0)]),
                         np.zeros(2, np.uint32))
    assert f[0] == 6 and list(h.view(0, 0, 2, np.int32)) == [77, -4]
    # 8-byte put, thread-level putmem/getmem of the issuing PE's own bytes
    h = oracle.Heap(2, 128)
    h.view(0, 64, 8, np.uint8)[:] = np.arange(8)
    oracle.small_ops(h, ops_array([(0, 1, 8, 0x1122334455667788, 0), (11, 1, 16, 64, 5)]),
                     np.zeros(2, np.uint32))
    assert h.view(1, 8, 1, np.int64)[0] == 0x1122334455667788
    assert list(h.view(1, 16, 8, np.uint8)) == [0, 1, 2, 3, 4, 0, 0, 0]
