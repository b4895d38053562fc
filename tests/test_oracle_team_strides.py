"""The oracle's team forms (members pe_start + k * pe_stride, any stride) against brute force in
numpy and against the active-set forms where the stride is a power of two."""
import numpy as np
import pytest

import oracle

N_PES, STRIDE_BYTES = 8, 4096


def filled_heap(seed):
    heap = oracle.Heap(N_PES, STRIDE_BYTES)
    rng = np.random.default_rng(seed)
    for p in range(N_PES):
        heap.view(p, 0, STRIDE_BYTES, np.uint8)[:] = rng.integers(0, 256, STRIDE_BYTES, dtype=np.uint8)
    return heap


def snapshot(heap):
    return [heap.view(p, 0, STRIDE_BYTES, np.uint8).copy() for p in range(N_PES)]


TEAMS = [(0, 3, 3), (1, 3, 3), (2, 5, 2), (0, 7, 2), (1, 2, 4), (3, 1, 4), (4, 3, 1)]


@pytest.mark.parametrize("pe_start,pe_stride,pe_size", TEAMS)
@pytest.mark.parametrize("op,fold", [(oracle.SUM, np.add), (oracle.XOR, np.bitwise_xor),
                                     (oracle.MAX, np.maximum), (oracle.PROD, np.multiply)])
def test_team_reduction_is_the_fold_over_the_members(pe_start, pe_stride, pe_size, op, fold):
    heap = filled_heap(pe_start * 10 + pe_stride)
    before = snapshot(heap)
    n, src_off, dst_off = 100, 16, 2048
    oracle.to_all(heap, oracle.LONG, op, dst_off, src_off, n, pe_start, pe_size=pe_size, pe_stride=pe_stride)
    members = [pe_start + k * pe_stride for k in range(pe_size)]
    want = before[members[0]][src_off:src_off + 8 * n].view(np.int64).copy()
    with np.errstate(over="ignore"):
        for m in members[1:]:
            want = fold(want, before[m][src_off:src_off + 8 * n].view(np.int64))
    for p in range(N_PES):
        after = heap.view(p, 0, STRIDE_BYTES, np.uint8)
        expect = before[p].copy()
        if p in members:
            expect[dst_off:dst_off + 8 * n] = want.view(np.uint8)
        assert np.array_equal(after, expect), "PE %d" % p


@pytest.mark.parametrize("pe_start,pe_stride,pe_size", TEAMS)
def test_team_broadcast_alltoall_fcollect_by_hand(pe_start, pe_stride, pe_size):
    members = [pe_start + k * pe_stride for k in range(pe_size)]
    block, src_off, dst_off = 24, 8, 2048
    # broadcast from the last member
    heap = filled_heap(1)
    before = snapshot(heap)
    oracle.broadcast(heap, dst_off, src_off, 100, pe_size - 1, pe_start, pe_size=pe_size, pe_stride=pe_stride)
    for p in range(N_PES):
        expect = before[p].copy()
        if p in members[:-1]:
            expect[dst_off:dst_off + 100] = before[members[-1]][src_off:src_off + 100]
        assert np.array_equal(heap.view(p, 0, STRIDE_BYTES, np.uint8), expect), "broadcast, PE %d" % p
    # alltoall: block j of member i's source lands in block i of member j's dest
    heap = filled_heap(2)
    before = snapshot(heap)
    oracle.alltoall(heap, dst_off, src_off, block, pe_start, pe_size=pe_size, pe_stride=pe_stride)
    for p in range(N_PES):
        expect = before[p].copy()
        if p in members:
            j = members.index(p)
            for i, q in enumerate(members):
                expect[dst_off + i * block:dst_off + (i + 1) * block] = \
                    before[q][src_off + j * block:src_off + (j + 1) * block]
        assert np.array_equal(heap.view(p, 0, STRIDE_BYTES, np.uint8), expect), "alltoall, PE %d" % p
    # fcollect: member i's block lands in block i of every member's dest
    heap = filled_heap(3)
    before = snapshot(heap)
    oracle.fcollect(heap, dst_off, src_off, block, pe_start, pe_size=pe_size, pe_stride=pe_stride)
    for p in range(N_PES):
        expect = before[p].copy()
        if p in members:
            for i, q in enumerate(members):
                expect[dst_off + i * block:dst_off + (i + 1) * block] = before[q][src_off:src_off + block]
        assert np.array_equal(heap.view(p, 0, STRIDE_BYTES, np.uint8), expect), "fcollect, PE %d" % p


@pytest.mark.parametrize("pe_start,log_stride,pe_size", [(0, 0, 8), (1, 1, 3), (0, 2, 2), (3, 0, 4)])
def test_team_forms_agree_with_the_active_set_forms(pe_start, log_stride, pe_size):
    calls = [
        lambda h, **kw: oracle.to_all(h, oracle.INT, oracle.SUM, 2048, 0, 200, pe_start, pe_size=pe_size, **kw),
        lambda h, **kw: oracle.broadcast(h, 2048, 4, 333, pe_size - 1, pe_start, pe_size=pe_size, **kw),
        lambda h, **kw: oracle.alltoall(h, 2048, 0, 40, pe_start, pe_size=pe_size, **kw),
        lambda h, **kw: oracle.fcollect(h, 2048, 0, 40, pe_start, pe_size=pe_size, **kw),
    ]
    for k, call in enumerate(calls):
        a, b = filled_heap(50 + k), filled_heap(50 + k)
        call(a, log_stride=log_stride)
        call(b, pe_stride=1 << log_stride)
        assert all(np.array_equal(x, y) for x, y in zip(snapshot(a), snapshot(b))), k
