"""Parity of broadcast / alltoall / fcollect / barrier with the CPU oracle."""
import numpy as np
import pytest

import oracle
import roc_shmem_amd as rs
from helpers import runtime

pytestmark = pytest.mark.gpu

GUARD = 0x3C


def setup(n_pes, src_bytes, dst_bytes, seed):
    src = rs.sym_array(src_bytes, np.uint8)
    dst = rs.sym_array(dst_bytes, np.uint8)
    heap = oracle.Heap(n_pes, src_bytes + dst_bytes + 128)
    rng = np.random.default_rng(seed)
    for p in range(n_pes):
        payload = rng.integers(0, 256, size=src_bytes, dtype=np.uint8)
        src.write(p, payload)
        heap.view(p, 0, src_bytes, np.uint8)[:] = payload
        dst.fill(GUARD, pe=p)
        heap.view(p, src_bytes, dst_bytes, np.uint8)[:] = GUARD
    return src, dst, heap


def compare(n_pes, dst, heap, src_bytes, dst_bytes):
    for p in range(n_pes):
        got = dst.read(p)
        exp = heap.view(p, src_bytes, dst_bytes, np.uint8)
        assert np.array_equal(got, exp), "PE %d: first difference at byte %d" % (
            p, int(np.argmax(got != exp)))


@pytest.mark.parametrize("elem_size", [1, 2, 4, 8])
@pytest.mark.parametrize("root", [0, 3])
def test_broadcast_active_set_world(elem_size, root):
    n_pes, nelem = 8, 3001
    nbytes = nelem * elem_size
    with runtime(n_pes):
        src, dst, heap = setup(n_pes, nbytes, nbytes + 64, seed=elem_size * 10 + root)
        psync = rs.sym_array(256 * 2, np.int64, fill=0)
        rs.roc_shmem_broadcast(elem_size, dst, src, nelem, root, 0, 0, n_pes, psync, rs.Launch(2, 256))
        rs.synchronize()
        oracle.broadcast(heap, nbytes, 0, nbytes, root)
        compare(n_pes, dst, heap, nbytes, nbytes + 64)
        # root's dest untouched (clients/sos_tests/broadcast_active_set.cpp:84-96)
        assert (dst.read(root) == GUARD).all()
        for p in range(n_pes):
            assert not psync.read(p).any()


@pytest.mark.parametrize("pe_start,log_stride,pe_size,root", [(2, 0, 5, 0), (1, 1, 3, 2), (0, 2, 2, 1)])
def test_broadcast_shrinking_and_strided_sets(pe_start, log_stride, pe_size, root):
    # PE_root counts within the active set (clients/sos_tests/broadcast_active_set.cpp:84-96
    # passes root 0 with PE_start = i and expects world PE i to be the root)
    n_pes, nelem = 8, 1000
    with runtime(n_pes):
        src, dst, heap = setup(n_pes, nelem * 8, nelem * 8, seed=pe_start + 31)
        psync = rs.sym_array(256, np.int64, fill=0)
        rs.roc_shmem_broadcast(8, dst, src, nelem, root, pe_start, log_stride, pe_size, psync)
        rs.synchronize()
        oracle.broadcast(heap, nelem * 8, 0, nelem * 8, root, pe_start, log_stride, pe_size)
        compare(n_pes, dst, heap, nelem * 8, nelem * 8)


@pytest.mark.parametrize("wgs,wg_size,tile,shift", [(2, 256, 0, 4), (3, 128, 0, 0), (4, 512, 0, 4),
                                                    (2, 256, 100000, 4), (2, 256, 0, (4, 5))])
def test_broadcast_large_payload_shared_by_several_workgroups(wgs, wg_size, tile, shift):
    # tile 0: the PE's workgroups share one broadcast pass by pass, reading the source through a
    # buffer descriptor (arrays aligned alike modulo 4, here 4 bytes past a 16-byte boundary) or
    # with unaligned vector loads (arrays one byte apart); tile > 0: one standard call per tile.
    # 3 MiB + 13 bytes, bytes around the payload untouched.
    n_pes, nbytes = 4, (3 << 20) + 13
    s_shift, d_shift = shift if isinstance(shift, tuple) else (shift, shift)
    with runtime(n_pes):
        src, dst, heap = setup(n_pes, nbytes + 64, nbytes + 64, seed=77)
        psync = rs.sym_array(256 * wgs, np.int64, fill=0)
        rs.roc_shmem_broadcast(1, dst.addr + d_shift, src.addr + s_shift, nbytes, 2, 0, 0, n_pes, psync,
                               rs.Launch(wgs, wg_size, tile))
        rs.synchronize()
        oracle.broadcast(heap, nbytes + 64 + d_shift, s_shift, nbytes, 2)
        compare(n_pes, dst, heap, nbytes + 64, nbytes + 64)
        for p in range(n_pes):
            assert not psync.read(p).any()


def test_broadcast_reference_pattern_and_team_form():
    # clients/functional_tests/tester.cpp:236-271: source 1, dest 2, non-roots read 1, root keeps 2
    n_pes, nelem = 4, 512
    with runtime(n_pes):
        src = rs.sym_array(nelem, np.int64)
        dst = rs.sym_array(nelem, np.int64)
        for p in range(n_pes):
            src.write(p, np.full(nelem, 1, np.int64))
            dst.write(p, np.full(nelem, 2, np.int64))
        rs.roc_shmem_team_broadcast(8, rs.roc_shmem_team_world(), dst, src, nelem, 0)
        rs.synchronize()
        assert (dst.read(0) == 2).all()
        for p in range(1, n_pes):
            assert (dst.read(p) == 1).all()
        # team-relative root: team {1,3}, root ordinal 1 -> world PE 3
        rc, team = rs.roc_shmem_team_split_strided(rs.roc_shmem_team_world(), 1, 2, 2)
        assert rc == 0
        for p in range(n_pes):
            src.write(p, np.full(nelem, 10 + p, np.int64))
            dst.write(p, np.full(nelem, -1, np.int64))
        rs.roc_shmem_team_broadcast(8, team, dst, src, nelem, 1, rs.Launch(2, 128))
        rs.synchronize()
        assert (dst.read(1) == 13).all()
        for p in (0, 2, 3):
            assert (dst.read(p) == -1).all()
        rs.roc_shmem_team_destroy(team)


@pytest.mark.parametrize("elem_size,nelem", [(4, 1000), (8, 257), (1, 4099), (2, 64)])
@pytest.mark.parametrize("wgs", [1, 3])
def test_alltoall_and_fcollect(elem_size, nelem, wgs):
    n_pes = 8
    block = elem_size * nelem
    with runtime(n_pes):
        world = rs.roc_shmem_team_world()
        src, dst, heap = setup(n_pes, block * n_pes, block * n_pes + 32, seed=nelem)
        rs.roc_shmem_alltoall(elem_size, world, dst, src, nelem, rs.Launch(wgs, 256))
        rs.synchronize()
        oracle.alltoall(heap, block * n_pes, 0, block)
        compare(n_pes, dst, heap, block * n_pes, block * n_pes + 32)
        src.free()
        dst.free()
        src, dst, heap = setup(n_pes, block, block * n_pes + 32, seed=nelem + 1)
        rs.roc_shmem_fcollect(elem_size, world, dst, src, nelem, rs.Launch(wgs, 256))
        rs.synchronize()
        oracle.fcollect(heap, block, 0, block)
        compare(n_pes, dst, heap, block, block * n_pes + 32)


@pytest.mark.parametrize("elem_size,nelem,wgs,wg_size", [(4, 30011, 3, 128), (8, 16384, 4, 128),
                                                         (1, 200003, 2, 256)])
def test_alltoall_and_fcollect_large_blocks_shared_by_several_workgroups(elem_size, nelem, wgs, wg_size):
    # large blocks cut into one range per workgroup, with block sizes that leave sources and
    # destinations misaligned against each other in some blocks and aligned in others
    n_pes = 4
    block = elem_size * nelem
    with runtime(n_pes):
        world = rs.roc_shmem_team_world()
        src, dst, heap = setup(n_pes, block * n_pes, block * n_pes + 32, seed=nelem)
        rs.roc_shmem_alltoall(elem_size, world, dst, src, nelem, rs.Launch(wgs, wg_size))
        rs.synchronize()
        oracle.alltoall(heap, block * n_pes, 0, block)
        compare(n_pes, dst, heap, block * n_pes, block * n_pes + 32)
        src.free()
        dst.free()
        src, dst, heap = setup(n_pes, block, block * n_pes + 32, seed=nelem + 1)
        rs.roc_shmem_fcollect(elem_size, world, dst, src, nelem, rs.Launch(wgs, wg_size))
        rs.synchronize()
        oracle.fcollect(heap, block, 0, block)
        compare(n_pes, dst, heap, block, block * n_pes + 32)


def test_alltoall_reference_pattern_on_a_sub_team():
    # clients/functional_tests/tester.cpp:310-334: value (src_pe << 16) + dst_pe, int64
    n_pes, nelem = 8, 100
    with runtime(n_pes):
        rc, team = rs.roc_shmem_team_split_strided(rs.roc_shmem_team_world(), 0, 2, 4)
        assert rc == 0
        members = [0, 2, 4, 6]
        src = rs.sym_array(nelem * 4, np.int64)
        dst = rs.sym_array(nelem * 4, np.int64, fill=0xFF)
        for i, p in enumerate(members):
            vals = np.repeat(np.array([(i << 16) + j for j in range(4)], np.int64), nelem)
            src.write(p, vals)
        rs.roc_shmem_alltoall(8, team, dst, src, nelem, rs.Launch(2, 128))
        rs.synchronize()
        for j, p in enumerate(members):
            exp = np.repeat(np.array([(i << 16) + j for i in range(4)], np.int64), nelem)
            assert np.array_equal(dst.read(p), exp)
        for p in (1, 3, 5, 7):
            assert (dst.read(p).view(np.uint8) == 0xFF).all()
        rs.roc_shmem_team_destroy(team)


def test_fcollect_reference_pattern():
    # clients/functional_tests/tester.cpp:336-355 (FcollectTester<int64_t>): source = own rank,
    # dest = -1; afterwards block i of every PE's dest holds i.
    n_pes, nelem = 8, 333
    with runtime(n_pes):
        world = rs.roc_shmem_team_world()
        src = rs.sym_array(nelem, np.int64)
        dst = rs.sym_array(nelem * n_pes, np.int64)
        for p in range(n_pes):
            src.write(p, np.full(nelem, p, np.int64))
            dst.write(p, np.full(nelem * n_pes, -1, np.int64))
        rs.roc_shmem_fcollect(8, world, dst, src, nelem, rs.Launch(2, 256))
        rs.synchronize()
        exp = np.repeat(np.arange(n_pes, dtype=np.int64), nelem)
        for p in range(n_pes):
            assert np.array_equal(dst.read(p), exp), "PE %d" % p


def test_barrier_all_many_rounds():
    with runtime(8, num_blocks=8):
        rs.roc_shmem_wg_barrier_all(200, rs.Launch(4, 64))
        rs.synchronize()
        assert rs.take_status() == 0


def test_barriers_keep_count_across_launches_of_different_shapes():
    # sync_all / barrier_all count their calls per context block in the team's barrier pool and
    # never reset a slot: launches with other numbers of workgroups and rounds, with collectives on
    # the world team and on a sub-team in between, must leave every block's count in step on all PEs
    # (a count out of step ends in a wait that gives up and raises the status word).
    import time
    n_pes = 8
    with runtime(n_pes, num_blocks=16):
        world = rs.roc_shmem_team_world()
        rc, evens = rs.roc_shmem_team_split_strided(world, 0, 2, 4)
        assert rc == 0
        src, dst, heap = setup(n_pes, 4096, 4096, seed=3)
        t0 = time.perf_counter()
        for rounds, wgs, wg_size in ((3, 1, 64), (2, 3, 256), (5, 2, 1024), (1, 16, 64), (4, 1, 512), (7, 16, 128)):
            rs.roc_shmem_wg_barrier_all(rounds, rs.Launch(wgs, wg_size))
            rs.roc_shmem_team_broadcast(1, evens, dst, src, 4096, 1, rs.Launch(2, 128))
            rs.roc_shmem_team_to_all(rs.INT, rs.SUM, world, dst, src, 1024, rs.Launch(wgs, wg_size))
        rs.synchronize()
        assert rs.take_status() == 0
        assert time.perf_counter() - t0 < 1.0, "a barrier waited for its time limit"
        rs.roc_shmem_team_destroy(evens)
        # a new team gets a cleared pool, wherever the allocator puts it
        rc, again = rs.roc_shmem_team_split_strided(world, 1, 2, 4)
        assert rc == 0
        rs.roc_shmem_team_broadcast(1, again, dst, src, 4096, 0, rs.Launch(1, 64))
        rs.synchronize()
        assert rs.take_status() == 0
        rs.roc_shmem_team_destroy(again)


def test_barrier_pool_is_put_back_in_order_after_a_wait_that_gave_up():
    # sync_all / barrier_all keep a count of calls per context block in the team's barrier pool.
    # If a wait gives up, the counts of the members that got through and of those that did not
    # differ from then on.  The condition is forced from the host: PE 1's count for block 0 is
    # set ahead of everybody else's, so PE 1 announces a call number the others never reach and
    # its wait gives up after the (tiny) limit; every kernel exits normally.  Reading the status
    # word must report the timeout once and zero the pools, after which barriers work again.
    import os
    import time
    os.environ["ROC_SHMEM_WAIT_LIMIT_S"] = "0.02"
    try:
        rs.roc_shmem_init(4, 4 << 20, 2, 64)
    finally:
        del os.environ["ROC_SHMEM_WAIT_LIMIT_S"]
    try:
        rs.roc_shmem_wg_barrier_all(3, rs.Launch(2, 64))
        rs.synchronize()
        assert rs.take_status() == 0
        # device Team object: TeamInfo (4 ints), valid, pad, then the barrier pool's heap offset
        team = rs.read_device(rs.roc_shmem_team_world(), 32)
        pool_off = int(np.frombuffer(team, dtype=np.uint64)[3])
        epoch_slot = 255                                     # last long of a 256-long slice
        count_at = rs.heap_base(1) + pool_off + epoch_slot * 8
        assert int(np.frombuffer(rs.read_device(count_at, 8), dtype=np.uint64)[0]) == 3
        rs.write_device(count_at, np.array([10], dtype=np.uint64))
        rs.roc_shmem_wg_barrier_all(1, rs.Launch(1, 64))
        rs.synchronize()
        assert rs.take_status() == 1, "the skewed barrier must time out and say so"
        assert int(np.frombuffer(rs.read_device(count_at, 8), dtype=np.uint64)[0]) == 0, \
            "reading a raised status word zeroes the barrier pools"
        t0 = time.perf_counter()
        rs.roc_shmem_wg_barrier_all(5, rs.Launch(2, 64))
        rs.synchronize()
        assert rs.take_status() == 0
        assert time.perf_counter() - t0 < 0.5, "a barrier waited for its time limit after the reset"
    finally:
        rs.roc_shmem_finalize()
