"""Seeded random shapes: reductions, put/get, broadcast, alltoall and fcollect with random sizes,
alignments, active sets, launch shapes and tiles, each compared bit for bit with the CPU oracle
through the helpers of the other parity tests."""
import numpy as np
import pytest

import oracle
import roc_shmem_amd as rs
import test_gpu_coll as coll
import test_gpu_rma as rma
import test_gpu_to_all as to_all
from helpers import runtime

pytestmark = pytest.mark.gpu

N_PES = 8


class Draw:
    def __init__(self, seed):
        self.rng = np.random.default_rng(seed)

    def pick(self, options):
        return options[int(self.rng.integers(0, len(options)))]

    def between(self, lo, hi):
        return int(self.rng.integers(lo, hi))

    def size(self, *ranges):
        """One of several ranges, each as likely as the others, then a value inside it."""
        lo, hi = self.pick(list(ranges))
        return self.between(lo, hi)

    def active_set(self, strides=(0, 0, 1, 2)):
        log_stride = self.pick(list(strides))
        max_size = (N_PES - 1) // (1 << log_stride) + 1
        pe_size = self.between(1, max_size + 1)
        pe_start = self.between(0, N_PES - ((pe_size - 1) << log_stride))
        return pe_start, log_stride, pe_size


def reduction_case(d, case):
    dtype, op = d.pick(to_all.INT_TYPES), d.pick(to_all.INT_OPS)
    n = d.size((1, 300), (300, 20000), (20000, 300000))
    pe_start, log_stride, pe_size = d.active_set()
    wgs, wg_size = d.pick([1, 2, 3, 4]), d.pick([64, 128, 256, 512, 1024])
    tile = d.pick([0, 0, d.between(max(1, n // 100), max(2, n))])   # at most ~100 calls per workgroup
    shift, in_place = d.pick([0, 0, 1, 2, 3]), d.pick([False, False, True])
    what = "to_all dtype=%d op=%d n=%d set=(%d,%d,%d) wgs=%d wg=%d tile=%d shift=%d in_place=%s" % (
        dtype, op, n, pe_start, log_stride, pe_size, wgs, wg_size, tile, shift, in_place)
    got, expect, _ = to_all.run_case(dtype, op, N_PES, n, seed=case, pe_start=pe_start,
                                     log_stride=log_stride, pe_size=pe_size, wgs=wgs, wg_size=wg_size,
                                     tile=tile, in_place=in_place, elem_shift=shift)
    for p in range(N_PES):
        assert np.array_equal(got[p], expect[p]), "%s: PE %d differs, first at element %d" % (
            what, p, int(np.argmax(got[p] != expect[p])))
    return what


def rma_case(d, case):
    kind = d.pick([rs.PUT, rs.GET, rs.PUT_NBI, rs.GET_NBI])
    gran = d.pick([rs.WG, rs.WAVE, rs.THREAD, rs.WG_SHARED])
    msg = d.size((1, 64), (64, 5000), (5000, 300000))
    if gran == rs.THREAD:
        msg = min(msg, 3000)          # one lane moves the whole message
    n_msgs = 1 if gran == rs.WG_SHARED else d.pick([1, 2, 7])
    if gran == rs.WG_SHARED and kind in (rs.PUT_NBI, rs.GET_NBI):
        kind = rs.PUT
    src_mis, dst_mis = d.pick([0, 0, 1, 4, 7, 12]), d.pick([0, 0, 1, 4, 8, 13])
    wgs, wg_size = d.pick([1, 2, 4]), d.pick([64, 256, 512, 1024])
    pe_shift, pad = d.between(0, N_PES), d.pick([0, 0, 3, 64])
    what = "rma kind=%d gran=%d msg=%d n=%d mis=%d/%d wgs=%d wg=%d shift=%d pad=%d" % (
        kind, gran, msg, n_msgs, src_mis, dst_mis, wgs, wg_size, pe_shift, pad)
    try:
        rma.run_rma(kind, gran, N_PES, msg, n_msgs, seed=case, pe_shift=pe_shift, src_mis=src_mis,
                    dst_mis=dst_mis, wgs=wgs, wg_size=wg_size, stride_pad=pad)
    except AssertionError as e:
        raise AssertionError("%s: %s" % (what, e))
    return what


def broadcast_case(d, case):
    nbytes = d.size((1, 300), (300, 70000), (70000, 3 << 20))
    wgs, wg_size = d.pick([1, 2, 4]), d.pick([64, 256, 1024])
    s_shift = d.pick([0, 0, 4, 5])
    d_shift = d.pick([s_shift, s_shift, 0, 9])
    pe_start, log_stride, pe_size = d.active_set(strides=(0, 0, 1))
    root = d.between(0, pe_size)
    tile = d.pick([0, 0, d.between(max(1, nbytes // 100), nbytes + 1)])
    what = "broadcast n=%d wgs=%d wg=%d shifts=%d/%d set=(%d,%d,%d) root=%d tile=%d" % (
        nbytes, wgs, wg_size, s_shift, d_shift, pe_start, log_stride, pe_size, root, tile)
    src, dst, heap = coll.setup(N_PES, nbytes + 64, nbytes + 64, seed=case)
    psync = rs.sym_array(rs.ROC_SHMEM_BCAST_SYNC_SIZE * wgs, np.int64, fill=0)
    rs.roc_shmem_broadcast(1, dst.addr + d_shift, src.addr + s_shift, nbytes, root, pe_start, log_stride,
                           pe_size, psync, rs.Launch(wgs, wg_size, tile))
    rs.synchronize()
    oracle.broadcast(heap, nbytes + 64 + d_shift, s_shift, nbytes, root, pe_start, log_stride, pe_size)
    try:
        coll.compare(N_PES, dst, heap, nbytes + 64, nbytes + 64)
    except AssertionError as e:
        raise AssertionError("%s: %s" % (what, e))
    assert not any(psync.read(p).any() for p in range(N_PES)), what + ": pSync not restored"
    for a in (psync, dst, src):
        a.free()
    return what


def exchange_case(d, case):
    elem_size = d.pick([1, 2, 4, 8])
    nelem = d.size((1, 100), (100, 40000))
    wgs, wg_size = d.pick([1, 2, 3]), d.pick([64, 256, 1024])
    block = elem_size * nelem
    what = "alltoall/fcollect elem=%d nelem=%d wgs=%d wg=%d" % (elem_size, nelem, wgs, wg_size)
    world = rs.roc_shmem_team_world()
    try:
        src, dst, heap = coll.setup(N_PES, block * N_PES, block * N_PES + 32, seed=case)
        rs.roc_shmem_alltoall(elem_size, world, dst, src, nelem, rs.Launch(wgs, wg_size))
        rs.synchronize()
        oracle.alltoall(heap, block * N_PES, 0, block)
        coll.compare(N_PES, dst, heap, block * N_PES, block * N_PES + 32)
        src.free()
        dst.free()
        src, dst, heap = coll.setup(N_PES, block, block * N_PES + 32, seed=case + 1)
        rs.roc_shmem_fcollect(elem_size, world, dst, src, nelem, rs.Launch(wgs, wg_size))
        rs.synchronize()
        oracle.fcollect(heap, block, 0, block)
        coll.compare(N_PES, dst, heap, block, block * N_PES + 32)
        src.free()
        dst.free()
    except AssertionError as e:
        raise AssertionError("%s: %s" % (what, e))
    return what


def team_case(d, case):
    """One collective over a team of any stride (roc_shmem_team_split_strided takes any)."""
    pe_stride = d.between(1, 8)
    pe_size = d.between(1, (N_PES - 1) // pe_stride + 2)
    pe_start = d.between(0, N_PES - (pe_size - 1) * pe_stride)
    which = d.pick(["to_all", "broadcast", "alltoall", "fcollect"])
    wgs, wg_size = d.pick([1, 2, 4]), d.pick([64, 256, 1024])
    what = "team (%d,%d,%d) %s wgs=%d wg=%d" % (pe_start, pe_stride, pe_size, which, wgs, wg_size)
    rc, team = rs.roc_shmem_team_split_strided(rs.roc_shmem_team_world(), pe_start, pe_stride, pe_size)
    assert rc == 0 and team, what + ": split refused"
    kw = dict(pe_size=pe_size, pe_stride=pe_stride)
    try:
        if which == "to_all":
            dtype, op = d.pick(to_all.INT_TYPES), d.pick(to_all.INT_OPS)
            es = np.dtype(rs.NP_DTYPE[dtype]).itemsize
            n = d.size((1, 300), (300, 20000), (20000, 200000))
            tile = d.pick([0, 0, d.between(max(1, n // 100), max(2, n))])
            what += " dtype=%d op=%d n=%d tile=%d" % (dtype, op, n, tile)
            src, dst, heap = coll.setup(N_PES, n * es, n * es + 32, seed=case)
            rs.roc_shmem_team_to_all(dtype, op, team, dst, src, n, rs.Launch(wgs, wg_size, tile))
            rs.synchronize()
            oracle.to_all(heap, dtype, op, n * es, 0, n, pe_start, **kw)
            coll.compare(N_PES, dst, heap, n * es, n * es + 32)
        elif which == "broadcast":
            nbytes = d.size((1, 300), (300, 70000), (70000, 2 << 20))
            root = d.between(0, pe_size)
            what += " n=%d root=%d" % (nbytes, root)
            src, dst, heap = coll.setup(N_PES, nbytes, nbytes + 32, seed=case)
            rs.roc_shmem_team_broadcast(1, team, dst, src, nbytes, root, rs.Launch(wgs, wg_size))
            rs.synchronize()
            oracle.broadcast(heap, nbytes, 0, nbytes, root, pe_start, **kw)
            coll.compare(N_PES, dst, heap, nbytes, nbytes + 32)
        else:
            elem_size, nelem = d.pick([1, 2, 4, 8]), d.size((1, 100), (100, 30000))
            block = elem_size * nelem
            what += " elem=%d nelem=%d" % (elem_size, nelem)
            src_bytes = block * pe_size if which == "alltoall" else block
            src, dst, heap = coll.setup(N_PES, src_bytes, block * pe_size + 32, seed=case)
            call = rs.roc_shmem_alltoall if which == "alltoall" else rs.roc_shmem_fcollect
            call(elem_size, team, dst, src, nelem, rs.Launch(wgs, wg_size))
            rs.synchronize()
            getattr(oracle, which)(heap, src_bytes, 0, block, pe_start, **kw)
            coll.compare(N_PES, dst, heap, src_bytes, block * pe_size + 32)
    except AssertionError as e:
        raise AssertionError("%s: %s" % (what, e))
    src.free()
    dst.free()
    rs.roc_shmem_team_destroy(team)
    return what


@pytest.mark.parametrize("seed,ncases", [(101, 120), (202, 120)])
def test_random_shapes_match_the_oracle(seed, ncases):
    d = Draw(seed)
    makers = [reduction_case, reduction_case, rma_case, broadcast_case, exchange_case, team_case]
    # the allocator never merges freed blocks, so the library is brought up afresh every 30 cases
    for first in range(0, ncases, 30):
        with runtime(N_PES, heap_size=256 << 20):
            for case in range(first, min(ncases, first + 30)):
                what = d.pick(makers)(d, case)
                status = rs.take_status()
                assert status == 0, "%s: device status word %d" % (what, status)
