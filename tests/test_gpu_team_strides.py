"""Teams whose stride is not a power of two (roc_shmem_team_split_strided accepts any stride,
library/src/roc_shmem.cpp:236-250; clients/sos_tests/shmem_team_translate.cpp splits by 3):
reduction, broadcast, alltoall and fcollect over them, bit for bit against the oracle's team forms."""
import numpy as np
import pytest

import oracle
import roc_shmem_amd as rs
import test_gpu_coll as coll
from helpers import runtime

pytestmark = pytest.mark.gpu

N_PES = 8
TEAMS = [(0, 3, 3), (1, 3, 3), (2, 5, 2), (0, 7, 2), (1, 2, 4), (0, 6, 2)]


def split(pe_start, pe_stride, pe_size):
    rc, team = rs.roc_shmem_team_split_strided(rs.roc_shmem_team_world(), pe_start, pe_stride, pe_size)
    assert rc == 0 and team, "split (%d, %d, %d) refused" % (pe_start, pe_stride, pe_size)
    assert rs.roc_shmem_team_n_pes(team) == pe_size
    for k in range(pe_size):
        assert rs.roc_shmem_team_translate_pe(team, k, rs.roc_shmem_team_world()) == pe_start + k * pe_stride
    return team


@pytest.mark.parametrize("pe_start,pe_stride,pe_size", TEAMS)
@pytest.mark.parametrize("dtype,op,n,wgs,tile", [(rs.LONG, rs.SUM, 70001, 4, 0), (rs.INT, rs.XOR, 5000, 2, 1024),
                                                (rs.SHORT, rs.MAX, 333, 1, 0), (rs.LONGLONG, rs.PROD, 4099, 3, 0)])
def test_team_reduction(pe_start, pe_stride, pe_size, dtype, op, n, wgs, tile):
    npd = rs.NP_DTYPE[dtype]
    es = np.dtype(npd).itemsize
    with runtime(N_PES):
        team = split(pe_start, pe_stride, pe_size)
        src, dst, heap = coll.setup(N_PES, n * es, n * es + 64, seed=pe_start * 100 + pe_stride * 10 + op)
        rs.roc_shmem_team_to_all(dtype, op, team, dst, src, n, rs.Launch(wgs, 256, tile))
        rs.synchronize()
        oracle.to_all(heap, dtype, op, n * es, 0, n, pe_start, pe_size=pe_size, pe_stride=pe_stride)
        coll.compare(N_PES, dst, heap, n * es, n * es + 64)
        assert rs.take_status() == 0
        rs.roc_shmem_team_destroy(team)


@pytest.mark.parametrize("pe_start,pe_stride,pe_size", TEAMS)
def test_team_broadcast_alltoall_fcollect(pe_start, pe_stride, pe_size):
    nelem, elem = 6007, 4
    block = nelem * elem
    with runtime(N_PES):
        team = split(pe_start, pe_stride, pe_size)
        for root in sorted({0, pe_size - 1}):
            for launch in (rs.Launch(2, 256), rs.Launch(3, 128, 1000)):
                src, dst, heap = coll.setup(N_PES, block, block + 64, seed=root + 7)
                rs.roc_shmem_team_broadcast(elem, team, dst, src, nelem, root, launch)
                rs.synchronize()
                oracle.broadcast(heap, block, 0, block, root, pe_start, pe_size=pe_size, pe_stride=pe_stride)
                coll.compare(N_PES, dst, heap, block, block + 64)
                src.free()
                dst.free()
        src, dst, heap = coll.setup(N_PES, block * pe_size, block * pe_size + 64, seed=21)
        rs.roc_shmem_alltoall(elem, team, dst, src, nelem, rs.Launch(2, 256))
        rs.synchronize()
        oracle.alltoall(heap, block * pe_size, 0, block, pe_start, pe_size=pe_size, pe_stride=pe_stride)
        coll.compare(N_PES, dst, heap, block * pe_size, block * pe_size + 64)
        src.free()
        dst.free()
        src, dst, heap = coll.setup(N_PES, block, block * pe_size + 64, seed=22)
        rs.roc_shmem_fcollect(elem, team, dst, src, nelem, rs.Launch(3, 512))
        rs.synchronize()
        oracle.fcollect(heap, block, 0, block, pe_start, pe_size=pe_size, pe_stride=pe_stride)
        coll.compare(N_PES, dst, heap, block, block * pe_size + 64)
        assert rs.take_status() == 0
        rs.roc_shmem_team_destroy(team)


def test_split_of_a_strided_team_multiplies_the_strides():
    with runtime(N_PES):
        threes = split(0, 3, 3)                       # world PEs 0, 3, 6
        rc, outer = rs.roc_shmem_team_split_strided(threes, 0, 2, 2)   # members 0 and 2 of it: PEs 0, 6
        assert rc == 0 and outer
        world = rs.roc_shmem_team_world()
        assert [rs.roc_shmem_team_translate_pe(outer, k, world) for k in range(2)] == [0, 6]
        assert rs.roc_shmem_team_translate_pe(outer, 1, threes) == 2
        assert rs.roc_shmem_team_translate_pe(threes, 1, outer) == -1
        n = 1000
        src, dst, heap = coll.setup(N_PES, n * 8, n * 8, seed=5)
        rs.roc_shmem_team_to_all(rs.LONG, rs.SUM, outer, dst, src, n, rs.Launch(2, 256))
        rs.synchronize()
        oracle.to_all(heap, oracle.LONG, oracle.SUM, n * 8, 0, n, 0, pe_size=2, pe_stride=6)
        coll.compare(N_PES, dst, heap, n * 8, n * 8)
        # a split that would reach past the last PE is refused
        rc, bad = rs.roc_shmem_team_split_strided(world, 2, 3, 3)
        assert rc != 0 and not bad
        rs.roc_shmem_team_destroy(outer)
        rs.roc_shmem_team_destroy(threes)
