"""The largest PE counts: 128 members fill both halves of a 256-long pSync, the flag lanes of a
barrier span two waves (or loop, in a 64-lane workgroup), and alltoall walks 128 blocks."""
import numpy as np
import pytest

import oracle
import roc_shmem_amd as rs
import test_gpu_coll as coll
from helpers import runtime

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n_pes,wg_size", [(128, 64), (128, 256), (96, 128), (65, 1024)])
def test_collectives_among_many_pes(n_pes, wg_size):
    n = 3000
    with runtime(n_pes, heap_size=8 << 20, num_blocks=4):
        world = rs.roc_shmem_team_world()
        launch = rs.Launch(2, wg_size)
        psync = rs.sym_array(2 * rs.ROC_SHMEM_REDUCE_SYNC_SIZE, np.int64, fill=0)
        # reduction, active-set form over everybody
        src, dst, heap = coll.setup(n_pes, n * 8, n * 8 + 32, seed=n_pes)
        rs.roc_shmem_to_all(rs.LONG, rs.SUM, dst, src, n, 0, 0, n_pes, None, psync, launch)
        rs.synchronize()
        oracle.to_all(heap, oracle.LONG, oracle.SUM, n * 8, 0, n)
        coll.compare(n_pes, dst, heap, n * 8, n * 8 + 32)
        assert not any(psync.read(p).any() for p in range(n_pes)), "pSync not restored"
        # broadcast from the last PE, team form
        src2, dst2, heap2 = coll.setup(n_pes, 5000, 5000 + 32, seed=n_pes + 1)
        rs.roc_shmem_team_broadcast(1, world, dst2, src2, 5000, n_pes - 1, launch)
        rs.synchronize()
        oracle.broadcast(heap2, 5000, 0, 5000, n_pes - 1)
        coll.compare(n_pes, dst2, heap2, 5000, 5000 + 32)
        # alltoall and fcollect: n_pes blocks each
        block = 48
        src3, dst3, heap3 = coll.setup(n_pes, block * n_pes, block * n_pes + 32, seed=n_pes + 2)
        rs.roc_shmem_alltoall(4, world, dst3, src3, block // 4, launch)
        rs.synchronize()
        oracle.alltoall(heap3, block * n_pes, 0, block)
        coll.compare(n_pes, dst3, heap3, block * n_pes, block * n_pes + 32)
        src4, dst4, heap4 = coll.setup(n_pes, block, block * n_pes + 32, seed=n_pes + 3)
        rs.roc_shmem_fcollect(2, world, dst4, src4, block // 2, launch)
        rs.synchronize()
        oracle.fcollect(heap4, block, 0, block)
        coll.compare(n_pes, dst4, heap4, block, block * n_pes + 32)
        # barriers, several rounds and launches
        rs.roc_shmem_wg_barrier_all(20, launch)
        rs.roc_shmem_wg_barrier_all(3, rs.Launch(1, wg_size))
        rs.synchronize()
        assert rs.take_status() == 0
