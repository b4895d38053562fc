"""Arguments that would send a kernel past the end of a symmetric allocation are refused on the host
(entry points return an error, nothing is launched) or skipped on the device with the status word
raised (operations of a small-op stream, whose targets live in device memory)."""
import numpy as np
import pytest

import roc_shmem_amd as rs
from helpers import runtime

pytestmark = pytest.mark.gpu

HEAP = 8 << 20


def test_collectives_and_rma_beyond_the_heap_are_refused():
    n_pes = 4
    rs.roc_shmem_init(n_pes, HEAP, 8, 1024)
    try:
        world = rs.roc_shmem_team_world()
        a = rs.sym_array(1 << 18, np.int64, fill=1)          # 2 MiB each
        b = rs.sym_array(1 << 18, np.int64, fill=2)
        psync = rs.sym_array(256, np.int64, fill=0)
        too_many = HEAP // 8                                   # as many elements as the whole heap holds
        with pytest.raises(rs.RocShmemError, match="do not fit the symmetric allocation"):
            rs.roc_shmem_to_all(rs.LONG, rs.SUM, b, a, too_many, 0, 0, n_pes, None, psync)
        with pytest.raises(rs.RocShmemError, match="do not fit the symmetric allocation"):
            rs.roc_shmem_team_to_all(rs.LONG, rs.SUM, world, b, a, too_many)
        with pytest.raises(rs.RocShmemError, match="pSync"):   # 2 workgroups per PE need 2 pSync slices
            rs.roc_shmem_to_all(rs.LONG, rs.SUM, b, a, 16, 0, 0, n_pes, None, psync, rs.Launch(2, 64))
        with pytest.raises(rs.RocShmemError, match="do not fit the symmetric allocation"):
            rs.roc_shmem_broadcast(8, b, a, too_many, 0, 0, 0, n_pes, psync)
        with pytest.raises(rs.RocShmemError, match="do not fit the symmetric allocation"):
            rs.roc_shmem_alltoall(8, world, b, a, 1 << 17)     # 4 blocks of 1 MiB do not fit b's 2 MiB
        with pytest.raises(rs.RocShmemError, match="do not fit the symmetric allocation"):
            rs.roc_shmem_fcollect(8, world, b, a, too_many // 2)
        with pytest.raises(rs.RocShmemError, match="do not fit the symmetric allocation"):
            rs.roc_shmem_rma(rs.PUT, rs.WG, b, a, 1 << 20, 64)  # 64 messages of 1 MiB
        with pytest.raises(rs.RocShmemError, match="do not fit the symmetric allocation"):
            rs.roc_shmem_rma(rs.GET, rs.THREAD, b, a, HEAP, 1)
        rs.synchronize()
        # nothing ran: the operands are as they were, the status word is clear
        for p in range(n_pes):
            assert (a.read(p).view(np.uint8) == 1).all() and (b.read(p).view(np.uint8) == 2).all()
            assert not psync.read(p).any()
        assert rs.take_status() == 0
        # an address inside the heap that no allocation covers
        b_addr = b.addr
        b.free()
        with pytest.raises(rs.RocShmemError, match="not inside a live symmetric allocation"):
            rs.roc_shmem_to_all(rs.LONG, rs.SUM, b_addr, a, 16, 0, 0, n_pes, None, psync)
    finally:
        rs.roc_shmem_finalize()


def test_small_operations_outside_the_heap_are_skipped_and_reported():
    n_pes = 4
    rs.roc_shmem_init(n_pes, HEAP, 8, 1024)
    try:
        word = rs.sym_array(16, np.int64, fill=0)
        ops = np.zeros(6, dtype=rs.SMALL_OP_DTYPE)
        ops["kind"] = [rs.OP_P64, rs.OP_FADD64, rs.OP_P64, rs.OP_FADD64, rs.OP_PUTMEM, rs.OP_P64]
        ops["pe"] = [1, 1, n_pes, 2, 1, 3]                     # op 2: a PE that does not exist
        ops["offset"] = [word.offset, word.offset + 8, word.offset, HEAP - 4, word.offset, word.offset + 16]
        ops["value"] = [7, 5, 9, 1, word.offset + 64, 11]      # op 3: the last 4 bytes of the heap
        ops["aux"] = [0, 0, 0, 0, HEAP, 0]                     # op 4: a putmem as long as the heap
        dev = rs.device_array(ops)
        fetched = rs.device_array(np.full(6, -1, np.int64))
        rs.roc_shmem_small_ops(dev, 6, fetched, rs.Launch(1, 64))
        rs.synchronize()
        assert rs.take_status() == 2                           # bad argument, raised on the device
        assert rs.take_status() == 0                           # and cleared by reading it
        got1 = word.read(1)
        assert got1[0] == 7 and got1[1] == 5                   # the valid operations were carried out
        assert word.read(3)[2] == 11
        assert not word.read(0).any() and not word.read(2).any()
        dev.free()
        fetched.free()
    finally:
        rs.roc_shmem_finalize()
