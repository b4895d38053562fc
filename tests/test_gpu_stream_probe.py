"""rsm_stream_probe: the write stream leaves the documented pattern in every PE's buffer and
nothing outside it; the read stream's checksum is the XOR of all 16-byte vectors it was
pointed at (so its loads are real)."""
import numpy as np
import pytest

import roc_shmem_amd as rs
from helpers import runtime

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("wgs,wg_size,nbytes", [(3, 256, (3 << 20) + 80), (8, 1024, 16), (2, 64, (1 << 20) - 16)])
def test_write_pattern_and_read_checksum(wgs, wg_size, nbytes):
    n_pes, seed, guard = 4, 0x5EED1234, 256
    with runtime(n_pes, heap_size=64 << 20, num_blocks=8):
        buf = rs.sym_array(nbytes + 2 * guard, np.uint8, fill=0xA5)
        chk = rs.sym_array(4, np.uint32, fill=0)
        rs.stream_probe(rs.STREAM_WRITE, buf.addr + guard, nbytes, None, seed, rs.Launch(wgs, wg_size))
        rs.synchronize()
        nvec = nbytes // 16
        for p in range(n_pes):
            got = buf.read(p)
            assert (got[:guard] == 0xA5).all() and (got[guard + nbytes:] == 0xA5).all(), p
            vec = got[guard:guard + nbytes].view(np.uint32).reshape(nvec, 4)
            i = np.arange(nvec, dtype=np.uint64)
            assert np.array_equal(vec[:, 0], (i & np.uint64(0xFFFFFFFF)).astype(np.uint32))
            assert np.array_equal(vec[:, 1], (i >> np.uint64(32)).astype(np.uint32))
            assert (vec[:, 2] == p).all() and (vec[:, 3] == seed).all()
        # other contents for the read: seeded bytes, different in every PE
        rng = np.random.default_rng(5)
        payload = [rng.integers(0, 256, nbytes + 2 * guard, dtype=np.uint8) for _ in range(n_pes)]
        for p in range(n_pes):
            buf.write(p, payload[p])
        rs.stream_probe(rs.STREAM_READ, buf.addr + guard, nbytes, chk, 0, rs.Launch(wgs, wg_size))
        rs.synchronize()
        for p in range(n_pes):
            want = np.bitwise_xor.reduce(payload[p][guard:guard + nbytes].view(np.uint32).reshape(nvec, 4), axis=0)
            assert np.array_equal(chk.read(p), want), p
        chk.free()
        buf.free()


def test_refused_arguments():
    with runtime(2, heap_size=16 << 20, num_blocks=4):
        buf = rs.sym_array(4096, np.uint8)
        chk = rs.sym_array(4, np.uint32, fill=0)
        with pytest.raises(rs.RocShmemError):
            rs.stream_probe(rs.STREAM_WRITE, buf, 4090, None, 0, rs.Launch(1, 64))       # not a multiple of 16
        with pytest.raises(rs.RocShmemError):
            rs.stream_probe(rs.STREAM_WRITE, buf, 8192, None, 0, rs.Launch(1, 64))       # past the allocation
        with pytest.raises(rs.RocShmemError):
            rs.stream_probe(rs.STREAM_READ, buf, 4096, None, 0, rs.Launch(1, 64))        # no checksum
        with pytest.raises(rs.RocShmemError):
            rs.stream_probe(2, buf, 4096, chk, 0, rs.Launch(1, 64))                      # unknown kind
        chk.free()
        buf.free()
