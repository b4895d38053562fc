"""rsm_stream_probe: the write stream leaves the documented pattern in every PE's buffer and
nothing outside it; the read stream's checksum is the XOR of all 16-byte vectors it was
pointed at (so its loads are real)."""
import numpy as np
import pytest

import roc_shmem_amd as rs
from helpers import runtime

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("wgs,wg_size,accesses,nbytes", [(3, 256, 0, (3 << 20) + 80), (8, 1024, 0, 16), (2, 64, 0, (1 << 20) - 64),
                                                         (300, 256, 1, (1 << 20) + 4096 + 64), (5, 128, 2, (1 << 20) - 32),
                                                         (7, 512, 4, (2 << 20) + 16)])
def test_write_pattern_and_read_checksum(wgs, wg_size, accesses, nbytes):
    n_pes, seed, guard = 4, 0x5EED1234, 256
    launch = rs.Launch(wgs, wg_size, wg_size * 16 * accesses)
    with runtime(n_pes, heap_size=64 << 20, num_blocks=8):
        buf = rs.sym_array(nbytes + 2 * guard, np.uint8, fill=0xA5)
        chk = rs.sym_array(4, np.uint32, fill=0)
        rs.stream_probe(rs.STREAM_WRITE, buf.addr + guard, nbytes, None, seed, launch)
        rs.synchronize()
        nvec = nbytes // 16
        for p in range(n_pes):
            got = buf.read(p)
            assert (got[:guard] == 0xA5).all() and (got[guard + nbytes:] == 0xA5).all(), p
            vec = got[guard:guard + nbytes].view(np.uint32).reshape(nvec, 4)
            i = np.arange(nvec, dtype=np.uint64)
            bad = np.nonzero(vec[:, 0] != (i & np.uint64(0xFFFFFFFF)).astype(np.uint32))[0]
            assert bad.size == 0, (p, bad.size, bad[:8], vec[bad[:4]])
            assert np.array_equal(vec[:, 1], (i >> np.uint64(32)).astype(np.uint32))
            assert (vec[:, 2] == p).all() and (vec[:, 3] == seed).all()
        # other contents for the read: seeded bytes, different in every PE
        rng = np.random.default_rng(5)
        payload = [rng.integers(0, 256, nbytes + 2 * guard, dtype=np.uint8) for _ in range(n_pes)]
        for p in range(n_pes):
            buf.write(p, payload[p])
        rs.stream_probe(rs.STREAM_READ, buf.addr + guard, nbytes, chk, 0, launch)
        rs.synchronize()
        for p in range(n_pes):
            want = np.bitwise_xor.reduce(payload[p][guard:guard + nbytes].view(np.uint32).reshape(nvec, 4), axis=0)
            assert np.array_equal(chk.read(p), want), p
        # without a checksum the read changes nothing
        rs.stream_probe(rs.STREAM_READ, buf.addr + guard, nbytes, None, 0, launch)
        rs.synchronize()
        for p in range(n_pes):
            assert np.array_equal(buf.read(p), payload[p]), p
        # the copy: first half onto second half, nothing else
        if nbytes % 32 == 0:
            rs.stream_probe(rs.STREAM_COPY, buf.addr + guard, nbytes, None, 0, launch)
            rs.synchronize()
            half = nbytes // 2
            for p in range(n_pes):
                want = payload[p].copy()
                want[guard + half:guard + nbytes] = want[guard:guard + half]
                assert np.array_equal(buf.read(p), want), p
        assert rs.take_status() == 0
        chk.free()
        buf.free()


def test_runtime_fill_and_copy():
    """The two kinds that run the HIP runtime's own fill and copy over the same buffers."""
    n_pes, guard, nbytes = 4, 256, (1 << 20) + 64
    with runtime(n_pes, heap_size=64 << 20, num_blocks=8):
        buf = rs.sym_array(nbytes + 2 * guard, np.uint8, fill=0xA5)
        rs.stream_probe(rs.STREAM_RUNTIME_FILL, buf.addr + guard, nbytes, None, 0x1C3, rs.Launch(1, 64))
        rs.synchronize()
        for p in range(n_pes):
            got = buf.read(p)
            assert (got[:guard] == 0xA5).all() and (got[guard + nbytes:] == 0xA5).all(), p
            assert (got[guard:guard + nbytes] == 0xC3).all(), p
        rng = np.random.default_rng(6)
        payload = [rng.integers(0, 256, nbytes + 2 * guard, dtype=np.uint8) for _ in range(n_pes)]
        for p in range(n_pes):
            buf.write(p, payload[p])
        rs.stream_probe(rs.STREAM_RUNTIME_COPY, buf.addr + guard, nbytes, None, 0, rs.Launch(1, 64))
        rs.synchronize()
        half = nbytes // 2
        for p in range(n_pes):
            want = payload[p].copy()
            want[guard + half:guard + nbytes] = want[guard:guard + half]
            assert np.array_equal(buf.read(p), want), p
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
            rs.stream_probe(rs.STREAM_READ, buf, 4096, buf.addr + 8192, 0, rs.Launch(1, 64))  # checksum outside
        with pytest.raises(rs.RocShmemError):
            rs.stream_probe(rs.STREAM_WRITE, buf, 4096, None, 0, rs.Launch(1, 64, 3000))  # pass size not 1, 2, 4 or 8 accesses
        with pytest.raises(rs.RocShmemError):
            rs.stream_probe(rs.STREAM_COPY, buf, 4080, None, 0, rs.Launch(1, 64))         # halves of 16n+8 bytes
        with pytest.raises(rs.RocShmemError):
            rs.stream_probe(5, buf, 4096, chk, 0, rs.Launch(1, 64))                      # unknown kind
        with pytest.raises(rs.RocShmemError):
            rs.stream_probe(rs.STREAM_RUNTIME_COPY, buf, 4080, None, 0, rs.Launch(1, 64))  # halves of 16n+8 bytes
        chk.free()
        buf.free()
