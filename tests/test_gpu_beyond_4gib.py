"""Arrays of more than 4 GiB per PE: a put, a reduction and a broadcast whose byte offsets do not
fit 32 bits.  The arrays are filled on the device with one byte value per PE and seeded with random
windows at the places where 32-bit arithmetic would wrap (2^31 and 2^32 bytes), at both ends and at
a few other offsets; windows and a scatter of untouched words are checked against their closed forms."""
import numpy as np
import pytest

import roc_shmem_amd as rs
from helpers import runtime

pytestmark = pytest.mark.gpu

N_PES = 2
N = (5 << 30) // 4 + 12345            # int32 elements: 5 GiB and an odd tail
WINDOW = 4096                         # elements per seeded window
FILL = (0x11, 0x23)                   # byte each PE's source is filled with


def window_starts():
    marks = [0, (1 << 31) // 4 - WINDOW // 2, (1 << 32) // 4 - WINDOW // 2, (3 << 30) // 4 + 7, N - WINDOW]
    return [int(m) for m in marks]


def seed_source(src):
    """Returns {(pe, start): values} of what was written over the fill."""
    written = {}
    for p in range(N_PES):
        src.fill(FILL[p], pe=p)
        rng = np.random.default_rng(100 + p)
        for start in window_starts():
            vals = rng.integers(-(1 << 31), 1 << 31, WINDOW, dtype=np.int64).astype(np.int32)
            src.write(p, vals, elem_offset=start)
            written[(p, start)] = vals
    return written


def fill_word(p):
    return np.frombuffer(bytes([FILL[p]] * 4), np.int32)[0]


def expected(written, p, start, count):
    """Source of PE p at [start, start + count)."""
    out = np.full(count, fill_word(p), np.int32)
    for (q, s), vals in written.items():
        if q != p:
            continue
        lo, hi = max(s, start), min(s + WINDOW, start + count)
        if lo < hi:
            out[lo - start:hi - start] = vals[lo - s:hi - s]
    return out


def probes():
    rng = np.random.default_rng(7)
    spots = [int(x) for x in rng.integers(0, N - 64, 24)]
    return [(s, WINDOW) for s in window_starts()] + [(s, 64) for s in spots]


def test_put_reduce_broadcast_past_4_gib():
    with runtime(N_PES, heap_size=24 << 30, num_blocks=64):
        src = rs.sym_array(N, np.int32)
        dst = rs.sym_array(N, np.int32)
        written = seed_source(src)
        big = rs.Launch(64, 1024)
        # put: every PE p into PE p + 1, one message of 4 N bytes shared by the PE's workgroups
        for p in range(N_PES):
            dst.fill(0xEE, pe=p)
        rs.roc_shmem_rma(rs.PUT, rs.WG_SHARED, dst, src, 4 * N, 1, 4 * N, 4 * N, 1, big)
        rs.synchronize()
        for p in range(N_PES):
            for start, count in probes():
                got = dst.read(p, count, elem_offset=start)
                assert np.array_equal(got, expected(written, (p - 1) % N_PES, start, count)), \
                    "put: PE %d at element %d" % (p, start)
        # reduction: wrapping int32 sum over both PEs
        psync = rs.sym_array(64 * rs.ROC_SHMEM_REDUCE_SYNC_SIZE, np.int64, fill=0)
        for p in range(N_PES):
            dst.fill(0xEE, pe=p)
        rs.roc_shmem_to_all(rs.INT, rs.SUM, dst, src, N, 0, 0, N_PES, None, psync, big)
        rs.synchronize()
        for start, count in probes():
            with np.errstate(over="ignore"):
                want = expected(written, 0, start, count) + expected(written, 1, start, count)
            for p in range(N_PES):
                assert np.array_equal(dst.read(p, count, elem_offset=start), want), \
                    "sum_to_all: PE %d at element %d" % (p, start)
        # broadcast from PE 1: PE 0 receives, the root's dest keeps its fill
        for p in range(N_PES):
            dst.fill(0xEE, pe=p)
        rs.roc_shmem_team_broadcast(4, rs.roc_shmem_team_world(), dst, src, N, 1, big)
        rs.synchronize()
        untouched = np.frombuffer(bytes([0xEE] * 4), np.int32)[0]
        for start, count in probes():
            assert np.array_equal(dst.read(0, count, elem_offset=start), expected(written, 1, start, count)), \
                "broadcast: PE 0 at element %d" % start
            assert (dst.read(1, count, elem_offset=start) == untouched).all(), "broadcast: root's dest written"
        assert rs.take_status() == 0
        for a in (psync, dst, src):
            a.free()
