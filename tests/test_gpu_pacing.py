"""Lockstep pacing of large sharded reductions and transfers changes when workgroups issue
their loads and stores, never what they compute: results with pacing on are bit-identical to
the oracle's, whatever the rate (too low and too high rates only cost time).  The library
paces a call only when its grid fills the chip (at least one workgroup per compute unit, all
of them resident) and every workgroup has two passes or more, so the cases below are that large:
256 workgroups of 512 lanes, 32 MiB and more per PE."""
import numpy as np
import pytest

import oracle
import roc_shmem_amd as rs
from helpers import random_values, runtime

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("rate,mib", [(40000, 80), (64000, 32), (90000, 80)])
def test_paced_reduction_matches_the_oracle(rate, mib):
    n_pes, wgs, wg_size = 8, 32, 512        # 256 workgroups, 64 KiB per member per pass
    with runtime(n_pes, heap_size=512 << 20, num_blocks=32):   # power-of-two blocks: 2 x 128 MiB
        for dtype, op in ((rs.FLOAT, rs.SUM), (rs.LONG, rs.XOR), (rs.BF16, rs.MAX)):
            npd = rs.NP_DTYPE[dtype]
            es = np.dtype(npd).itemsize
            n = (mib << 20) // es + 77         # five (two) passes per workgroup and a ragged end
            src = rs.sym_array(n, npd)
            dst = rs.sym_array(n, npd, fill=0x5A)
            psync = rs.sym_array(wgs * rs.ROC_SHMEM_REDUCE_SYNC_SIZE, np.int64, fill=0)
            heap = oracle.Heap(n_pes, 2 * n * es)
            for p in range(n_pes):
                vals = random_values(dtype, n, 50 + p)
                src.write(p, vals)
                heap.view(p, 0, n, npd)[:] = vals
            rs.set_pacing(0, rate)
            assert rs.get_pacing() == (0, rate)
            rs.roc_shmem_to_all(dtype, op, dst, src, n, 0, 0, n_pes, None, psync, rs.Launch(wgs, wg_size))
            rs.synchronize()
            rs.set_pacing(0, 0)
            oracle.to_all_rounded_once(heap, dtype, op, n * es, 0, n)
            for p in range(n_pes):
                assert np.array_equal(dst.read(p), heap.view(p, n * es, n, npd)), (dtype, op, p)
            for a in (psync, dst, src):
                a.free()


@pytest.mark.parametrize("n_pes,wgs,wg_size,mib", [(16, 16, 1024, 80), (4, 64, 512, 40), (2, 128, 1024, 72),
                                                   (8, 48, 640, 60), (8, 32, 768, 60)])
def test_paced_reduction_with_other_numbers_of_pes(n_pes, wgs, wg_size, mib):
    """256 workgroups in all, two to five passes each, a ragged end, the library's default rate:
    2, 4 and 16 members (with 2 and 4 PEs the workgroups of a PE are spread over several XCDs).
    Also workgroups of 640 and 768 lanes, whose passes are no power of two: 384 of 640 lanes are
    not all resident (one per compute unit) and run free, 256 of 768 lanes follow the schedule."""
    with runtime(n_pes, heap_size=512 << 20, num_blocks=wgs):   # two power-of-two blocks of 128 MiB
        n = (mib << 20) // 4 + 41
        src = rs.sym_array(n, np.float32)
        dst = rs.sym_array(n, np.float32, fill=0x5A)
        psync = rs.sym_array(wgs * rs.ROC_SHMEM_REDUCE_SYNC_SIZE, np.int64, fill=0)
        heap = oracle.Heap(n_pes, 2 * n * 4)
        for p in range(n_pes):
            vals = random_values(rs.FLOAT, n, 90 + p)
            src.write(p, vals)
            heap.view(p, 0, n, np.float32)[:] = vals
        assert rs.get_pacing()[1] != 0
        rs.roc_shmem_to_all(rs.FLOAT, rs.SUM, dst, src, n, 0, 0, n_pes, None, psync, rs.Launch(wgs, wg_size))
        rs.synchronize()
        oracle.to_all_rounded_once(heap, rs.FLOAT, rs.SUM, n * 4, 0, n)
        for p in range(n_pes):
            assert np.array_equal(dst.read(p).view(np.uint32), heap.view(p, n * 4, n, np.float32).view(np.uint32)), p
        for a in (psync, dst, src):
            a.free()


def test_paced_reduction_of_arrays_that_start_off_a_vector_boundary():
    """Source and destination three elements into their allocations: the elements in front of the
    first 1 KiB boundary and behind the last whole vector go one by one, the rest is paced."""
    n_pes, wgs, wg_size, shift = 8, 32, 512, 3
    with runtime(n_pes, heap_size=256 << 20, num_blocks=wgs):
        n = (40 << 20) // 4 + 5
        src = rs.sym_array(n + 16, np.float32)
        dst = rs.sym_array(n + 16, np.float32, fill=0x5A)
        psync = rs.sym_array(wgs * rs.ROC_SHMEM_REDUCE_SYNC_SIZE, np.int64, fill=0)
        heap = oracle.Heap(n_pes, 2 * (n + 16) * 4)
        for p in range(n_pes):
            vals = random_values(rs.FLOAT, n + 16, 110 + p)
            src.write(p, vals)
            heap.view(p, 0, n + 16, np.float32)[:] = vals
            heap.view(p, (n + 16) * 4, n + 16, np.uint32)[:] = 0x5A5A5A5A
        rs.roc_shmem_to_all(rs.FLOAT, rs.SUM, dst.addr + 4 * shift, src.addr + 4 * shift, n, 0, 0, n_pes, None, psync,
                            rs.Launch(wgs, wg_size))
        rs.synchronize()
        oracle.to_all_rounded_once(heap, rs.FLOAT, rs.SUM, (n + 16 + shift) * 4, shift * 4, n)
        for p in range(n_pes):     # the whole allocation: nothing in front of or behind the range is touched
            assert np.array_equal(dst.read(p).view(np.uint32), heap.view(p, (n + 16) * 4, n + 16, np.uint32)), p
        for a in (psync, dst, src):
            a.free()


def test_paced_reduction_in_place():
    """dest == source at the default rate and the headline's launch shape: every byte range is
    read in a load slot and overwritten in the next store slot by the same lanes."""
    n_pes, wgs, wg_size = 8, 32, 1024       # 256 workgroups, 128 KiB per member per pass
    with runtime(n_pes, heap_size=512 << 20, num_blocks=32):
        n = (160 << 20) // 4 + 13            # five passes per workgroup and a ragged end
        buf = rs.sym_array(n, np.float32)
        psync = rs.sym_array(wgs * rs.ROC_SHMEM_REDUCE_SYNC_SIZE, np.int64, fill=0)
        heap = oracle.Heap(n_pes, n * 4)
        for p in range(n_pes):
            vals = random_values(rs.FLOAT, n, 70 + p)
            buf.write(p, vals)
            heap.view(p, 0, n, np.float32)[:] = vals
        assert rs.get_pacing()[1] != 0       # the library's default rate is in force
        rs.roc_shmem_to_all(rs.FLOAT, rs.SUM, buf, buf, n, 0, 0, n_pes, None, psync, rs.Launch(wgs, wg_size))
        rs.synchronize()
        oracle.to_all_rounded_once(heap, rs.FLOAT, rs.SUM, 0, 0, n)
        for p in range(n_pes):
            assert np.array_equal(buf.read(p).view(np.uint32), heap.view(p, 0, n, np.float32).view(np.uint32)), p
        assert rs.take_status() == 0
        psync.free()
        buf.free()


@pytest.mark.parametrize("rate,wgs,wg_size,tiles_per_wg", [(68000, 32, 1024, 1), (40000, 32, 512, 1),
                                                           (90000, 64, 512, 2), (68000, 32, 1024, 2)])
def test_paced_standard_calls_tiled_over_the_grid_match_the_oracle(rate, wgs, wg_size, tiles_per_wg):
    """The unchanged roc_shmem_ctx_<T>_<op>_wg_to_all, one call per tile, 256 or 512 workgroups in
    the grid and two passes or more per member and call: every call deals its tile's passes to
    its members, starts at the turn its address gives, counts itself among the streaming
    workgroups and follows the schedule.  Bit-identical to the oracle whatever the rate, with a
    ragged last tile, in place too."""
    n_pes = 8
    with runtime(n_pes, heap_size=1 << 30, num_blocks=64):
        for dtype, op, in_place in ((rs.FLOAT, rs.SUM, False), (rs.LONG, rs.SUM, True), (rs.BF16, rs.MIN, False)):
            npd = rs.NP_DTYPE[dtype]
            es = np.dtype(npd).itemsize
            tile = 3 * n_pes * wg_size * 128 // es          # three passes per member and call
            n = tile * wgs * tiles_per_wg - tile // 2 + 5    # the last tile is half a tile and ragged
            src = rs.sym_array(n, npd)
            dst = src if in_place else rs.sym_array(n, npd, fill=0x5A)
            psync = rs.sym_array(wgs * rs.ROC_SHMEM_REDUCE_SYNC_SIZE, np.int64, fill=0)
            heap = oracle.Heap(n_pes, 2 * n * es)
            for p in range(n_pes):
                vals = random_values(dtype, n, 130 + p)
                src.write(p, vals)
                heap.view(p, 0, n, npd)[:] = vals
            rs.set_pacing(0, rate)
            rs.roc_shmem_to_all(dtype, op, dst, src, n, 0, 0, n_pes, None, psync, rs.Launch(wgs, wg_size, tile))
            rs.synchronize()
            rs.set_pacing(0, 0)
            oracle.to_all_rounded_once(heap, dtype, op, 0 if in_place else n * es, 0, n)
            for p in range(n_pes):
                assert np.array_equal(dst.read(p), heap.view(p, 0 if in_place else n * es, n, npd)), (dtype, op, p)
            assert rs.take_status() == 0
            for a in ((psync, src) if in_place else (psync, dst, src)):
                a.free()


@pytest.mark.parametrize("rate", [40000, 66000, 90000])
def test_paced_shared_put_and_get_are_exact(rate):
    n_pes, nbytes = 8, (72 << 20) + 4099        # 32 x 256 per PE: 72 passes per workgroup
    with runtime(n_pes, heap_size=512 << 20, num_blocks=32):
        src = rs.sym_array(nbytes + 64, np.uint8)
        dst = rs.sym_array(nbytes + 64, np.uint8, fill=0xA5)
        rng = np.random.default_rng(9)
        payload = [rng.integers(0, 256, nbytes + 64, dtype=np.uint8) for _ in range(n_pes)]
        for p in range(n_pes):
            src.write(p, payload[p])
        rs.set_pacing(rate, 0)
        for kind, shift in ((rs.PUT, 0), (rs.GET, 16)):
            for p in range(n_pes):
                dst.fill(0xA5, pe=p)
            rs.roc_shmem_rma(kind, rs.WG_SHARED, dst.addr + shift, src.addr + shift, nbytes, 1, nbytes, nbytes, 1,
                             rs.Launch(32, 256))
            rs.synchronize()
            for p in range(n_pes):
                sender = (p - 1) % n_pes if kind == rs.PUT else (p + 1) % n_pes
                got = dst.read(p)
                assert np.array_equal(got[shift:shift + nbytes], payload[sender][shift:shift + nbytes]), (kind, p)
                assert (got[:shift] == 0xA5).all() and (got[shift + nbytes:] == 0xA5).all()
        rs.set_pacing(0, 0)
        dst.free()
        src.free()


@pytest.mark.parametrize("rate,n_pes,wgs,wg_size,ragged", [(40000, 16, 16, 512, 0), (67000, 8, 32, 1024, 0),
                                                          (90000, 16, 16, 1024, 0), (67000, 16, 16, 512, 512)])
def test_paced_alltoall_is_exact(rate, n_pes, wgs, wg_size, ragged):
    """An alltoall whose blocks are large enough to stream keeps one schedule across its blocks
    (256 workgroups, 256 KiB of every block per workgroup; with the ragged size some workgroups'
    ranges start off a 1 KiB boundary and take the unpaced path beside the others): byte for
    byte the oracle's result whatever the rate, nothing written beside the blocks."""
    block = (wgs * (256 << 10)) + ragged
    nbytes = block * n_pes
    with runtime(n_pes, heap_size=4 << (nbytes + 64).bit_length(), num_blocks=32):
        world = rs.roc_shmem_team_world()
        src = rs.sym_array(nbytes, np.uint8)
        dst = rs.sym_array(nbytes + 64, np.uint8)
        heap = oracle.Heap(n_pes, 2 * nbytes + 128)
        rng = np.random.default_rng(rate + n_pes)
        for p in range(n_pes):
            payload = rng.integers(0, 256, size=nbytes, dtype=np.uint8)
            src.write(p, payload)
            heap.view(p, 0, nbytes, np.uint8)[:] = payload
            dst.fill(0xA5, pe=p)
            heap.view(p, nbytes, nbytes + 64, np.uint8)[:] = 0xA5
        rs.set_pacing(rate, 0)
        rs.roc_shmem_alltoall(1, world, dst, src, block, rs.Launch(wgs, wg_size))
        rs.synchronize()
        rs.set_pacing(0, 0)
        oracle.alltoall(heap, nbytes, 0, block)
        for p in range(n_pes):
            assert np.array_equal(dst.read(p), heap.view(p, nbytes, nbytes + 64, np.uint8)), p
        dst.free()
        src.free()


def test_tuner_leaves_a_usable_setting_and_the_right_result():
    # The tuner may decide that pacing does not pay for this reduction on this card (rate 0);
    # what is checked is that it returns, reports both timings, leaves the rate it reports,
    # and that the reduction's result is in place.
    n_pes, n = 8, 1 << 24
    with runtime(n_pes, heap_size=256 << 20, num_blocks=32):
        src = rs.sym_array(n, np.int32)
        dst = rs.sym_array(n, np.int32, fill=0)
        psync = rs.sym_array(32 * rs.ROC_SHMEM_REDUCE_SYNC_SIZE, np.int64, fill=0)
        vals = [random_values(rs.INT, n, 70 + p) for p in range(n_pes)]
        for p in range(n_pes):
            src.write(p, vals[p])
        copy_rate = rs.get_pacing()[0]
        res = rs.tune_reduce_pacing(rs.INT, rs.SUM, dst, src, n, 0, 0, n_pes, psync, rs.Launch(32, 512))
        assert res["free_ms"] > 0 and res["paced_ms"] > 0 and res["paced_ms"] <= res["free_ms"]
        assert rs.get_pacing() == (copy_rate, res["rate"])     # the rate for copies is left alone
        assert res["rate"] == 0 or 50000 <= res["rate"] <= 72000
        want = np.sum(np.stack(vals).astype(np.int64), axis=0).astype(np.int32)
        for p in range(n_pes):
            assert np.array_equal(dst.read(p), want)
        for a in (psync, dst, src):
            a.free()
