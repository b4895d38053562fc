"""The five benchmark workloads at their full sizes, through the C ABI.

Small-size parity is covered elsewhere; here the same paths run at the sizes the
throughput figures are quoted on and are compared with the oracle on the full data (or,
where that would take minutes, on the whole result through exact properties plus an
oracle comparison of a large sample)."""
import numpy as np
import pytest

import oracle
import roc_shmem_amd as rs
from helpers import check_fp, runtime

pytestmark = pytest.mark.gpu


def test_config1_int64_sum_4_slices_2e20():
    n_pes, n = 4, 1 << 20
    with runtime(n_pes, heap_size=64 << 20, num_blocks=64):
        src = rs.sym_array(n, np.int64)
        dst = rs.sym_array(n, np.int64, fill=0x5A)
        psync = rs.sym_array(64 * 256, np.int64, fill=0)
        heap = oracle.Heap(n_pes, 2 * n * 8)
        rng = np.random.default_rng(1)
        for p in range(n_pes):
            vals = rng.integers(-(1 << 30), (1 << 30) + 1, size=n, dtype=np.int64)
            src.write(p, vals)
            heap.view(p, 0, n, np.int64)[:] = vals
        for launch in (rs.Launch(1, 64), rs.Launch(64, 512)):
            for p in range(n_pes):
                dst.fill(0x5A, pe=p)
            rs.roc_shmem_to_all(rs.LONG, rs.SUM, dst, src, n, 0, 0, n_pes, None, psync, launch)
            rs.synchronize()
            oracle.to_all(heap, oracle.LONG, oracle.SUM, n * 8, 0, n)
            for p in range(n_pes):
                assert np.array_equal(dst.read(p), heap.view(p, n * 8, n, np.int64))


def test_config2_putmem_getmem_sweep_8_slices_1GiB_heap():
    n_pes = 8
    biggest = 64 << 20
    with runtime(n_pes, heap_size=1 << 30, num_blocks=64):
        src = rs.sym_array(biggest, np.uint8)
        dst = rs.sym_array(biggest, np.uint8)
        rng = np.random.default_rng(2)
        payload = [rng.integers(0, 256, size=biggest, dtype=np.uint8) for _ in range(n_pes)]
        for p in range(n_pes):
            src.write(p, payload[p])
        size = 8
        while size <= biggest:
            for kind in (rs.PUT, rs.GET):
                for p in range(n_pes):
                    dst.fill(0xA5, pe=p)
                if size <= 256 << 10:
                    rs.roc_shmem_rma(kind, rs.WG, dst, src, size, 1, size, size, 1, rs.Launch(1, 256))
                else:  # large messages tiled over the PE's workgroups, 256 KiB per call
                    tile = 256 << 10
                    rs.roc_shmem_rma(kind, rs.WG, dst, src, tile, size // tile, tile, tile, 1,
                                     rs.Launch(32, 512))
                rs.synchronize()
                for p in (0, 3, 7):
                    sender = (p - 1) % n_pes if kind == rs.PUT else (p + 1) % n_pes
                    got = dst.read(p, min(size + 64, biggest))
                    assert np.array_equal(got[:size], payload[sender][:size]), (size, kind, p)
                    assert (got[size:] == 0xA5).all(), "bytes beyond the message were touched"
            size *= 2


@pytest.mark.parametrize("dtype,kind", [(rs.FLOAT, "normal"), (rs.BF16, "lognormal")])
def test_config3_sum_max_min_8_slices_2e26(dtype, kind):
    n_pes, n = 8, 1 << 26
    npd = rs.NP_DTYPE[dtype]
    es = np.dtype(npd).itemsize
    sample = 1 << 22                       # elements compared against the long-double truth
    with runtime(n_pes, heap_size=1 << 30, num_blocks=64):
        src = rs.sym_array(n, npd)
        dst = rs.sym_array(n, npd)
        psync = rs.sym_array(64 * 256, np.int64, fill=0)
        heap = oracle.Heap(n_pes, 2 * sample * es)
        rng = np.random.default_rng(3)
        offset = (n // 2) - 12345           # the sample sits away from the array's start
        for p in range(n_pes):
            x = rng.standard_normal(n, dtype=np.float32)
            if kind == "lognormal":
                x = np.sign(x) * np.exp(2.0 * rng.standard_normal(n, dtype=np.float32))
            vals = oracle.float_to_bf16(x) if dtype == rs.BF16 else x
            src.write(p, vals)
            heap.view(p, 0, sample, npd)[:] = vals[offset:offset + sample]
        launch = rs.Launch(64, 512)
        for op in (rs.SUM, rs.MAX, rs.MIN):
            rs.roc_shmem_to_all(dtype, op, dst, src, n, 0, 0, n_pes, None, psync, launch)
            rs.synchronize()
            first = dst.read(0)
            for p in range(1, n_pes):       # every PE holds the same bits
                assert np.array_equal(dst.read(p), first)
            got = first[offset:offset + sample]
            if op == rs.SUM:
                check_fp(dtype, got, oracle.to_all_f64(heap, dtype, op, 0, sample),
                         oracle.abs_sum_f64(heap, dtype, 0, sample))
            else:
                oracle.to_all(heap, dtype, op, sample * es, 0, sample)
                assert np.array_equal(got, heap.view(0, sample * es, sample, npd))


def test_config4_ten_million_small_ops_16_slices_64MiB():
    n_pes, n_ops, wgs_total, wg_size = 16, 10_000_000, 1024, 256
    slice_bytes = 64 << 20
    words = slice_bytes // 8
    num_blocks = 64
    with runtime(n_pes, heap_size=256 << 20, num_blocks=num_blocks, sq_size=1024):
        mem = rs.sym_array(words, np.int64, fill=0)
        rng = np.random.default_rng(4)
        ops = np.zeros(n_ops, rs.SMALL_OP_DTYPE)
        is_put = np.arange(n_ops) % 2 == 0
        ops["kind"] = np.where(is_put, rs.OP_P64, rs.OP_FADD64)
        ops["pe"] = rng.integers(0, n_pes, n_ops)
        uniq = rng.permutation(n_pes * (words // 2))[:n_ops]          # puts: unique (pe, word)
        ops["pe"][is_put] = uniq[is_put] // (words // 2)
        ops["offset"] = np.where(is_put, (uniq % (words // 2)) * 8,
                                 (words // 2 + rng.integers(0, words // 2, n_ops)) * 8)
        ops["value"] = np.where(is_put, rng.integers(-(1 << 62), 1 << 62, n_ops),
                                rng.integers(-1000, 1000, n_ops))
        shifted = ops.copy()
        shifted["offset"] += mem.offset
        dev = rs.device_array(shifted)
        rs.sq_reset()
        rs.roc_shmem_small_ops(dev, n_ops, None, rs.Launch(wgs_total // n_pes, wg_size))
        rs.synchronize()
        # final heap state, bit for bit
        i = np.arange(n_ops)
        total_threads = wgs_total * wg_size
        blk = (i % total_threads) // wg_size
        issuer = (blk % n_pes).astype(np.uint32)
        heap = oracle.Heap(n_pes, slice_bytes)
        oracle.small_ops(heap, ops, issuer)
        for p in range(n_pes):
            assert np.array_equal(mem.read(p), heap.view(p, 0, words, np.int64)), "heap of PE %d" % p
        # every ring: producer indices equal the number of entries its workgroup posted
        ring_block = (blk // n_pes) % num_blocks
        per_ring = np.bincount(issuer.astype(np.int64) * num_blocks + ring_block,
                               minlength=n_pes * num_blocks)
        per_ring_amo = np.bincount((issuer.astype(np.int64) * num_blocks + ring_block)[~is_put],
                                   minlength=n_pes * num_blocks)
        base0, stride = rs.heap_base(0), rs.heap_base(1) - rs.heap_base(0)
        for pe in range(n_pes):
            for block in range(0, num_blocks, 9):          # a sample of rings in full detail
                st = rs.sq_state(pe, block)
                assert st["sq_counter"] == st["published"] == per_ring[pe * num_blocks + block]
                assert st["atomic_counter"] == per_ring_amo[pe * num_blocks + block]
                image = rs.sq_image(pe, block, 1024)
                count = int(st["sq_counter"])
                assert count > 1024            # the ring wrapped several times
                # the ring holds the last 1024 entries: indices form one cyclic run
                idx = (image[:, 1].astype(np.int64) << 8) | image[:, 2]
                slot = np.arange(1024)
                newest = (count - 1) % 1024
                want = np.where(slot <= newest, count - 1 - (newest - slot),
                                count - 1 - (newest + 1024 - slot)) & 0xFFFF
                assert np.array_equal(idx, want)
                # every entry is one of this ring's operations: check target and operand
                mine = np.nonzero((issuer == pe) & (ring_block == block))[0]
                raddr_of = base0 + shifted["pe"][mine].astype(np.int64) * stride + shifted["offset"][mine].astype(np.int64)
                put_keys = set(zip(raddr_of[is_put[mine]].tolist(), shifted["value"][mine][is_put[mine]].tolist()))
                amo_keys = set(zip(raddr_of[~is_put[mine]].tolist(), shifted["value"][mine][~is_put[mine]].tolist()))
                for k in range(0, 1024, 7):
                    e = image[k]
                    raddr = int.from_bytes(bytes(e[16:24]), "big")
                    if e[3] == oracle.OP_WRITE:
                        val = int.from_bytes(bytes(e[36:44]), "little", signed=True)
                        assert bytes(e[32:36]) == bytes([0x80, 0, 0, 8]) and (raddr, val) in put_keys
                    else:
                        val = int.from_bytes(bytes(e[32:40]), "big", signed=True)
                        assert e[3] == oracle.OP_ATOMIC_FA and e[7] == 4 and (raddr, val) in amo_keys
                    dest = (raddr - base0) // stride
                    assert int.from_bytes(bytes(e[24:28]), "little") == rs.sq_rkey(dest)
        dev.free()


def test_config5_broadcast_and_alltoall_16_slices_64MiB():
    n_pes, slice_bytes = 16, 64 << 20
    with runtime(n_pes, heap_size=256 << 20, num_blocks=64):
        world = rs.roc_shmem_team_world()
        src = rs.sym_array(slice_bytes, np.uint8)
        dst = rs.sym_array(slice_bytes, np.uint8)
        rng = np.random.default_rng(5)
        # uniform random 32-bit patterns, NaN patterns included: they must move bit for bit
        data = [rng.integers(0, 1 << 32, size=slice_bytes // 4, dtype=np.uint32).view(np.uint8)
                for _ in range(n_pes)]
        for p in range(n_pes):
            src.write(p, data[p])
        nelem = slice_bytes // 4
        for root in (0, 7):
            for p in range(n_pes):
                dst.fill(0xC3, pe=p)
            rs.roc_shmem_team_broadcast(4, world, dst, src, nelem, root, rs.Launch(16, 512))
            rs.synchronize()
            for p in range(n_pes):
                got = dst.read(p)
                if p == root:
                    assert (got == 0xC3).all()
                else:
                    assert np.array_equal(got, data[root])
        block = nelem // n_pes                      # 2^20 four-byte elements per block
        rs.roc_shmem_alltoall(4, world, dst, src, block, rs.Launch(16, 512))
        rs.synchronize()
        bb = block * 4
        for j in (0, 5, 15):
            got = dst.read(j)
            for i in range(n_pes):
                assert np.array_equal(got[i * bb:(i + 1) * bb], data[i][j * bb:(j + 1) * bb]), (i, j)
