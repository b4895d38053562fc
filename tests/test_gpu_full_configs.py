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
        for launch in (rs.Launch(1, 64), rs.Launch(64, 512), rs.Launch(64, 256)):
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
                for p in range(n_pes):
                    sender = (p - 1) % n_pes if kind == rs.PUT else (p + 1) % n_pes
                    got = dst.read(p, min(size + 64, biggest))
                    assert np.array_equal(got[:size], payload[sender][:size]), (size, kind, p)
                    assert (got[size:] == 0xA5).all(), "bytes beyond the message were touched"
            size *= 2


@pytest.mark.parametrize("dtype,kind", [(rs.FLOAT, "normal"), (rs.FLOAT, "lognormal"),
                                        (rs.BF16, "normal"), (rs.BF16, "lognormal")])
def test_config3_sum_max_min_8_slices_2e26(dtype, kind):
    n_pes, n = 8, 1 << 26
    npd = rs.NP_DTYPE[dtype]
    es = np.dtype(npd).itemsize
    # Three windows (start, middle, end of the arrays; 3 x 5.6 M > 2^24 elements in all) are compared
    # with the CPU oracle: bit for bit with the restated fold, and for sums also within the stated
    # tolerance of the long-double truth.  The rest of the result is covered by "every PE holds
    # the same bits".
    window = 5_600_000
    starts = [0, n // 2 - 12345, n - window]
    with runtime(n_pes, heap_size=1 << 30, num_blocks=64):
        src = rs.sym_array(n, npd)
        dst = rs.sym_array(n, npd)
        psync = rs.sym_array(64 * 256, np.int64, fill=0)
        heap = oracle.Heap(n_pes, 2 * 3 * window * es)
        rng = np.random.default_rng(3)
        for p in range(n_pes):
            x = rng.standard_normal(n, dtype=np.float32)
            if kind == "lognormal":
                x = np.sign(x) * np.exp(2.0 * rng.standard_normal(n, dtype=np.float32))
            vals = oracle.float_to_bf16(x) if dtype == rs.BF16 else x
            src.write(p, vals)
            for w, at in enumerate(starts):
                heap.view(p, w * window * es, window, npd)[:] = vals[at:at + window]
        m = 3 * window
        # sum: the benchmark's own configurations, at the library's default pacing rates - the
        # standard call, one per workgroup over a tile of 2^21 elements, 32 workgroups of 1024
        # lanes per PE (the headline), and the sharded extension with the same launch; max and min
        # with 64 x 512 lanes per PE sharing one call (not paced at that grid size)
        assert rs.get_pacing()[1] != 0
        cases = [(rs.SUM, rs.Launch(32, 1024, 1 << 21)), (rs.SUM, rs.Launch(32, 1024)),
                 (rs.MAX, rs.Launch(64, 512)), (rs.MIN, rs.Launch(64, 512))]
        for op, launch in cases:
            for p in range(n_pes):
                dst.fill(0x5A, pe=p)
            rs.roc_shmem_to_all(dtype, op, dst, src, n, 0, 0, n_pes, None, psync, launch)
            rs.synchronize()
            first = dst.read(0)
            for p in range(1, n_pes):       # every PE holds the same bits
                assert np.array_equal(dst.read(p), first)
            got = np.concatenate([first[at:at + window] for at in starts])
            oracle.to_all_rounded_once(heap, dtype, op, m * es, 0, m)
            assert np.array_equal(got, heap.view(0, m * es, m, npd)), "differs from the restated fold"
            if op == rs.SUM:
                check_fp(dtype, got, oracle.to_all_f64(heap, dtype, op, 0, m),
                         oracle.abs_sum_f64(heap, dtype, 0, m))


class Config4:
    """10 M small operations (8-byte puts to unique words of the lower half of every slice,
    int64 fetch-adds to random words of the upper half) issued by 1024 workgroups of 256 threads
    over 16 slices of 64 MiB."""
    n_pes, n_ops, wgs_total, wg_size = 16, 10_000_000, 1024, 256
    slice_bytes = 64 << 20
    words = slice_bytes // 8
    num_blocks = 64

    def __init__(self):
        rng = np.random.default_rng(4)
        n_ops, n_pes, words = self.n_ops, self.n_pes, self.words
        ops = np.zeros(n_ops, rs.SMALL_OP_DTYPE)
        self.is_put = np.arange(n_ops) % 2 == 0
        ops["kind"] = np.where(self.is_put, rs.OP_P64, rs.OP_FADD64)
        ops["pe"] = rng.integers(0, n_pes, n_ops)
        uniq = rng.permutation(n_pes * (words // 2))[:n_ops]          # puts: unique (pe, word)
        ops["pe"][self.is_put] = uniq[self.is_put] // (words // 2)
        ops["offset"] = np.where(self.is_put, (uniq % (words // 2)) * 8,
                                 (words // 2 + rng.integers(0, words // 2, n_ops)) * 8)
        ops["value"] = np.where(self.is_put, rng.integers(-(1 << 62), 1 << 62, n_ops),
                                rng.integers(-1000, 1000, n_ops))
        self.ops = ops
        i = np.arange(n_ops)
        blk = (i % (self.wgs_total * self.wg_size)) // self.wg_size
        self.issuer = (blk % n_pes).astype(np.uint32)
        self.ring = self.issuer.astype(np.int64) * self.num_blocks + (blk // n_pes) % self.num_blocks

    def run(self, mem, launch_stream=None):
        shifted = self.ops.copy()
        shifted["offset"] += mem.offset
        dev = rs.device_array(shifted)
        rs.roc_shmem_small_ops(dev, self.n_ops, None,
                               rs.Launch(self.wgs_total // self.n_pes, self.wg_size, 0, launch_stream))
        return dev, shifted

    def check_heap(self, mem):
        heap = oracle.Heap(self.n_pes, self.slice_bytes)
        oracle.small_ops(heap, self.ops, self.issuer)
        for p in range(self.n_pes):
            assert np.array_equal(mem.read(p), heap.view(p, 0, self.words, np.int64)), "heap of PE %d" % p

    def check_rings(self, shifted, sq, live=False):
        """Every entry the rings hold against the CPU builder, byte for byte: all entries when no
        ring wrapped (then every operation must also be found exactly once), else the newest `sq`
        of every ring.  live: the rings were queues with a live consumer, where the quiet that ends
        each workgroup's part of the kernel posts a zero-byte read (one workgroup per ring here:
        one more entry per ring, its newest)."""
        n_pes, num_blocks = self.n_pes, self.num_blocks
        base0, stride = rs.heap_base(0), rs.heap_base(1) - rs.heap_base(0)
        expect = np.zeros(self.n_ops, oracle.WQE_EXPECT_DTYPE)
        expect["opcode"] = np.where(self.is_put, oracle.OP_WRITE, oracle.OP_ATOMIC_FA)
        expect["raddr"] = (base0 + shifted["pe"].astype(np.int64) * stride +
                           shifted["offset"].astype(np.int64)).astype(np.uint64)
        expect["data"] = shifted["value"].astype(np.int64).view(np.uint64)
        expect["size"] = 8
        flush = [rs.sq_flush_target(p) for p in range(n_pes)]
        order = np.argsort(self.ring, kind="stable")
        bounds = np.searchsorted(self.ring[order], np.arange(n_pes * num_blocks + 1))
        rkeys = [rs.sq_rkey(p) for p in range(n_pes)]
        checked = 0
        for pe in range(n_pes):
            for block in range(num_blocks):
                r = pe * num_blocks + block
                mine = order[bounds[r]:bounds[r + 1]]
                st = rs.sq_state(pe, block)
                count = int(st["sq_counter"])
                assert count == st["published"] == len(mine) + (1 if live else 0), (pe, block)
                assert st["atomic_counter"] == int((~self.is_put[mine]).sum())
                wrapped = count > sq
                first = count - sq if wrapped else 0
                image = rs.sq_image(pe, block, sq)
                c = rs.sq_constants(pe, block)
                qp = oracle.Qp()
                qp.ctrl_qp_sq, qp.ctrl_sig, qp.lkey = c["ctrl_qp_sq"], c["ctrl_sig"], c["lkey"]
                qp.atomic_lkey, qp.atomic_ret_base, qp.max_nwqe = c["atomic_lkey"], c["atomic_ret_base"], sq
                mine_expect = expect[mine]
                if live:
                    quiet_entry = np.zeros(1, oracle.WQE_EXPECT_DTYPE)
                    quiet_entry["opcode"], quiet_entry["raddr"] = oracle.OP_READ, base0 + pe * stride
                    mine_expect = np.concatenate([mine_expect, quiet_entry])
                res = oracle.ring_check(image, qp, first, count - first, oracle.sort_wqe_expect(mine_expect),
                                        base0, stride, self.slice_bytes * 4, rkeys, full_slot=not wrapped,
                                        flush_base=flush[0][0], flush_rkeys=[k for _, k in flush])
                assert res["ok"], "ring %d/%d entry %d: %s" % (pe, block, first + res["position"], res["reason"])
                checked += count - first
                newest = image[(count - 1) % sq]
                assert newest[11] == 8, "the entry that closes the last post asks for a completion"
                if live:    # READ, two segments, addressed to the issuing PE's heap
                    assert newest[3] == oracle.OP_READ and newest[7] == 2
                    assert int.from_bytes(bytes(newest[16:24]), "big") == base0 + pe * stride
                assert np.array_equal(st["mailbox"], oracle.doorbell(newest, count))
                if not wrapped:
                    assert res["used"].all(), "an operation of ring %d/%d left no entry" % (pe, block)
                    n_atomic = res["n_atomic"]
                    dense = n_atomic // 4096 + (np.arange(4096) < n_atomic % 4096)
                    assert np.array_equal(res["pos_count"], dense), "AMO return slots are handed out densely"
                    assert not image[count:].any(), "slots beyond the producer index stay untouched"
        return checked


def test_config4_every_ring_entry_of_ten_million_small_ops_byte_exact():
    # Rings of 16384 entries hold everything a workgroup posts (about 9766 entries each): all
    # 10 M entries are compared with the CPU builder and every operation is accounted for.
    cfg = Config4()
    with runtime(cfg.n_pes, heap_size=256 << 20, num_blocks=cfg.num_blocks, sq_size=16384):
        mem = rs.sym_array(cfg.words, np.int64, fill=0)
        rs.sq_reset()
        dev, shifted = cfg.run(mem)
        rs.synchronize()
        cfg.check_heap(mem)
        assert cfg.check_rings(shifted, 16384) == cfg.n_ops
        totals = rs.sq_consume()
        assert totals["retired"] == cfg.n_ops and totals["rejected"] == 0 and totals["lost"] == 0
        assert totals["writes"] == cfg.n_ops // 2 and totals["atomics"] == cfg.n_ops // 2
        dev.free()


def test_config4_ten_million_small_ops_16_slices_64MiB():
    # The benchmark's shape: 1024-entry rings that wrap about nine times.  The heap is compared
    # in full, and all 1 Mi entries that survive in the rings with the CPU builder.
    cfg = Config4()
    with runtime(cfg.n_pes, heap_size=256 << 20, num_blocks=cfg.num_blocks, sq_size=1024):
        mem = rs.sym_array(cfg.words, np.int64, fill=0)
        rs.sq_reset()
        dev, shifted = cfg.run(mem)
        rs.synchronize()
        cfg.check_heap(mem)
        assert cfg.check_rings(shifted, 1024) == cfg.n_pes * cfg.num_blocks * 1024
        dev.free()


def test_config4_through_queues_with_a_live_consumer_nothing_lost():
    # The same stream through 1024-entry rings run as queues: a consumer kernel retires entries
    # while the producers post, producers wait for space instead of overwriting, quiet collects
    # the completions.  Every one of the 10 M entries is seen by the consumer.
    cfg = Config4()
    with runtime(cfg.n_pes, heap_size=256 << 20, num_blocks=cfg.num_blocks, sq_size=1024):
        mem = rs.sym_array(cfg.words, np.int64, fill=0)
        rs.sq_reset()
        stream = rs.Stream()
        rs.sq_consumer_start()
        try:
            dev, shifted = cfg.run(mem, stream)
            stream.synchronize()
        finally:
            totals = rs.sq_consumer_stop()
        assert totals["lost"] == 0 and totals["rejected"] == 0, totals
        # every workgroup's closing quiet posts one zero-byte read before it collects completions
        assert totals["retired"] == cfg.n_ops + cfg.wgs_total and totals["bytes"] == 8 * cfg.n_ops
        assert totals["writes"] == cfg.n_ops // 2 and totals["atomics"] == cfg.n_ops // 2
        assert totals["reads"] == cfg.wgs_total
        assert rs.take_status() == 0
        cfg.check_heap(mem)
        assert cfg.check_rings(shifted, 1024, live=True) == cfg.n_pes * cfg.num_blocks * 1024
        completions = 0
        for pe in range(cfg.n_pes):
            for block in range(cfg.num_blocks):
                cons, reader = rs.sq_consumer_state(pe, block), rs.cq_reader_state(pe, block)
                assert cons["consumed"] == rs.sq_state(pe, block)["published"]
                # quiet took every completion the queue had asked for
                assert reader == {"cq_consumer": cons["cq_producer"], "quiet_counter": 0,
                                  "cq_doorbell_record": cons["cq_producer"]}, (pe, block)
                completions += cons["cq_producer"]
        assert completions == totals["completions"]
        stream.destroy()
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
        for j in range(n_pes):
            got = dst.read(j)
            for i in range(n_pes):
                assert np.array_equal(got[i * bb:(i + 1) * bb], data[i][j * bb:(j + 1) * bb]), (i, j)
