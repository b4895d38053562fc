"""Consumer pass over the GPU-built send queues: replaying the rings onto a copy of the heap
reproduces what the producers did; completion entries, retirement and queue mode."""
import os

import numpy as np
import pytest

import oracle
import roc_shmem_amd as rs
from helpers import runtime
from test_gpu_small_ops import Issue, qp_of

pytestmark = pytest.mark.gpu

WORDS = 1 << 16                      # int64 words of the test object per PE
SRC, PUT_DST, GET_DST, COUNTERS, CSWAP, SMALL = 0, 8192, 24576, 40960, 41984, 49152
CHUNK = 1024                         # bytes reserved per putmem / getmem destination


def build_stream(n_ops, n_pes, wgs, wg_size, num_blocks, seed):
    """Operations whose final memory image does not depend on the order rings are served in:
    unique destinations for puts, gets and compare-swaps, fetch-add counters private to the
    issuing ring, sources nobody writes."""
    rng = np.random.default_rng(seed)
    issue = Issue(n_ops, n_pes, wgs, wg_size, num_blocks)
    ops = np.zeros(n_ops, rs.SMALL_OP_DTYPE)
    kind = rng.choice([rs.OP_P64, rs.OP_P32, rs.OP_PUTMEM, rs.OP_GETMEM, rs.OP_FADD64, rs.OP_FINC64,
                       rs.OP_ADD64, rs.OP_INC64, rs.OP_CSWAP64, rs.OP_FETCH64],
                      n_ops, p=[.32, .1, .03, .03, .15, .1, .07, .05, .1, .05])
    ops["kind"] = kind
    ops["pe"] = rng.integers(0, n_pes, n_ops)
    ops["value"] = rng.integers(-(1 << 40), 1 << 40, n_ops)

    small = np.isin(kind, [rs.OP_P64, rs.OP_P32])
    uniq = rng.permutation(n_pes * (WORDS - SMALL))[:n_ops]
    ops["pe"][small] = uniq[small] // (WORDS - SMALL)
    ops["offset"][small] = (SMALL + uniq[small] % (WORDS - SMALL)) * 8

    put = np.nonzero(kind == rs.OP_PUTMEM)[0]
    chunks = rng.permutation(n_pes * ((GET_DST - PUT_DST) * 8 // CHUNK))[:len(put)]
    ops["pe"][put] = chunks // ((GET_DST - PUT_DST) * 8 // CHUNK)
    ops["offset"][put] = PUT_DST * 8 + (chunks % ((GET_DST - PUT_DST) * 8 // CHUNK)) * CHUNK \
        + rng.integers(0, 8, len(put))                                  # odd alignments too
    ops["aux"][put] = rng.choice([3, 8, 9, 16, 64, 200, 1000], len(put))
    ops["value"][put] = SRC * 8 + rng.integers(0, (PUT_DST - SRC) * 8 - 1024, len(put))

    get = np.nonzero(kind == rs.OP_GETMEM)[0]
    per_pe = np.zeros(n_pes, np.int64)
    for i in get:                                                        # local destination: issuer's slice
        pe = int(issue.pe[i])
        ops["value"][i] = GET_DST * 8 + per_pe[pe] * CHUNK
        per_pe[pe] += 1
    assert per_pe.max() <= (COUNTERS - GET_DST) * 8 // CHUNK
    ops["aux"][get] = rng.choice([12, 16, 256, 1000], len(get))
    ops["offset"][get] = SRC * 8 + rng.integers(0, (PUT_DST - SRC) * 8 - 1024, len(get))

    amo = np.isin(kind, [rs.OP_FADD64, rs.OP_FINC64, rs.OP_ADD64, rs.OP_INC64])
    ops["pe"][amo] = (issue.pe[amo] + 1) % n_pes
    ops["offset"][amo] = (COUNTERS + issue.ring_block[amo] * 4 + rng.integers(0, 4, amo.sum())) * 8

    cs = np.nonzero(kind == rs.OP_CSWAP64)[0]
    cells = rng.permutation(n_pes * (SMALL - CSWAP))[:len(cs)]
    ops["pe"][cs] = cells // (SMALL - CSWAP)
    ops["offset"][cs] = (CSWAP + cells % (SMALL - CSWAP)) * 8
    ops["aux"][cs] = rng.integers(0, 2, len(cs))                         # the cells hold 0 or 1

    fetch = kind == rs.OP_FETCH64
    ops["offset"][fetch] = (SRC + rng.integers(0, PUT_DST - SRC, fetch.sum())) * 8
    return ops, issue


def test_replaying_the_rings_reproduces_the_heap_and_matches_the_cpu_consumer():
    n_pes, wgs, wg_size, num_blocks, sq = 4, 4, 256, 4, 1024
    n_ops = 12000
    ops, issue = build_stream(n_ops, n_pes, wgs, wg_size, num_blocks, seed=21)
    rng = np.random.default_rng(22)
    with runtime(n_pes, heap_size=16 << 20, num_blocks=num_blocks, sq_size=sq):
        mem = rs.sym_array(WORDS, np.int64)
        for p in range(n_pes):
            init = rng.integers(-(1 << 62), 1 << 62, WORDS, dtype=np.int64)
            init[CSWAP:SMALL] = rng.integers(0, 2, SMALL - CSWAP)
            mem.write(p, init)
        shifted = ops.copy()
        shifted["offset"] += mem.offset
        moves = np.isin(shifted["kind"], [rs.OP_PUTMEM, rs.OP_GETMEM])
        shifted["value"][moves] += mem.offset

        base, nbytes, stride = rs.arena()
        assert base == rs.heap_base(0) and stride == rs.heap_base(1) - rs.heap_base(0)
        before = rs.read_device(base, nbytes)
        shadow = rs.device_array(before)

        dev_ops = rs.device_array(shifted)
        rs.sq_reset()
        rs.roc_shmem_small_ops(dev_ops, n_ops, None, rs.Launch(wgs, wg_size))
        rs.synchronize()
        after = rs.read_device(base, nbytes)
        assert not np.array_equal(before, after)

        totals = rs.sq_consume(target_arena=shadow)
        replayed = shadow.read(np.uint8, nbytes)
        assert totals["rejected"] == 0 and totals["lost"] == 0 and totals["local_skipped"] == 0
        diff = np.nonzero(replayed != after)[0]
        assert diff.size == 0, "replay differs from the heap at arena offset %d (%d bytes)" % (
            diff[0], diff.size)
        assert np.array_equal(rs.read_device(base, nbytes), after), "the pass must not touch the heap"

        # The same rings through the CPU consumer: memory, return windows, completion queues, totals.
        rkeys = [rs.sq_rkey(p) for p in range(n_pes)]
        host_target = before.copy()
        sum_totals = oracle.ConsumeTotals()
        retired = 0
        for pe in range(n_pes):
            for block in range(num_blocks):
                st = rs.sq_state(pe, block)
                assert st["published"] == st["sq_counter"] <= sq
                cons = rs.sq_consumer_state(pe, block)
                assert cons["consumed"] == st["published"]
                retired += st["published"]
                qp = qp_of(pe, block)
                ring = rs.sq_image(pe, block, sq).reshape(-1)
                ret = np.zeros(4096, np.uint64)
                cq = np.zeros(sq * 64, np.uint8)
                cq[63::64] = 0xF0
                prod, _ = oracle.sq_consume(qp, ring, 0, st["published"], base, stride, 16 << 20, rkeys,
                                            host_target, after, ret, cq, 0, sum_totals)
                assert prod == cons["cq_producer"] and prod > 0
                assert np.array_equal(rs.cq_image(pe, block, sq).reshape(-1), cq), (pe, block)
                assert np.array_equal(rs.atomic_ret_image(pe, block), ret), (pe, block)
        assert np.array_equal(host_target, after)
        assert sum_totals.as_dict() == totals and totals["retired"] == retired
        assert totals["writes"] > 0 and totals["reads"] > 0 and totals["atomics"] > 0

        # Nothing is left: a second pass retires nothing.
        again = rs.sq_consume(target_arena=shadow)
        assert again["retired"] == 0 and again["completions"] == 0
        dev_ops.free()
        shadow.free()
        mem.free()


def test_check_only_pass_completes_entries_without_touching_memory():
    n_pes, num_blocks = 2, 2
    with runtime(n_pes, heap_size=4 << 20, num_blocks=num_blocks, sq_size=256):
        mem = rs.sym_array(4096, np.int64, fill=0)
        n_ops = 2 * 2 * 64
        issue = Issue(n_ops, n_pes, 2, 64, num_blocks)
        ops = np.zeros(n_ops, rs.SMALL_OP_DTYPE)
        ops["kind"] = rs.OP_P64
        ops["pe"] = (issue.pe + 1) % n_pes
        ops["offset"] = mem.offset + np.arange(n_ops) * 16       # not lane-contiguous: nothing merges
        ops["value"] = np.arange(n_ops) + 1
        dev_ops = rs.device_array(ops)
        rs.sq_reset()
        rs.roc_shmem_small_ops(dev_ops, n_ops, None, rs.Launch(2, 64))
        rs.synchronize()
        base, nbytes, _ = rs.arena()
        after = rs.read_device(base, nbytes)
        totals = rs.sq_consume()
        assert totals == {"retired": n_ops, "writes": n_ops, "reads": 0, "atomics": 0, "bytes": 8 * n_ops,
                          "completions": 4, "lost": 0, "rejected": 0, "local_skipped": 0}
        assert np.array_equal(rs.read_device(base, nbytes), after)
        for pe in range(n_pes):
            for block in range(num_blocks):
                cq = rs.cq_image(pe, block, 256)
                # one wave posted 64 entries and asked for a completion on the last one
                assert int.from_bytes(bytes(cq[0][60:62]), "big") == 63 and cq[0][63] == 0
                assert (cq[1:, 63] == 0xF0).all() and not cq[1:, :63].any()
        dev_ops.free()
        mem.free()


def test_wrapped_log_reports_overwritten_entries_as_lost():
    n_pes, sq = 2, 64
    with runtime(n_pes, heap_size=4 << 20, num_blocks=1, sq_size=sq):
        mem = rs.sym_array(8192, np.int64, fill=0)
        n_ops = n_pes * 64 * 5                                     # five posts of one wave per ring
        ops = np.zeros(n_ops, rs.SMALL_OP_DTYPE)
        ops["kind"] = rs.OP_FADD64
        ops["pe"] = np.arange(n_ops) % n_pes
        ops["offset"] = mem.offset + (np.arange(n_ops) % 4096) * 16
        ops["value"] = 1
        dev_ops = rs.device_array(ops)
        rs.sq_reset()
        rs.roc_shmem_small_ops(dev_ops, n_ops, None, rs.Launch(1, 64))
        rs.synchronize()
        totals = rs.sq_consume()
        assert totals["lost"] == n_ops - n_pes * sq and totals["retired"] == n_pes * sq
        assert totals["rejected"] == 0 and totals["atomics"] == n_pes * sq
        dev_ops.free()
        mem.free()


def test_ring_shared_by_workgroups_on_different_xcds_keeps_the_newest_entries():
    # 32 workgroups per PE feed one ring (ROC_SHMEM_NUM_BLOCKS = 1) and wrap it many times.  Every
    # slot must end up holding the entry of the last lap (shared rings are written through to memory
    # so that this does not depend on the order in which the XCDs' L2s are written back): the
    # consumer pass finds each index field equal to the slot's position in the stream.
    n_pes, sq, wgs, wg_size = 2, 256, 32, 256
    with runtime(n_pes, heap_size=8 << 20, num_blocks=1, sq_size=sq):
        mem = rs.sym_array(1 << 16, np.int64, fill=0)
        n_ops = n_pes * wgs * wg_size * 6
        rng = np.random.default_rng(3)
        ops = np.zeros(n_ops, rs.SMALL_OP_DTYPE)
        ops["kind"] = rng.choice([rs.OP_P64, rs.OP_FADD64, rs.OP_P32], n_ops)
        ops["pe"] = rng.integers(0, n_pes, n_ops)
        ops["offset"] = mem.offset + rng.integers(0, 1 << 16, n_ops) * 8
        ops["value"] = rng.integers(-5, 5, n_ops)
        dev_ops = rs.device_array(ops)
        rs.sq_reset()
        rs.roc_shmem_small_ops(dev_ops, n_ops, None, rs.Launch(wgs, wg_size))
        rs.synchronize()
        per_ring = n_ops // n_pes
        for pe in range(n_pes):
            st = rs.sq_state(pe, 0)
            assert st["sq_counter"] == per_ring and st["published"] == per_ring
            image = rs.sq_image(pe, 0, sq)
            for k in range(sq):
                newest = per_ring - sq + ((k - (per_ring - sq)) % sq)
                assert int.from_bytes(bytes(image[k][1:3]), "big") == newest & 0xFFFF, (pe, k)
        totals = rs.sq_consume()
        assert totals["rejected"] == 0 and totals["retired"] == n_pes * sq
        assert totals["lost"] == n_pes * (per_ring - sq)
        dev_ops.free()
        mem.free()


def post_one_wave_per_ring(mem, n_pes, value):
    n_ops = n_pes * 64
    ops = np.zeros(n_ops, rs.SMALL_OP_DTYPE)
    ops["kind"] = rs.OP_P64
    ops["pe"] = np.arange(n_ops) % n_pes
    ops["offset"] = mem.offset + np.arange(n_ops) * 16
    ops["value"] = value
    dev_ops = rs.device_array(ops)
    rs.roc_shmem_small_ops(dev_ops, n_ops, None, rs.Launch(1, 64))
    rs.synchronize()
    dev_ops.free()


def test_queue_mode_slots_are_freed_by_the_consumer_pass():
    n_pes, sq = 2, 64
    with runtime(n_pes, heap_size=4 << 20, num_blocks=1, sq_size=sq):
        mem = rs.sym_array(4096, np.int64, fill=0)
        rs.sq_reset()
        rs.sq_set_mode(True)
        try:
            for lap in range(3):                                   # each lap fills the ring exactly
                post_one_wave_per_ring(mem, n_pes, lap + 1)
                assert rs.take_status() == 0
                st = rs.sq_state(0, 0)
                assert st["published"] == sq * (lap + 1)
                assert rs.sq_consumer_state(0, 0)["consumed"] == sq * lap
                totals = rs.sq_consume()
                assert totals["retired"] == n_pes * sq and totals["lost"] == 0 and totals["rejected"] == 0
                # per lap: the entry in slot sq - 2 and the one that closes the wave's post
                assert rs.sq_consumer_state(0, 0) == {"consumed": sq * (lap + 1), "cq_producer": 2 * (lap + 1)}
        finally:
            rs.sq_set_mode(False)
        mem.free()


def test_queue_mode_full_ring_raises_the_status_word_instead_of_hanging():
    n_pes, sq = 2, 64
    os.environ["ROC_SHMEM_WAIT_LIMIT_S"] = "0.02"                  # the producers' bounded wait
    try:
        rs.roc_shmem_init(n_pes, 4 << 20, 1, sq)
    finally:
        del os.environ["ROC_SHMEM_WAIT_LIMIT_S"]
    try:
        mem = rs.sym_array(4096, np.int64, fill=0)
        rs.sq_reset()
        rs.sq_set_mode(True)
        post_one_wave_per_ring(mem, n_pes, 1)
        assert rs.take_status() == 0
        post_one_wave_per_ring(mem, n_pes, 2)                       # nobody has retired anything
        assert rs.take_status() == 1, "a full queue must time out and say so"
        assert mem.read(1, 128)[2::4].tolist() == [2] * 32, "the operations themselves still ran"
        rs.sq_set_mode(False)
        mem.free()
    finally:
        rs.roc_shmem_finalize()


# ---- a consumer that runs while the producers post --------------------------------------

def put_and_add_stream(n_ops, n_pes, words, seed):
    """8-byte puts to distinct words of the lower halves, fetch-adds anywhere in the upper halves."""
    rng = np.random.default_rng(seed)
    ops = np.zeros(n_ops, rs.SMALL_OP_DTYPE)
    is_put = rng.random(n_ops) < 0.5
    uniq = rng.permutation(n_pes * (words // 2))[:n_ops]
    ops["kind"] = np.where(is_put, rs.OP_P64, rs.OP_FADD64)
    ops["pe"] = np.where(is_put, uniq // (words // 2), rng.integers(0, n_pes, n_ops))
    ops["offset"] = np.where(is_put, (uniq % (words // 2)) * 8,
                             (words // 2 + rng.integers(0, 256, n_ops)) * 8)
    ops["value"] = rng.integers(-(1 << 50), 1 << 50, n_ops)
    return ops


@pytest.mark.parametrize("wgs,wg_size,num_blocks,sq", [(2, 256, 2, 64), (6, 128, 2, 128), (1, 64, 1, 64)])
def test_live_consumer_retires_entries_while_producers_post(wgs, wg_size, num_blocks, sq):
    # Rings far smaller than what is posted through them (dozens of laps), several workgroups per
    # ring in the second shape, two producer kernels in one session: nothing may be lost, producers
    # must not time out, quiet must have collected every completion.
    n_pes, words, n_ops = 4, 1 << 15, 40000
    with runtime(n_pes, heap_size=8 << 20, num_blocks=num_blocks, sq_size=sq):
        mem = rs.sym_array(words, np.int64, fill=0)
        heap = oracle.Heap(n_pes, words * 8)
        stream = rs.Stream()
        rs.sq_reset()
        pacing = rs.get_pacing()
        rs.sq_consumer_start()
        assert rs.sq_consumer_running()
        assert rs.get_pacing() == (0, 0), "pacing rests while consumer waves hold compute units"
        devs = []
        try:
            with pytest.raises(rs.RocShmemError, match="live send-queue consumer"):
                rs.synchronize()
            with pytest.raises(rs.RocShmemError, match="live"):
                rs.sq_reset()
            for seed in (31, 32):
                ops = put_and_add_stream(n_ops, n_pes, words, seed)
                issue = Issue(n_ops, n_pes, wgs, wg_size, num_blocks)
                oracle.small_ops(heap, ops, issue.pe)
                shifted = ops.copy()
                shifted["offset"] += mem.offset
                devs.append(rs.device_array(shifted))
                rs.roc_shmem_small_ops(devs[-1], n_ops, None, rs.Launch(wgs, wg_size, 0, stream))
            stream.synchronize()
        finally:
            totals = rs.sq_consumer_stop()
        assert not rs.sq_consumer_running()
        assert rs.get_pacing() == pacing and pacing[1] != 0
        assert rs.take_status() == 0, "a producer's wait for queue space or a quiet gave up"
        # besides the operations, every workgroup's closing quiet posts one zero-byte read per launch
        quiets = 2 * n_pes * wgs
        assert totals["retired"] == 2 * n_ops + quiets and totals["lost"] == 0 and totals["rejected"] == 0
        assert totals["bytes"] == 16 * n_ops and totals["reads"] == quiets
        for p in range(n_pes):
            assert np.array_equal(mem.read(p), heap.view(p, 0, words, np.int64)), "heap of PE %d" % p
        for pe in range(n_pes):
            for block in range(num_blocks):
                st, cons, reader = rs.sq_state(pe, block), rs.sq_consumer_state(pe, block), rs.cq_reader_state(pe, block)
                assert st["published"] == st["sq_counter"] == cons["consumed"] > 4 * sq
                assert reader["quiet_counter"] == 0 and reader["cq_consumer"] == cons["cq_producer"]
                if wgs <= num_blocks:   # one workgroup per queue: its quiet wrote the record last
                    assert reader["cq_doorbell_record"] == cons["cq_producer"]
                # the newest completion entry: owner bit = lap parity of its number, the queue's number
                number = cons["cq_producer"] - 1
                cqe = rs.cq_image(pe, block, sq)[number % sq]
                assert cqe[63] == (number // sq) & 1 and not cqe[:56].any()
                assert bytes(cqe[57:60]) == rs.sq_constants(pe, block)["ctrl_qp_sq"].to_bytes(3, "little")
        # the previous mode is back: rings are logs again and a plain pass finds nothing left
        again = rs.sq_consume()
        assert again["retired"] == 0
        for d in devs:
            d.free()
        stream.destroy()
        mem.free()


def test_finalize_with_a_running_consumer_stops_it():
    rs.roc_shmem_init(2, 4 << 20, 1, 64)
    rs.sq_consumer_start()
    rs.roc_shmem_finalize()           # must tell the consumer to stop and wait for it, not hang
    rs.roc_shmem_init(2, 4 << 20, 1, 64)
    try:
        assert not rs.sq_consumer_running()
        rs.sq_consumer_start()
        assert rs.sq_consumer_stop()["retired"] == 0
        assert rs.take_status() == 0
    finally:
        rs.roc_shmem_finalize()


def test_calls_that_wait_for_the_whole_device_are_refused_while_a_consumer_runs():
    # Each of them would otherwise block until the consumer waves give up by themselves
    # (ROC_SHMEM_CONSUMER_IDLE_S, 5 s) and leave the live queues without a consumer.  They
    # return an error at once instead, and the consumer goes on serving its queues.
    import time
    rs.roc_shmem_init(2, 4 << 20, 2, 64)
    try:
        buf = rs.sym_array(1024, np.int64, fill=0)
        world = rs.roc_shmem_team_world()
        _, team = rs.roc_shmem_team_split_strided(world, 0, 1, 2)
        rs.sq_consumer_start()
        t0 = time.perf_counter()
        refused = [lambda: rs.synchronize(), lambda: rs.sq_reset(), lambda: rs.take_status(),
                   lambda: rs.set_pacing(0, 0), lambda: rs.sq_set_mode(1), lambda: rs.sq_consume(),
                   lambda: rs.sq_state(0, 0), lambda: rs.sq_read(0, 0, 0), lambda: rs.sq_image(0, 0, 4),
                   lambda: rs.cq_reader_state(0, 0), lambda: rs.sq_consumer_state(0, 0),
                   lambda: rs.cq_image(0, 0, 4), lambda: rs.atomic_ret_image(0, 0, 8),
                   lambda: rs.roc_shmem_free(buf.addr), lambda: rs.roc_shmem_team_destroy(team)]
        for call in refused:
            try:
                result = call()
            except rs.RocShmemError as e:
                assert "consumer" in str(e), str(e)
            else:
                assert result == -1, "call went through: %r" % (result,)   # take_status reports -1
        assert time.perf_counter() - t0 < 2.0         # nobody sat out the consumer's idle limit
        assert rs.sq_consumer_running()
        # the consumer is still there and still serves: a small stream goes through its queues
        stream = rs.Stream()
        ops = np.zeros(256, rs.SMALL_OP_DTYPE)
        ops["kind"] = rs.OP_P64
        ops["pe"] = np.arange(256) % 2
        ops["offset"] = buf.offset + (np.arange(256) // 2) * 8
        ops["value"] = np.arange(256) + 1
        dev = rs.device_array(ops)
        rs.roc_shmem_small_ops(dev, 256, None, rs.Launch(2, 64, 0, stream))
        stream.synchronize()
        totals = rs.sq_consumer_stop()
        assert totals["lost"] == 0 and totals["rejected"] == 0 and totals["retired"] >= 256
        assert rs.take_status() == 0
        for p in range(2):
            assert np.array_equal(buf.read(p)[:128], np.arange(256)[p::2] + 1)
        dev.free()
        stream.destroy()
        rs.roc_shmem_team_destroy(team)
        buf.free()
    finally:
        rs.roc_shmem_finalize()


def test_a_consumer_left_alone_leaves_by_itself():
    # Every wave of the persistent kernel reaches an exit whatever the host does: with nothing
    # published for ROC_SHMEM_CONSUMER_IDLE_S the waves leave; stop then says so.
    import time
    os.environ["ROC_SHMEM_CONSUMER_IDLE_S"] = "0.05"
    try:
        rs.roc_shmem_init(2, 4 << 20, 2, 64)
    finally:
        del os.environ["ROC_SHMEM_CONSUMER_IDLE_S"]
    try:
        rs.sq_consumer_start()
        time.sleep(0.5)
        with pytest.raises(rs.RocShmemError, match="had left before the stop request"):
            rs.sq_consumer_stop()
        assert not rs.sq_consumer_running()
        assert rs.take_status() == 0
    finally:
        rs.roc_shmem_finalize()
