"""CPU consumer of a send-queue ring (oracle/consume.c): hand-computed cases, rejection of
malformed entries, completion entries, and agreement with the small-operation model.

The reference's rings are consumed by a NIC, so it holds no vector for this; the consumer is
pinned by construction: entries built by the (separately checked) WQE builder from known
operations must replay to the memory image memcpy / the small-op model give for them.
"""
import numpy as np

import oracle

BASE = 0x7F12_0000_0000          # address the entries use for PE 0's heap
P, HEAP, STRIDE = 3, 4096, 8192   # 4 KiB of heap per PE, 4 KiB of padding between slices
RKEYS = np.array([int.from_bytes((0x1000 + p).to_bytes(4, "big"), "little") for p in range(P)],
                 dtype=np.uint32)


def make_qp(max_nwqe=64):
    qp = oracle.Qp()
    qp.ctrl_qp_sq = 0x00A1B2C3 & 0xFFFFFF
    qp.ctrl_sig = 0
    qp.lkey = 0x11223344
    qp.atomic_lkey = 0x55667788
    qp.atomic_ret_base = 0x7F55_0000_1000
    qp.max_nwqe = max_nwqe
    return qp


def addr(pe, off):
    return BASE + pe * STRIDE + off


class Ring:
    def __init__(self, qp):
        self.qp = qp
        self.image = np.zeros(qp.max_nwqe * 64, np.uint8)
        self.count = 0
        self.atomics = 0

    def slot(self, counter):
        k = counter % self.qp.max_nwqe
        return self.image[64 * k:64 * k + 64]

    def post(self, opcode, dest_pe, dest_off, cqe=False, **kw):
        if opcode in (oracle.OP_ATOMIC_FA, oracle.OP_ATOMIC_CS):
            kw["atomic_pos"] = self.atomics % 4096
            self.atomics += 1
        oracle.wqe_build(self.slot(self.count), self.qp, self.count, opcode,
                         raddr=addr(dest_pe, dest_off), rkey=int(RKEYS[dest_pe]), request_cqe=cqe, **kw)
        self.count += 1
        return self.count - 1


def consume(ring, target, sources, consumed=0, published=None, cq=None, cq_producer=0, ret=None):
    cq = np.full(ring.qp.max_nwqe * 64, 0, np.uint8) if cq is None else cq
    ret = np.zeros(4096, np.uint64) if ret is None else ret
    published = ring.count if published is None else published
    prod, totals = oracle.sq_consume(ring.qp, ring.image, consumed, published, BASE, STRIDE, HEAP, RKEYS,
                                     target, sources, ret, cq, cq_producer)
    return prod, totals.as_dict(), cq.reshape(-1, 64), ret


def fresh_arena(seed=0):
    rng = np.random.default_rng(seed)
    return rng.integers(0, 256, P * STRIDE, dtype=np.uint8)


def test_hand_computed_sequence():
    qp = make_qp()
    ring = Ring(qp)
    src = fresh_arena(1)
    tgt = src.copy()
    word = lambda a, pe, off: int(a[pe * STRIDE + off:pe * STRIDE + off + 8].view(np.uint64)[0])
    ring.post(oracle.OP_WRITE, 1, 16, size=8, inline=bytes(range(1, 9)))
    ring.post(oracle.OP_WRITE, 2, 1000, size=100, laddr=addr(0, 256))
    ring.post(oracle.OP_READ, 2, 1000, size=40, laddr=addr(0, 2048))
    ring.post(oracle.OP_ATOMIC_FA, 1, 16, size=8, atomic_data=5)
    after_add = (int.from_bytes(bytes(range(1, 9)), "little") + 5) & (2 ** 64 - 1)
    ring.post(oracle.OP_ATOMIC_CS, 1, 16, size=8, atomic_data=77, atomic_cmp=after_add)
    ring.post(oracle.OP_ATOMIC_CS, 1, 16, size=8, atomic_data=99, atomic_cmp=12345)   # mismatch
    ring.post(oracle.OP_WRITE, 0, 4092, size=4, inline=b"\xAA\xBB\xCC\xDD", cqe=True)

    expect = src.copy()
    expect[1 * STRIDE + 16:1 * STRIDE + 24] = np.arange(1, 9, dtype=np.uint8)
    expect[2 * STRIDE + 1000:2 * STRIDE + 1100] = src[256:356]
    expect[2048:2088] = src[256:296]                      # the read sees what entry 1 wrote
    expect[1 * STRIDE + 16:1 * STRIDE + 24] = np.frombuffer((77).to_bytes(8, "little"), np.uint8)
    expect[4092:4096] = [0xAA, 0xBB, 0xCC, 0xDD]

    prod, totals, cq, ret = consume(ring, tgt, src)
    assert np.array_equal(tgt, expect)
    assert word(tgt, 1, 16) == 77
    assert list(ret[:3]) == [after_add - 5, after_add, 77] and not ret[3:].any()
    assert totals == {"retired": 7, "writes": 3, "reads": 1, "atomics": 3, "bytes": 8 + 100 + 40 + 24 + 4,
                      "completions": 1, "lost": 0, "rejected": 0, "local_skipped": 0}
    assert prod == 1
    e = cq[0]
    assert not e[:56].any()
    assert bytes(e[56:60]) == b"\x00" + (qp.ctrl_qp_sq & 0xFFFFFF).to_bytes(3, "little")
    assert bytes(e[60:62]) == (6).to_bytes(2, "big") and e[62] == 0 and e[63] == 0
    assert not cq[1:].any()


def test_check_only_pass_moves_no_data():
    ring = Ring(make_qp())
    ring.post(oracle.OP_WRITE, 1, 0, size=8, inline=b"12345678", cqe=True)
    ring.post(oracle.OP_ATOMIC_FA, 2, 8, size=8, atomic_data=1, cqe=True)
    prod, totals, cq, ret = consume(ring, None, None)
    assert prod == 2 and totals["retired"] == 2 and totals["completions"] == 2 and not ret.any()
    assert [int(cq[i][61]) for i in range(2)] == [0, 1]


def corrupt(kind):
    qp = make_qp()
    ring = Ring(qp)
    s = ring.slot(0)
    if kind == "index":
        oracle.wqe_build(s, qp, 5, oracle.OP_WRITE, size=8, raddr=addr(1, 0), rkey=int(RKEYS[1]),
                         inline=b"abcdefgh")
        ring.count = 1
    elif kind == "rkey":
        oracle.wqe_build(s, qp, 0, oracle.OP_WRITE, size=8, raddr=addr(1, 0), rkey=int(RKEYS[2]),
                         inline=b"abcdefgh")
        ring.count = 1
    elif kind == "padding":          # between two heaps
        ring.post(oracle.OP_WRITE, 0, HEAP + 8, size=8, inline=b"abcdefgh")
    elif kind == "straddle":         # starts inside the heap, ends outside
        ring.post(oracle.OP_WRITE, 1, HEAP - 4, size=8, inline=b"abcdefgh")
    elif kind == "beyond":
        oracle.wqe_build(s, qp, 0, oracle.OP_WRITE, size=8, raddr=BASE + P * STRIDE, rkey=int(RKEYS[0]),
                         inline=b"abcdefgh")
        ring.count = 1
    elif kind == "below":
        oracle.wqe_build(s, qp, 0, oracle.OP_WRITE, size=8, raddr=BASE - 64, rkey=int(RKEYS[0]),
                         inline=b"abcdefgh")
        ring.count = 1
    elif kind == "ds":
        ring.post(oracle.OP_WRITE, 1, 0, size=8, inline=b"abcdefgh")
        s[7] = 4
    elif kind == "opcode":
        ring.post(oracle.OP_WRITE, 1, 0, size=8, inline=b"abcdefgh")
        s[3] = 0x0A
    elif kind == "queue":
        ring.post(oracle.OP_WRITE, 1, 0, size=8, inline=b"abcdefgh")
        s[5] ^= 0x40
    elif kind == "misaligned_atomic":
        ring.post(oracle.OP_ATOMIC_FA, 1, 12, size=8, atomic_data=1)
    elif kind == "return_slot":
        ring.post(oracle.OP_ATOMIC_FA, 1, 8, size=8, atomic_data=1)
        s[56:64] = np.frombuffer((qp.atomic_ret_base + 8 * 4096).to_bytes(8, "big"), np.uint8)
    elif kind == "lkey":
        ring.post(oracle.OP_WRITE, 1, 0, size=64, laddr=addr(0, 0))
        s[36] ^= 1
    elif kind == "long_inline":
        ring.post(oracle.OP_WRITE, 1, 0, size=8, inline=b"abcdefgh")
        s[32:36] = np.frombuffer((0x80000000 | 13).to_bytes(4, "big"), np.uint8)
    return ring


def test_malformed_entries_are_retired_but_never_executed():
    for kind in ("index", "rkey", "padding", "straddle", "beyond", "below", "ds", "opcode", "queue",
                 "misaligned_atomic", "return_slot", "lkey", "long_inline"):
        ring = corrupt(kind)
        src = fresh_arena(2)
        tgt = src.copy()
        prod, totals, cq, ret = consume(ring, tgt, src)
        assert totals["retired"] == 1 and totals["rejected"] == 1, kind
        assert totals["writes"] + totals["reads"] + totals["atomics"] + totals["bytes"] == 0, kind
        assert np.array_equal(tgt, src) and not ret.any(), kind


def test_local_buffer_outside_the_heap_is_skipped():
    ring = Ring(make_qp())
    oracle.wqe_build(ring.slot(0), ring.qp, 0, oracle.OP_WRITE, size=64, raddr=addr(1, 0),
                     rkey=int(RKEYS[1]), laddr=0x1000)
    ring.count = 1
    src = fresh_arena(3)
    tgt = src.copy()
    _, totals, _, _ = consume(ring, tgt, src)
    assert totals["local_skipped"] == 1 and totals["writes"] == 1 and totals["rejected"] == 0
    assert np.array_equal(tgt, src)


def test_entries_overwritten_before_the_pass_are_counted_as_lost():
    ring = Ring(make_qp(max_nwqe=64))
    for i in range(150):                                  # wraps twice; the last 64 survive
        ring.post(oracle.OP_WRITE, i % P, 8 * (i % 256), size=8, inline=i.to_bytes(8, "little"))
    src = np.zeros(P * STRIDE, np.uint8)
    tgt = src.copy()
    _, totals, _, _ = consume(ring, tgt, src)
    assert totals["lost"] == 150 - 64 and totals["retired"] == 64 and totals["rejected"] == 0
    for i in range(150 - 64, 150):
        off = (i % P) * STRIDE + 8 * (i % 256)
        assert int(tgt[off:off + 8].view(np.uint64)[0]) == i


def test_owner_bit_flips_on_every_lap_of_the_completion_queue():
    qp = make_qp(max_nwqe=64)
    ring = Ring(qp)
    cq = np.zeros(64 * 64, np.uint8)
    cq[63::64] = 0xF0
    prod = 0
    consumed = 0
    for lap in range(3):
        for _ in range(64):
            ring.post(oracle.OP_WRITE, 0, 0, size=4, inline=b"wxyz", cqe=True)
        prod, totals, view, _ = consume(ring, None, None, consumed=consumed, cq=cq, cq_producer=prod)
        consumed = ring.count
        assert totals["completions"] == 64 and prod == 64 * (lap + 1)
        assert (view[:, 63] == (lap & 1)).all()
        counters = [int.from_bytes(bytes(view[i][60:62]), "big") for i in range(64)]
        assert counters == [(64 * lap + i) & 0xFFFF for i in range(64)]


def test_hand_assembled_completion_entries():
    # tests/golden/wqe_hand_assembled.json: completion entries written out by hand.
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                           "wqe_hand_assembled.json")) as f:
        g = json.load(f)
    assert len(g["completions"]) >= 2
    for e in g["completions"]:
        qp = make_qp(max_nwqe=1024)
        qp.ctrl_qp_sq = int.from_bytes(bytes.fromhex(e["qpn_bytes"]), "little")
        ring = Ring(qp)
        ring.count = e["wqe_index"]                       # the entry sits at this stream position
        ring.post(oracle.OP_WRITE, 0, 0, size=4, inline=b"abcd", cqe=True)
        cq = np.zeros(e["cq_size"] * 64, np.uint8)
        cq[63::64] = 0xF0
        prod, totals, view, _ = consume(ring, None, None, consumed=e["wqe_index"], cq=cq,
                                        cq_producer=e["cq_producer"])
        assert prod == e["cq_producer"] + 1 and totals["rejected"] == 0
        want = bytes.fromhex("".join(e["bytes"]).replace(" ", ""))
        assert bytes(view[e["cq_producer"] % e["cq_size"]]) == want, e["name"]


def test_replay_agrees_with_the_small_operation_model():
    # The same random stream through (a) the small-op model and (b) builder -> ring -> consumer.
    rng = np.random.default_rng(11)
    n = 600
    words = HEAP // 8
    kinds = rng.choice([oracle.OP_P64, oracle.OP_FADD64, oracle.OP_ADD64, oracle.OP_FINC64, oracle.OP_INC64,
                        oracle.OP_CSWAP64, oracle.OP_FETCH64, oracle.OP_P32], n)
    ops = np.zeros(n, oracle.SMALL_OP_DTYPE)
    ops["kind"] = kinds
    ops["pe"] = rng.integers(0, P, n)
    ops["offset"] = rng.integers(0, 32, n) * 8            # few targets: plenty of collisions
    ops["value"] = rng.integers(-(1 << 40), 1 << 40, n)
    ops["aux"] = rng.integers(-3, 3, n)
    heap = oracle.Heap(P, STRIDE)
    heap.buf[:] = fresh_arena(5)
    for p in range(P):                                     # small values so that cswap sometimes hits
        heap.view(p, 0, 32, np.int64)[:] = rng.integers(-3, 3, 32)
    src = heap.buf.copy()
    tgt = heap.buf.copy()
    issuer = np.zeros(n, np.uint32)
    fetched = oracle.small_ops(heap, ops, issuer)

    qp = make_qp(max_nwqe=1024)
    ring = Ring(qp)
    u64 = lambda v: int(v) & (2 ** 64 - 1)
    slots = {}
    for i, op in enumerate(ops):
        k, pe, off, v = int(op["kind"]), int(op["pe"]), int(op["offset"]), int(op["value"])
        if k == oracle.OP_P64:
            ring.post(oracle.OP_WRITE, pe, off, size=8, inline=u64(v).to_bytes(8, "little"))
        elif k == oracle.OP_P32:
            ring.post(oracle.OP_WRITE, pe, off, size=4, inline=(v & 0xFFFFFFFF).to_bytes(4, "little"))
        elif k == oracle.OP_CSWAP64:
            slots[i] = ring.atomics
            ring.post(oracle.OP_ATOMIC_CS, pe, off, size=8, atomic_data=u64(v), atomic_cmp=u64(op["aux"]))
        else:
            operand = {oracle.OP_FADD64: v, oracle.OP_ADD64: v, oracle.OP_FINC64: 1, oracle.OP_INC64: 1,
                       oracle.OP_FETCH64: 0}[k]
            slots[i] = ring.atomics
            ring.post(oracle.OP_ATOMIC_FA, pe, off, size=8, atomic_data=u64(operand))
    _, totals, _, ret = consume(ring, tgt, src)
    assert totals["rejected"] == 0 and totals["retired"] == n
    assert np.array_equal(tgt, heap.buf)
    for i, pos in slots.items():
        if int(ops["kind"][i]) in (oracle.OP_FADD64, oracle.OP_FINC64, oracle.OP_CSWAP64, oracle.OP_FETCH64):
            assert int(ret[pos]) == u64(fetched[i]), i


# ---- the two entries that move no data: quiet's zero-byte read, fence's flush write -------------

FLUSH_BASE = 0x7F77_0000_0400
FLUSH_RKEYS = np.array([int.from_bytes((0x4000 + p).to_bytes(4, "big"), "little") for p in range(P)],
                       dtype=np.uint32)


def consume_with_flush(ring, target, sources):
    cq = np.zeros(ring.qp.max_nwqe * 64, np.uint8)
    ret = np.zeros(4096, np.uint64)
    prod, totals = oracle.sq_consume(ring.qp, ring.image, 0, ring.count, BASE, STRIDE, HEAP, RKEYS, target,
                                     sources, ret, cq, 0, flush_base=FLUSH_BASE, flush_rkeys=FLUSH_RKEYS)
    return prod, totals.as_dict(), cq.reshape(-1, 64)


def post_raw(ring, opcode, raddr, rkey, cqe=False, **kw):
    oracle.wqe_build(ring.slot(ring.count), ring.qp, ring.count, opcode, raddr=raddr, rkey=rkey,
                     request_cqe=cqe, **kw)
    ring.count += 1


def test_zero_byte_read_and_flush_write_are_completed_and_change_nothing():
    ring = Ring(make_qp())
    ring.image[:] = 0xEE                        # what older entries may have left in the slots
    src = fresh_arena(3)
    tgt = src.copy()
    ring.post(oracle.OP_WRITE, 1, 64, size=8, inline=b"ABCDEFGH")
    post_raw(ring, oracle.OP_WRITE, FLUSH_BASE + 64 * 2, int(FLUSH_RKEYS[2]), cqe=True, form=oracle.WQE_FLUSH_WRITE)
    post_raw(ring, oracle.OP_READ, addr(1, 0), int(RKEYS[1]), cqe=True, form=oracle.WQE_ZERO_BYTE_READ)
    prod, totals, cq = consume_with_flush(ring, tgt, src)
    expect = src.copy()
    expect[STRIDE + 64:STRIDE + 72] = np.frombuffer(b"ABCDEFGH", np.uint8)
    assert np.array_equal(tgt, expect)
    assert totals == {"retired": 3, "writes": 2, "reads": 1, "atomics": 0, "bytes": 8 + 4 + 0,
                      "completions": 2, "lost": 0, "rejected": 0, "local_skipped": 0}
    assert prod == 2 and [int(cq[i][61]) for i in range(2)] == [1, 2]
    # the zero-byte read's third and fourth segments are whatever the slot held
    assert (ring.slot(2)[32:] == 0xEE).all() and ring.slot(2)[7] == 2


def test_malformed_no_data_entries_are_rejected():
    def one(build):
        ring = Ring(make_qp())
        build(ring)
        _, totals, _ = consume_with_flush(ring, None, None)
        return totals["rejected"], totals["retired"]

    good = [
        lambda r: post_raw(r, oracle.OP_READ, addr(2, 0), int(RKEYS[2]), form=oracle.WQE_ZERO_BYTE_READ),
        lambda r: post_raw(r, oracle.OP_WRITE, FLUSH_BASE, int(FLUSH_RKEYS[0]), form=oracle.WQE_FLUSH_WRITE),
    ]
    for g in good:
        assert one(g) == (0, 1)

    def ds2_write(r):        # DS = 2 on anything but a read
        post_raw(r, oracle.OP_WRITE, addr(0, 0), int(RKEYS[0]), size=4, inline=b"abcd")
        r.slot(0)[7] = 2

    def read_wrong_key(r):
        post_raw(r, oracle.OP_READ, addr(2, 0), int(RKEYS[1]), form=oracle.WQE_ZERO_BYTE_READ)

    def read_outside(r):
        post_raw(r, oracle.OP_READ, BASE + P * STRIDE, int(RKEYS[0]), form=oracle.WQE_ZERO_BYTE_READ)

    def flush_heap_key(r):   # a flush word named under a heap key
        post_raw(r, oracle.OP_WRITE, FLUSH_BASE + 64, int(RKEYS[1]), form=oracle.WQE_FLUSH_WRITE)

    def flush_other_pe_key(r):
        post_raw(r, oracle.OP_WRITE, FLUSH_BASE + 64, int(FLUSH_RKEYS[2]), form=oracle.WQE_FLUSH_WRITE)

    def flush_misaligned(r):
        post_raw(r, oracle.OP_WRITE, FLUSH_BASE + 68, int(FLUSH_RKEYS[1]), form=oracle.WQE_FLUSH_WRITE)

    def flush_wrong_payload(r):
        post_raw(r, oracle.OP_WRITE, FLUSH_BASE, int(FLUSH_RKEYS[0]), form=oracle.WQE_FLUSH_WRITE)
        r.slot(0)[36] = 0

    def flush_wrong_size(r):
        post_raw(r, oracle.OP_WRITE, FLUSH_BASE, int(FLUSH_RKEYS[0]), size=8, inline=b"\x01" + bytes(7))

    def flush_beyond_the_last_pe(r):
        post_raw(r, oracle.OP_WRITE, FLUSH_BASE + 64 * P, int(FLUSH_RKEYS[0]), form=oracle.WQE_FLUSH_WRITE)

    for bad in (ds2_write, read_wrong_key, read_outside, flush_heap_key, flush_other_pe_key, flush_misaligned,
                flush_wrong_payload, flush_wrong_size, flush_beyond_the_last_pe):
        assert one(bad) == (1, 1), bad.__name__
