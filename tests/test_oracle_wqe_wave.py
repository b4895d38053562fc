"""The oracle's WQE builder and wave-level models.

The reference holds no test or fixture for WQE bytes (parity unpinned); the checks
here are what the entry format itself fixes, plus three entries assembled by hand from the
field table of the format."""
import itertools
import json
import os

import numpy as np

import oracle


def qp(ctrl_qp_sq=0x030201, ctrl_sig=0, lkey=0x00200000, atomic_lkey=0x00300000,
       ret_base=0x7F0000001000, n=1024):
    q = oracle.Qp()
    q.ctrl_qp_sq, q.ctrl_sig, q.lkey, q.atomic_lkey = ctrl_qp_sq, ctrl_sig, lkey, atomic_lkey
    q.atomic_ret_base, q.max_nwqe = ret_base, n
    return q


def golden():
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                           "wqe_hand_assembled.json")) as f:
        return json.load(f)


def num(v):
    return int(v, 0) if isinstance(v, str) else int(v)


def test_hand_assembled_entries():
    # Entries written out by hand from the entry format (tests/golden/wqe_hand_assembled.json).
    g = golden()
    q = g["queue"]
    queue = qp(num(q["ctrl_qp_sq"]), num(q["ctrl_sig"]), num(q["lkey"]), num(q["atomic_lkey"]),
               num(q["atomic_ret_base"]), num(q["max_nwqe"]))
    assert len(g["entries"]) >= 6 and {e.get("form", 0) for e in g["entries"]} == {0, 1, 2}
    for e in g["entries"]:
        slot = np.full(64, int(e["background"], 16), np.uint8)
        oracle.wqe_build(slot, queue, num(e["counter"]), num(e["opcode"]), size=e["size"],
                         raddr=num(e["raddr"]), rkey=num(e["rkey"]), laddr=num(e.get("laddr", 0)),
                         atomic_data=num(e.get("atomic_data", 0)), atomic_cmp=num(e.get("atomic_cmp", 0)),
                         inline=bytes.fromhex(e.get("inline", "")), atomic_pos=e.get("atomic_pos", 0),
                         request_cqe=e["cqe"], form=e.get("form", oracle.WQE_DATA))
        want = bytes.fromhex("".join(e["bytes"]).replace(" ", ""))
        assert len(want) == 64
        assert bytes(slot) == want, e["name"]


def test_format_invariants():
    rng = np.random.default_rng(0)
    for _ in range(200):
        counter = int(rng.integers(0, 1 << 32))
        opcode = int(rng.choice([oracle.OP_WRITE, oracle.OP_READ, oracle.OP_ATOMIC_CS, oracle.OP_ATOMIC_FA]))
        size = int(rng.choice([1, 3, 4, 8, 9, 64, 1 << 20]))
        raddr = int(rng.integers(0, 1 << 48))
        laddr = int(rng.integers(0, 1 << 48))
        data = int(rng.integers(-(1 << 62), 1 << 62))
        q = qp(ctrl_sig=int(rng.integers(0, 1 << 62)))
        before = rng.integers(0, 256, 64, dtype=np.uint8)
        slot = before.copy()
        cqe = bool(rng.integers(0, 2))
        oracle.wqe_build(slot, q, counter, opcode, size=size, raddr=raddr, rkey=0x11223344, laddr=laddr,
                         atomic_data=data, atomic_cmp=5, inline=bytes(range(8)), atomic_pos=9, request_cqe=cqe)
        atomic = opcode in (oracle.OP_ATOMIC_CS, oracle.OP_ATOMIC_FA)
        inline = opcode == oracle.OP_WRITE and size <= 8
        assert slot[0] == 0 and slot[3] == opcode
        assert int.from_bytes(bytes(slot[1:3]), "big") == counter & 0xFFFF          # 16-bit index, big-endian
        assert slot[7] == (4 if atomic else 3)                                       # DS = 16-byte segments
        assert slot[11] == (8 if cqe else (q.ctrl_sig >> 24) & 0xFF)                 # completion byte
        assert slot[8] == q.ctrl_sig & 0xFF
        assert int.from_bytes(bytes(slot[12:16]), "little") == q.ctrl_sig >> 32
        assert int.from_bytes(bytes(slot[16:24]), "big") == raddr                    # big-endian address
        assert oracle.wqe_raddr(slot) == raddr and oracle.wqe_index(slot) == counter & 0xFFFF
        assert oracle.wqe_opcode(slot) == opcode
        assert np.array_equal(slot[9:11], before[9:11]) and np.array_equal(slot[28:32], before[28:32])
        if atomic:
            assert int.from_bytes(bytes(slot[32:40]), "big") == data & 0xFFFFFFFFFFFFFFFF
            assert int.from_bytes(bytes(slot[40:48]), "big") == 5
            assert int.from_bytes(bytes(slot[48:52]), "big") == 8
            assert int.from_bytes(bytes(slot[56:64]), "big") == q.atomic_ret_base + 72
        elif inline:
            bc = int.from_bytes(bytes(slot[32:36]), "big")
            assert bc >> 31 == 1 and bc & 0x3FF == size                              # inline flag is bit 31
            assert bytes(slot[36:36 + size]) == bytes(range(size))
            assert np.array_equal(slot[36 + size:], before[36 + size:])              # the rest survives
        else:
            assert int.from_bytes(bytes(slot[32:36]), "big") == size
            assert int.from_bytes(bytes(slot[40:48]), "big") == laddr
            assert np.array_equal(slot[48:], before[48:])                            # segment 3 survives
    # byte swaps are involutions and agree with int.from_bytes
    for v in (0, 1, 0x1234, 0xFFFF):
        assert oracle.bswap16(oracle.bswap16(v)) == v
        assert oracle.bswap16(v) == int.from_bytes(v.to_bytes(2, "little"), "big")
    for v in (0, 0x12345678, 0xFFFFFFFF, 0x80000001):
        assert oracle.bswap32(oracle.bswap32(v)) == v
        assert oracle.bswap32(v) == int.from_bytes(v.to_bytes(4, "little"), "big")
    for v in (0, 0x0123456789ABCDEF, 1 << 63):
        assert oracle.bswap64(oracle.bswap64(v)) == v
        assert oracle.bswap64(v) == int.from_bytes(v.to_bytes(8, "little"), "big")
    # doorbell record = counter big-endian; doorbell value = first eight bytes of the entry
    slot = np.arange(64, dtype=np.uint8)
    mb = oracle.doorbell(slot, 0x01020304)
    assert bytes(mb.view(np.uint8)[:8]) == bytes([1, 2, 3, 4, 0, 0, 0, 0])
    assert bytes(mb.view(np.uint8)[8:]) == bytes(range(8))


def brute_coalesce(mask, pe, src, dst, size, lanes):
    """Independent formulation: maximal runs of chained lanes; the head of a run sends for all of it."""
    must, out = {}, {}
    l = 0
    while l < lanes:
        if not (mask >> l) & 1:
            l += 1
            continue
        run = 1
        while (l + run < lanes and (mask >> (l + run)) & 1 and size[l + run] == size[l + run - 1]
               and pe[l + run] == pe[l + run - 1] and src[l + run] == src[l + run - 1] + size[l + run]
               and dst[l + run] == dst[l + run - 1] + size[l + run]):
            run += 1
        must[l], out[l] = 1, size[l] * run
        for k in range(1, run):
            must[l + k], out[l + k] = 0, size[l + k]
        l += run
    return must, out


def test_coalesce_documented_example_and_brute_force():
    # library/src/wf_coal_policy.cpp:39-53: lanes 0-8 chain, lane 9 alone, lanes 10-63 chain -> 3 messages
    pe = np.ones(64, np.int32)
    size = np.full(64, 8, np.uint64)
    src = np.zeros(64, np.uint64)
    dst = np.zeros(64, np.uint64)
    for l in range(64):
        group = 0 if l <= 8 else (1 if l == 9 else 2)
        src[l] = 0x1000 * (group + 1) + 8 * l
        dst[l] = 0x100000 * (group + 1) + 8 * l
    must, out = oracle.coalesce(0xFFFFFFFFFFFFFFFF, pe, src, dst, size)
    assert list(np.nonzero(must)[0]) == [0, 9, 10]
    assert (out[0], out[9], out[10]) == (72, 8, 432)
    # exhaustive on 8-lane miniatures: every active mask x every chaining pattern of neighbours
    for mask in range(1, 256):
        for links in itertools.product((0, 1), repeat=7):
            pe = np.zeros(64, np.int32)
            size = np.full(64, 4, np.uint64)
            src = np.zeros(64, np.uint64)
            dst = np.zeros(64, np.uint64)
            for l in range(1, 8):
                step = 4 if links[l - 1] else 40
                src[l] = src[l - 1] + step
                dst[l] = dst[l - 1] + step
            must, out = oracle.coalesce(mask, pe, src, dst, size)
            bm, bo = brute_coalesce(mask, pe, src, dst, size, 8)
            for l in range(8):
                if (mask >> l) & 1:
                    assert must[l] == bm[l] and out[l] == bo[l], (mask, links, l)
    # a different PE, size or discontiguous source breaks the chain
    pe = np.zeros(64, np.int32)
    size = np.full(64, 8, np.uint64)
    src = np.arange(64, dtype=np.uint64) * 8
    dst = np.arange(64, dtype=np.uint64) * 8 + 4096
    pe[5] = 1
    size[20] = 16
    src[40] += 8
    must, _ = oracle.coalesce(0xFFFFFFFFFFFFFFFF, pe, src, dst, size)
    assert list(np.nonzero(must)[0]) == [0, 5, 6, 20, 21, 40, 41]


def test_fetch_incr_known_answers():
    # clients/unit_tests/bitwise_gtest.cpp:1384-1526
    for mask, total in ((0xA, 2), (0xFFFFFFFFFFFFFFFF, 64), (0xFFFFFFFF00000000, 32),
                        (0xF0F0F0F0F0F0F0F0, 32)):
        out, counter = oracle.fetch_incr(mask, 0)
        assert counter == total
        active = [l for l in range(64) if (mask >> l) & 1]
        assert [int(out[l]) for l in active] == list(range(total))
        assert all(out[l] == 0xFFFFFFFFFFFFFFFF for l in range(64) if l not in active)
    # 1024 x 1024 threads -> 1048576; the second active lane of a wave always sees base + 1
    counter = 0
    for _ in range(1024 * 1024 // 64):
        out, counter = oracle.fetch_incr(0xFFFFFFFFFFFFFFFF, counter)
        assert out[1] % 64 == 1
    assert counter == 1048576


# ---- the bulk ring checker used by the full-size GPU tests ---------------------------------

BASE0, STRIDE, N_PES = 0x7F1000000000, 1 << 26, 4
RKEYS = [oracle.bswap32(0x1000 + p) for p in range(N_PES)]


def ring_of(q, ops, first_counter=0, closes=64, background=0):
    """Ring image the scalar builder leaves for `ops` = [(opcode, raddr, data, cmp, size)] posted
    in that order from running number first_counter; every `closes`-th entry closes a post."""
    ring = np.full((q.max_nwqe, 64), background, np.uint8)
    n_atomic = 0
    for k, (opcode, raddr, data, cmp_, size) in enumerate(ops):
        c = first_counter + k
        pos = 0
        if opcode in (oracle.OP_ATOMIC_FA, oracle.OP_ATOMIC_CS):
            pos = n_atomic % 4096
            n_atomic += 1
        oracle.wqe_build(ring[c % q.max_nwqe], q, c, opcode, size=size, raddr=raddr,
                         rkey=RKEYS[(raddr - BASE0) // STRIDE], atomic_data=data, atomic_cmp=cmp_,
                         inline=(data & (2 ** 64 - 1)).to_bytes(8, "little"), atomic_pos=pos,
                         request_cqe=oracle.requests_cqe(c, q.max_nwqe, (k + 1) % closes == 0 or k == len(ops) - 1))
    return ring


def expect_of(ops):
    e = np.zeros(len(ops), oracle.WQE_EXPECT_DTYPE)
    for k, (opcode, raddr, data, cmp_, size) in enumerate(ops):
        e[k] = (raddr, data & (2 ** 64 - 1), cmp_ & (2 ** 64 - 1), opcode, size)
    return oracle.sort_wqe_expect(e)


def random_ops(rng, n):
    ops = []
    for k in range(n):
        pe = int(rng.integers(0, N_PES))
        raddr = BASE0 + pe * STRIDE + 8 * int(rng.integers(0, 50))     # collisions on purpose
        kind = int(rng.integers(0, 3))
        if kind == 0:
            ops.append((oracle.OP_WRITE, raddr, int(rng.integers(0, 1 << 63)), 0, int(rng.choice([4, 8]))))
            if ops[-1][4] == 4:
                ops[-1] = ops[-1][:2] + (ops[-1][2] & 0xFFFFFFFF,) + ops[-1][3:]
        elif kind == 1:
            ops.append((oracle.OP_ATOMIC_FA, raddr, int(rng.integers(0, 4)), 0, 8))
        else:
            ops.append((oracle.OP_ATOMIC_CS, raddr, int(rng.integers(0, 1 << 40)), int(rng.integers(0, 3)), 8))
    return ops


def run_check(q, ring, first, count, expect, full):
    return oracle.ring_check(ring, q, first, count, expect, BASE0, STRIDE, STRIDE, RKEYS, full_slot=full)


def test_ring_check_accepts_what_the_builder_writes_and_counts():
    rng = np.random.default_rng(21)
    q = qp(n=256)
    ops = random_ops(rng, 200)
    ring = ring_of(q, ops, closes=64)
    res = run_check(q, ring, 0, len(ops), expect_of(ops), full=True)
    assert res["ok"], res
    assert res["used"].all()
    n_atomic = sum(1 for o in ops if o[0] != oracle.OP_WRITE)
    assert res["n_atomic"] == n_atomic and res["pos_count"][:n_atomic].tolist() == [1] * n_atomic
    assert res["n_cqe"] == 4                    # entries 63, 127, 191 and the last one (199)
    # a ring that wrapped: leftover bytes of older entries are not compared, the newest 256 are checked
    ops = random_ops(rng, 700)
    ring = ring_of(q, ops, closes=64, background=0)
    assert not run_check(q, ring, 700 - 256, 256, expect_of(ops), full=True)["ok"]
    res = run_check(q, ring, 700 - 256, 256, expect_of(ops), full=False)
    assert res["ok"] and res["used"].sum() == 256


def test_ring_check_catches_each_kind_of_damage():
    rng = np.random.default_rng(22)
    q = qp(n=256)
    ops = random_ops(rng, 255)
    ops[254] = (oracle.OP_WRITE, BASE0 + 3 * STRIDE + 4096, 0x1122334455667788, 0, 8)
    ops[100] = (oracle.OP_ATOMIC_FA, BASE0 + 2 * STRIDE + 8192, 7, 0, 8)
    good = ring_of(q, ops, closes=64)
    expect = expect_of(ops)
    assert run_check(q, good, 0, 255, expect, True)["ok"]

    def damaged(slot, byte, value=None, xor=None):
        ring = good.copy()
        ring[slot, byte] = value if value is not None else ring[slot, byte] ^ xor
        return run_check(q, ring, 0, 255, expect, True)

    assert damaged(7, 2, xor=1)["reason"] == "index field"
    assert damaged(7, 3, value=0x10)["reason"] == "opcode"
    assert damaged(100, 63, xor=4)["reason"] == "AMO return slot outside the window"   # misaligned
    assert damaged(100, 57, xor=0x80)["reason"] == "AMO return slot outside the window"
    assert damaged(254, 32, value=0)["reason"] == "not an inline write of 1..8 bytes"
    assert damaged(9, 11, value=3)["reason"] == "completion flag"
    assert damaged(254, 11, value=0)["reason"] == "completion flag"                     # slot max_nwqe - 2
    r = damaged(254, 40, xor=0x10)                                                      # payload byte
    assert r["reason"].startswith("no operation") and r["position"] == 254
    assert damaged(100, 23, xor=8)["reason"].startswith("no operation")                 # remote address
    for byte in (4, 7, 8, 12, 24, 27):                                                  # qpn, DS, sig, imm, rkey
        r = damaged(100, byte, xor=0x21)
        assert not r["ok"] and r["reason"] == "bytes differ from the builder's" and r["position"] == 100
    for byte in (48, 52):                                                               # AMO data segment
        assert damaged(100, byte, xor=1)["reason"] == "bytes differ from the builder's"
    assert damaged(254, 50, value=9)["reason"] == "bytes differ from the builder's"     # must stay zero
    # an entry that appears twice, an operation that is missing from the list
    ring = good.copy()
    ring[10] = ring[254]
    ring[10, 1:3] = [0, 10]
    r = run_check(q, ring, 0, 255, expect, True)
    assert not r["ok"]
    r = run_check(q, good, 0, 255, expect_of(ops[:100] + ops[101:]), True)
    assert r["reason"].startswith("no operation") and r["position"] == 100


def test_ring_check_knows_the_two_entries_that_move_no_data():
    # quiet's zero-byte read and fence's flush write among ordinary entries, on a ring that has
    # wrapped (leftover bytes in the segments those entries do not write)
    flush_base = 0x7F2000000400
    flush_rkeys = [oracle.bswap32(0x4000 + p) for p in range(N_PES)]
    rng = np.random.default_rng(23)
    q = qp(n=64)
    ops = random_ops(rng, 40)
    ring = ring_of(q, ops, background=0xEE)
    zero_read = (oracle.OP_READ, BASE0 + 2 * STRIDE, 0, 0, 0)
    flush = (oracle.OP_WRITE, flush_base + 64 * 3, 1, 0, 4)
    oracle.wqe_build(ring[40], q, 40, oracle.OP_WRITE, raddr=flush[1], rkey=flush_rkeys[3],
                     form=oracle.WQE_FLUSH_WRITE, request_cqe=True)
    oracle.wqe_build(ring[41], q, 41, oracle.OP_READ, raddr=zero_read[1], rkey=RKEYS[2],
                     form=oracle.WQE_ZERO_BYTE_READ, request_cqe=True)
    expect = expect_of(ops + [flush, zero_read])

    def check(image, exp=expect, **kw):
        return oracle.ring_check(image, q, 0, 42, exp, BASE0, STRIDE, STRIDE, RKEYS, full_slot=False,
                                 flush_base=flush_base, flush_rkeys=flush_rkeys, **kw)

    res = check(ring)
    assert res["ok"] and res["used"].all(), res
    assert not check(ring, expect_of(ops + [flush]))["ok"]                      # an entry nobody posted
    for slot, byte, value, reason in ((41, 7, 3, "opcode"),                     # a read that moves data
                                      (41, 24, 0x55, "bytes differ from the builder's"),   # its key
                                      (40, 36, 0, "no operation"),              # the flush value
                                      (40, 35, 8, "not an inline write of 1..8 bytes"),    # its size
                                      (40, 27, 0x10, "bytes differ from the builder's")):  # heap key, not flush key
        bad = ring.copy()
        bad[slot, byte] = value
        r = check(bad)
        assert not r["ok"] and r["reason"].startswith(reason) and r["position"] == slot, (slot, byte, r)
    # without the flush words declared, a write to one of them is outside every heap
    r = oracle.ring_check(ring, q, 0, 42, expect, BASE0, STRIDE, STRIDE, RKEYS, full_slot=False)
    assert not r["ok"] and r["position"] == 40


def test_bulk_builder_and_threaded_small_ops_agree_with_the_scalar_forms():
    rng = np.random.default_rng(23)
    q = qp(n=64)
    ops = random_ops(rng, 300)
    reqs = (oracle.WqeReq * len(ops))()
    ring_a = np.zeros((64, 64), np.uint8)
    for k, (opcode, raddr, data, cmp_, size) in enumerate(ops):
        r = reqs[k]
        r.opcode, r.size, r.raddr, r.rkey = opcode, size, raddr, RKEYS[(raddr - BASE0) // STRIDE]
        r.atomic_data, r.atomic_cmp, r.atomic_pos, r.request_cqe = data, cmp_, k % 4096, int(k % 7 == 0)
        for i, b in enumerate((data & (2 ** 64 - 1)).to_bytes(8, "little")):
            r.inline_bytes[i] = b
        oracle.wqe_build(ring_a[(5 + k) % 64], q, 5 + k, opcode, size=size, raddr=raddr, rkey=r.rkey,
                         atomic_data=data, atomic_cmp=cmp_, inline=bytes(r.inline_bytes), atomic_pos=k % 4096,
                         request_cqe=bool(r.request_cqe))
    ring_b = np.zeros((64, 64), np.uint8)
    oracle.wqe_build_many(ring_b, q, 5, reqs)
    assert np.array_equal(ring_a, ring_b)
    # threaded puts + fetch-adds leave the heap the sequential model leaves
    n_pes, words = 4, 4096
    n = n_pes * (words // 2)                      # puts get distinct words of the lower halves
    stream = np.zeros(n, oracle.SMALL_OP_DTYPE)
    is_put = rng.random(n) < 0.5
    stream["kind"] = np.where(is_put, oracle.OP_P64, oracle.OP_FADD64)
    uniq = rng.permutation(n)
    stream["pe"] = np.where(is_put, uniq // (words // 2), rng.integers(0, n_pes, len(stream)))
    stream["offset"] = np.where(is_put, (uniq % (words // 2)) * 8,
                                (words // 2 + rng.integers(0, 32, len(stream))) * 8)
    stream["value"] = rng.integers(-1000, 1000, len(stream))
    a, b = oracle.Heap(n_pes, words * 8), oracle.Heap(n_pes, words * 8)
    oracle.small_ops(a, stream, np.zeros(len(stream), np.uint32))
    oracle.small_ops_mt(b, stream, 6)
    assert np.array_equal(a.buf, b.buf)
