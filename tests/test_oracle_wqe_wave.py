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
    assert len(g["entries"]) >= 4
    for e in g["entries"]:
        slot = np.full(64, int(e["background"], 16), np.uint8)
        oracle.wqe_build(slot, queue, num(e["counter"]), num(e["opcode"]), size=e["size"],
                         raddr=num(e["raddr"]), rkey=num(e["rkey"]), laddr=num(e.get("laddr", 0)),
                         atomic_data=num(e.get("atomic_data", 0)), atomic_cmp=num(e.get("atomic_cmp", 0)),
                         inline=bytes.fromhex(e.get("inline", "")), atomic_pos=e.get("atomic_pos", 0),
                         request_cqe=e["cqe"])
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
