"""Small puts and AMOs: final heap state, fetched values and the GPU-built WQE rings."""
import numpy as np
import pytest

import oracle
import roc_shmem_amd as rs
from helpers import runtime

pytestmark = pytest.mark.gpu

FETCHING = {rs.OP_FADD64, rs.OP_FINC64, rs.OP_CSWAP64, rs.OP_FETCH64, rs.OP_SWAP64, rs.OP_FADD32,
            rs.OP_FAND64, rs.OP_FOR64, rs.OP_FXOR64}
POSTS_WQE = {rs.OP_P64, rs.OP_FADD64, rs.OP_ADD64, rs.OP_FINC64, rs.OP_INC64, rs.OP_CSWAP64,
             rs.OP_FETCH64, rs.OP_SET64, rs.OP_SWAP64, rs.OP_P32, rs.OP_FADD32}


class Issue:
    """Who issues op i: the grid deals ops round-robin to its threads."""

    def __init__(self, n_ops, n_pes, wgs_per_pe, wg_size, num_blocks):
        i = np.arange(n_ops)
        total = n_pes * wgs_per_pe * wg_size
        t = i % total
        self.round = i // total
        blk = t // wg_size
        self.pe = (blk % n_pes).astype(np.uint32)
        self.ring_block = (blk // n_pes) % num_blocks
        self.wave = (t % wg_size) // 64
        self.lane = t % 64


def expected_wqe_fields(op, issuer_pe):
    """(opcode, size, raddr, atomic_data, atomic_cmp, inline bytes) of the entry op leaves."""
    kind = int(op["kind"])
    raddr = rs.heap_base(int(op["pe"])) + int(op["offset"])
    value = int(op["value"])
    u64 = value & 0xFFFFFFFFFFFFFFFF
    if kind == rs.OP_P64:
        return (oracle.OP_WRITE, 8, raddr, 0, 0, u64.to_bytes(8, "little"))
    if kind == rs.OP_P32:
        return (oracle.OP_WRITE, 4, raddr, 0, 0, (value & 0xFFFFFFFF).to_bytes(4, "little"))
    if kind in (rs.OP_FADD64, rs.OP_ADD64):
        return (oracle.OP_ATOMIC_FA, 8, raddr, u64, 0, b"")
    if kind in (rs.OP_FINC64, rs.OP_INC64):
        return (oracle.OP_ATOMIC_FA, 8, raddr, 1, 0, b"")
    if kind == rs.OP_FETCH64:
        return (oracle.OP_ATOMIC_FA, 8, raddr, 0, 0, b"")
    if kind == rs.OP_CSWAP64:
        return (oracle.OP_ATOMIC_CS, 8, raddr, u64, int(op["aux"]) & 0xFFFFFFFFFFFFFFFF, b"")
    if kind in (rs.OP_SET64, rs.OP_SWAP64):
        return (oracle.OP_ATOMIC_CS, 8, raddr, u64, 0, b"")
    if kind == rs.OP_FADD32:
        v32 = ((value & 0xFFFFFFFF) ^ 0x80000000) - 0x80000000  # operand widened as int64
        return (oracle.OP_ATOMIC_FA, 8, raddr, v32 & 0xFFFFFFFFFFFFFFFF, 0, b"")
    raise AssertionError(kind)


def qp_of(pe, block):
    c = rs.sq_constants(pe, block)
    qp = oracle.Qp()
    qp.ctrl_qp_sq, qp.ctrl_sig, qp.lkey = c["ctrl_qp_sq"], c["ctrl_sig"], c["lkey"]
    qp.atomic_lkey, qp.atomic_ret_base, qp.max_nwqe = c["atomic_lkey"], c["atomic_ret_base"], c["max_nwqe"]
    return qp


def be(slot, lo, hi):
    return int.from_bytes(bytes(slot[lo:hi]), "big")


def run_stream(ops, n_pes, wgs, wg_size, heap_bytes, init_heap):
    """Execute the stream on the GPU; returns (device heap words per PE, fetched)."""
    mem = rs.sym_array(heap_bytes // 8, np.int64)
    for p in range(n_pes):
        mem.write(p, init_heap[p])
    ops = np.ascontiguousarray(ops, dtype=rs.SMALL_OP_DTYPE)
    shifted = ops.copy()
    shifted["offset"] += mem.offset
    moves = np.isin(shifted["kind"], [rs.OP_PUTMEM, rs.OP_GETMEM])
    shifted["value"][moves] += mem.offset
    dev_ops = rs.device_array(shifted)
    fetched = rs.device_array(nbytes=len(ops) * 8)
    fetched.fill(0)
    rs.sq_reset()
    rs.roc_shmem_small_ops(dev_ops, len(ops), fetched, rs.Launch(wgs, wg_size))
    rs.synchronize()
    out = [mem.read(p) for p in range(n_pes)]
    got = fetched.read(np.int64, len(ops))
    dev_ops.free()
    fetched.free()
    return mem, shifted, out, got


def check_rings(shifted_ops, issue, n_pes, num_blocks, sq_size, masked_ce=True):
    """Every ring entry is byte-for-byte what the CPU builder writes for one op
    issued on that ring at the slot's counter (rings that did not wrap)."""
    posts = np.isin(shifted_ops["kind"], list(POSTS_WQE))
    for pe in range(n_pes):
        for block in range(num_blocks):
            sel = np.nonzero(posts & (issue.pe == pe) & (issue.ring_block == block))[0]
            st = rs.sq_state(pe, block)
            assert st["sq_counter"] == len(sel), (pe, block)
            assert st["published"] == len(sel)
            if len(sel) == 0:
                continue
            assert len(sel) <= sq_size, "use check_ring_history for rings that wrap"
            image = rs.sq_image(pe, block, sq_size)
            qp = qp_of(pe, block)
            # what the ops of this ring should leave, keyed by everything but the counter
            pending = {}
            for i in sel:
                key = expected_wqe_fields(shifted_ops[i], pe)
                pending[key] = pending.get(key, 0) + 1
            n_atomic = 0
            positions = set()
            for k in range(len(sel)):
                slot = image[k]
                assert be(slot, 1, 3) == k, "entry index field"
                opcode = int(slot[3])
                raddr = be(slot, 16, 24)
                if opcode in (oracle.OP_ATOMIC_FA, oracle.OP_ATOMIC_CS):
                    key = (opcode, 8, raddr, be(slot, 32, 40), be(slot, 40, 48), b"")
                    pos = (be(slot, 56, 64) - qp.atomic_ret_base) // 8
                    assert 0 <= pos < 4096 and pos not in positions
                    positions.add(pos)
                    n_atomic += 1
                else:
                    size = be(slot, 32, 36) & 0x3FF
                    key = (opcode, size, raddr, 0, 0, bytes(slot[36:36 + size]))
                    pos = 0
                assert pending.get(key, 0) > 0, "ring %d/%d slot %d holds an entry no op explains" % (pe, block, k)
                pending[key] -= 1
                dest_pe = (raddr - rs.heap_base(0)) // (rs.heap_base(1) - rs.heap_base(0)) if n_pes > 1 else 0
                exp = np.zeros(64, np.uint8)
                oracle.wqe_build(exp, qp, k, key[0], size=key[1], raddr=raddr, rkey=rs.sq_rkey(dest_pe),
                                 atomic_data=key[3], atomic_cmp=key[4], inline=key[5], atomic_pos=pos,
                                 request_cqe=bool(slot[11] == 8))
                assert slot[11] in (8, (qp.ctrl_sig >> 24) & 0xFF)
                if k == sq_size - 2:
                    assert slot[11] == 8, "slot max_nwqe - 2 asks for a completion (queue_pair.cpp:80-85)"
                assert np.array_equal(slot, exp), "ring %d/%d slot %d" % (pe, block, k)
            assert all(v == 0 for v in pending.values())
            assert positions == set(range(n_atomic)), "AMO return slots are handed out densely"
            assert st["atomic_counter"] == n_atomic
            last = image[len(sel) - 1]
            assert last[11] == 8, "the entry that closes the last post requests a completion"
            assert np.array_equal(st["mailbox"], oracle.doorbell(last, len(sel)))
            assert not image[len(sel):].any(), "slots beyond the producer index stay untouched"


def test_unique_puts_and_fetch_adds_heap_fetched_and_rings():
    # the small-operation benchmark workload at reduced size: puts to unique offsets in the lower half of
    # every slice, fetch-adds (collisions allowed) to the upper half.
    n_pes, wgs, wg_size, num_blocks, sq = 4, 4, 256, 4, 1024
    words = 1 << 14
    n_ops = 12000
    rng = np.random.default_rng(4)
    ops = np.zeros(n_ops, rs.SMALL_OP_DTYPE)
    is_put = rng.random(n_ops) < 0.5
    ops["kind"] = np.where(is_put, rs.OP_P64, rs.OP_FADD64)
    ops["pe"] = rng.integers(0, n_pes, n_ops)
    put_slots = rng.permutation(n_pes * (words // 2))[:n_ops]          # unique (pe, word) targets
    ops["pe"][is_put] = (put_slots[is_put] // (words // 2))
    ops["offset"] = np.where(is_put, (put_slots % (words // 2)) * 8,
                             (words // 2 + rng.integers(0, 64, n_ops)) * 8)
    ops["value"] = np.where(is_put, rng.integers(-(1 << 62), 1 << 62, n_ops), 3)
    issue = Issue(n_ops, n_pes, wgs, wg_size, num_blocks)
    init = [rng.integers(-1000, 1000, words, dtype=np.int64) for _ in range(n_pes)]
    with runtime(n_pes, num_blocks=num_blocks, sq_size=sq):
        mem, shifted, out, got = run_stream(ops, n_pes, wgs, wg_size, words * 8, init)
        heap = oracle.Heap(n_pes, words * 8)
        for p in range(n_pes):
            heap.view(p, 0, words, np.int64)[:] = init[p]
        model_fetched = oracle.small_ops(heap, ops, issue.pe)
        for p in range(n_pes):
            assert np.array_equal(out[p], heap.view(p, 0, words, np.int64)), "heap of PE %d" % p
        # equal addends: per target word the fetched values are the model's, in some order
        fa = np.nonzero(~is_put)[0]
        keys = ops["pe"][fa].astype(np.int64) * words + ops["offset"][fa] // 8
        for key in np.unique(keys):
            idx = fa[keys == key]
            assert np.array_equal(np.sort(got[idx]), np.sort(model_fetched[idx]))
        check_rings(shifted, issue, n_pes, num_blocks, sq)


def test_amo_family_closed_forms():
    # clients/functional_tests/amo_standard_tester.cpp:76-117: n fetch_add(2) -> last fetched
    # 2(n-1), final 2n; n fetch_inc -> fetched cover 0..n-1, final n; compare_swap chain;
    # clients/sos_tests/cxx_test_shmem_atomic_add.cpp:85-144: every PE adds me+1 -> npes(npes+1)/2
    n_pes, wgs, wg_size = 4, 2, 128
    words = 64
    with runtime(n_pes, num_blocks=2):
        init = [np.zeros(words, np.int64) for _ in range(n_pes)]
        n = 1000
        ops = np.zeros(4 * n, rs.SMALL_OP_DTYPE)
        ops["pe"] = 1
        ops["kind"][:n], ops["offset"][:n], ops["value"][:n] = rs.OP_FADD64, 0, 2
        ops["kind"][n:2 * n], ops["offset"][n:2 * n] = rs.OP_FINC64, 8
        ops["kind"][2 * n:3 * n], ops["offset"][2 * n:3 * n], ops["value"][2 * n:3 * n] = rs.OP_ADD64, 16, 2
        ops["kind"][3 * n:], ops["offset"][3 * n:] = rs.OP_INC64, 24
        mem, shifted, out, got = run_stream(ops, n_pes, wgs, wg_size, words * 8, init)
        assert out[1][0] == 2 * n and np.array_equal(np.sort(got[:n]), 2 * np.arange(n))
        assert out[1][1] == n and np.array_equal(np.sort(got[n:2 * n]), np.arange(n))
        assert out[1][2] == 2 * n and out[1][3] == n
        for p in (0, 2, 3):
            assert not out[p].any()
        mem.free()
        # every PE adds (me + 1) to word 5 of every PE
        issue = Issue(n_pes * n_pes * 64, n_pes, 1, 64, 2)
        ops = np.zeros(n_pes * n_pes * 64, rs.SMALL_OP_DTYPE)
        ops["kind"] = rs.OP_NONE
        for i in range(len(ops)):
            if issue.lane[i] < n_pes and issue.round[i] == 0:
                ops["kind"][i], ops["pe"][i], ops["offset"][i] = rs.OP_ADD64, issue.lane[i], 40
                ops["value"][i] = issue.pe[i] + 1
        mem, shifted, out, got = run_stream(ops, n_pes, 1, 64, words * 8, init)
        for p in range(n_pes):
            assert out[p][5] == n_pes * (n_pes + 1) // 2
        mem.free()


def assert_serialisation(fetched, addends, initial, final, modulus):
    """The fetched values are those of some order of the adds: sorted by what they fetched, each
    op finds the word as the previous one left it (all addends are positive and the total stays
    below the modulus... or wraps exactly once, which the sort key accounts for)."""
    seen = [int(f) % modulus for f in fetched]
    order = sorted(range(len(seen)), key=lambda i: (seen[i] - initial) % modulus)
    value = initial % modulus
    for i in order:
        assert seen[i] == value, "op %d fetched %d, the word held %d" % (i, seen[i], value)
        value = (value + int(addends[i])) % modulus
    assert value == final % modulus


@pytest.mark.parametrize("n_words,wg_size", [(1, 256), (3, 256), (16, 64), (40, 128)])
def test_fetch_adds_that_collide_form_a_serialisation(n_words, wg_size):
    # Lanes of a wave that name the same word share one atomic; every op must still fetch what
    # some order of all the adds would have shown it, and the word must end at the total.
    n_pes, wgs, words, n = 4, 2, 64, 6000
    rng = np.random.default_rng(n_words)
    with runtime(n_pes, num_blocks=2):
        init = [np.full(words, 1000 + p, np.int64) for p in range(n_pes)]
        ops = np.zeros(n, rs.SMALL_OP_DTYPE)
        word = rng.integers(0, n_words, n)
        ops["kind"] = rs.OP_FADD64
        ops["pe"] = word % n_pes
        ops["offset"] = (word // n_pes) * 8
        ops["value"] = rng.integers(1, 1000, n)
        same = rng.random(n) < 0.3
        ops["value"][same] = 7                     # runs of equal addends take the closed-form path
        mem, shifted, out, got = run_stream(ops, n_pes, wgs, wg_size, words * 8, init)
        for w in range(n_words):
            sel = np.nonzero(word == w)[0]
            pe, slot = w % n_pes, w // n_pes
            assert_serialisation(got[sel], ops["value"][sel], 1000 + pe, int(out[pe][slot]), 1 << 64)
            assert int(out[pe][slot]) == 1000 + pe + int(ops["value"][sel].sum())
        mem.free()


def test_colliding_32_bit_fetch_adds_wrap():
    n_pes, words, n = 2, 8, 3000
    rng = np.random.default_rng(5)
    with runtime(n_pes, num_blocks=2):
        init = [np.zeros(words, np.int64) for _ in range(n_pes)]
        init[1][0] = 0xFFFFF000                    # low word close to wrapping, high word zero
        ops = np.zeros(n, rs.SMALL_OP_DTYPE)
        ops["kind"], ops["pe"], ops["offset"] = rs.OP_FADD32, 1, 0
        ops["value"] = rng.integers(1, 100, n)
        mem, shifted, out, got = run_stream(ops, n_pes, 2, 256, words * 8, init)
        total = int(ops["value"].sum())
        low = int(out[1][0]) & 0xFFFFFFFF
        assert low == (0xFFFFF000 + total) & 0xFFFFFFFF
        assert int(out[1][0]) >> 32 == 0, "a 32-bit add reached the neighbouring word"
        assert_serialisation(got & 0xFFFFFFFF, ops["value"], 0xFFFFF000, low, 1 << 32)
        mem.free()


def test_swap_set_cswap_fetch_and_bitwise():
    n_pes, words = 2, 32
    with runtime(n_pes, num_blocks=1):
        init = [np.arange(words, dtype=np.int64) * 11 for _ in range(n_pes)]
        # one lane of one wave per op: a serial stream, so the sequential model is exact
        kinds = [(rs.OP_SWAP64, 1, 8, 777, 0), (rs.OP_CSWAP64, 1, 16, 5, 22), (rs.OP_CSWAP64, 1, 24, 5, 22),
                 (rs.OP_FETCH64, 0, 32, 0, 0), (rs.OP_SET64, 0, 40, -9, 0), (rs.OP_FAND64, 1, 48, 0x0F, 0),
                 (rs.OP_FOR64, 1, 56, 0xF00, 0), (rs.OP_FXOR64, 1, 64, 0xFF, 0), (rs.OP_P32, 1, 72, 0x12345678, 0),
                 (rs.OP_FADD32, 1, 84, -5, 0)]
        total = n_pes * 64
        ops = np.zeros(len(kinds) * total, rs.SMALL_OP_DTYPE)
        ops["kind"] = rs.OP_NONE
        for r, (k, pe, off, val, aux) in enumerate(kinds):
            ops[r * total] = (k, pe, off, val, aux)
        issue = Issue(len(ops), n_pes, 1, 64, 1)
        mem, shifted, out, got = run_stream(ops, n_pes, 1, 64, words * 8, init)
        heap = oracle.Heap(n_pes, words * 8)
        for p in range(n_pes):
            heap.view(p, 0, words, np.int64)[:] = init[p]
        model = oracle.small_ops(heap, ops, issue.pe)
        for p in range(n_pes):
            assert np.array_equal(out[p], heap.view(p, 0, words, np.int64))
        idx = [r * total for r, k in enumerate(kinds) if k[0] in FETCHING]
        assert np.array_equal(got[idx], model[idx])
        # 32-bit operands touch 32 bits only (the reference's NIC path moves 64):
        # word 10 = 110 initially; the fetch-add hits its upper half, the lower half stays
        assert int(out[1][10]) & 0xFFFFFFFF == 110
        assert (int(out[1][10]) >> 32) & 0xFFFFFFFF == (-5) & 0xFFFFFFFF
        check_rings(shifted, issue, n_pes, 1, 1024)


def test_ring_history_with_wraparound_is_byte_exact():
    # One wave per ring and one kind per round make the slot of every op known in
    # advance (counter = round*64 + lane), so the CPU builder can replay the whole history of a
    # 64-entry ring, including bytes that survive from an older entry of another shape.
    n_pes, sq = 2, 64
    words = 1 << 12
    round_kinds = [rs.OP_FADD64, rs.OP_P64, rs.OP_P32, rs.OP_CSWAP64, rs.OP_P64, rs.OP_ADD64, rs.OP_P32]
    total = n_pes * 64
    rng = np.random.default_rng(12)
    ops = np.zeros(len(round_kinds) * total, rs.SMALL_OP_DTYPE)
    for r, k in enumerate(round_kinds):
        sl = slice(r * total, (r + 1) * total)
        ops["kind"][sl] = k
        ops["pe"][sl] = rng.integers(0, n_pes, total)
        ops["offset"][sl] = (r * total + rng.permutation(total)) * 8   # all targets distinct
        ops["value"][sl] = rng.integers(-(1 << 40), 1 << 40, total)
        ops["aux"][sl] = rng.integers(-3, 3, total)
    issue = Issue(len(ops), n_pes, 1, 64, 1)
    init = [rng.integers(-3, 3, words, dtype=np.int64) for _ in range(n_pes)]
    with runtime(n_pes, num_blocks=1, sq_size=sq):
        mem, shifted, out, got = run_stream(ops, n_pes, 1, 64, words * 8, init)
        heap = oracle.Heap(n_pes, words * 8)
        for p in range(n_pes):
            heap.view(p, 0, words, np.int64)[:] = init[p]
        oracle.small_ops(heap, ops, issue.pe)
        for p in range(n_pes):
            assert np.array_equal(out[p], heap.view(p, 0, words, np.int64))
        for pe in range(n_pes):
            qp = qp_of(pe, 0)
            ring = np.zeros((sq, 64), np.uint8)
            n_atomic = 0
            counter = 0
            for r in range(len(round_kinds)):
                idx = np.nonzero((issue.pe == pe) & (issue.round == r))[0]
                idx = idx[np.argsort(issue.lane[idx])]
                for j, i in enumerate(idx):
                    opcode, size, raddr, adata, acmp, inl = expected_wqe_fields(shifted[i], pe)
                    pos = 0
                    if opcode in (oracle.OP_ATOMIC_FA, oracle.OP_ATOMIC_CS):
                        pos = n_atomic % 4096
                        n_atomic += 1
                    oracle.wqe_build(ring[counter % sq], qp, counter, opcode, size=size, raddr=raddr,
                                     rkey=rs.sq_rkey(int(shifted[i]["pe"])), atomic_data=adata,
                                     atomic_cmp=acmp, inline=inl, atomic_pos=pos,
                                     request_cqe=oracle.requests_cqe(counter, sq, j == len(idx) - 1))
                    counter += 1
            st = rs.sq_state(pe, 0)
            assert st["sq_counter"] == counter and st["published"] == counter
            assert st["atomic_counter"] == n_atomic
            image = rs.sq_image(pe, 0, sq)
            assert np.array_equal(image, ring), "ring of PE %d: first differing slot %d" % (
                pe, int(np.argmax((image != ring).any(axis=1))))
            assert np.array_equal(st["mailbox"], oracle.doorbell(ring[(counter - 1) % sq], counter))


def test_coalesced_thread_puts_post_one_entry_per_run():
    # 64 lanes putting 8 contiguous bytes each to the same PE merge into a single 512-byte
    # entry that names the first lane's source (library/src/wf_coal_policy.cpp:57-172).
    n_pes, words = 2, 4096
    with runtime(n_pes, num_blocks=1):
        rng = np.random.default_rng(2)
        init = [rng.integers(-9, 9, words, dtype=np.int64) for _ in range(n_pes)]
        total = n_pes * 64
        ops = np.zeros(total, rs.SMALL_OP_DTYPE)
        issue = Issue(total, n_pes, 1, 64, 1)
        ops["kind"] = rs.OP_PUTMEM
        ops["pe"] = (issue.pe + 1) % n_pes
        ops["offset"] = (1024 + issue.lane) * 8           # destination: contiguous by lane
        ops["value"] = (16 + issue.lane) * 8              # source offset: contiguous by lane
        ops["aux"] = 8
        mem, shifted, out, got = run_stream(ops, n_pes, 1, 64, words * 8, init)
        heap = oracle.Heap(n_pes, words * 8)
        for p in range(n_pes):
            heap.view(p, 0, words, np.int64)[:] = init[p]
        oracle.small_ops(heap, ops, issue.pe)
        for p in range(n_pes):
            assert np.array_equal(out[p], heap.view(p, 0, words, np.int64))
        for pe in range(n_pes):
            st = rs.sq_state(pe, 0)
            assert st["sq_counter"] == 1
            qp = qp_of(pe, 0)
            exp = np.zeros(64, np.uint8)
            dest = (pe + 1) % n_pes
            oracle.wqe_build(exp, qp, 0, oracle.OP_WRITE, size=512,
                             raddr=rs.heap_base(dest) + mem.offset + 1024 * 8, rkey=rs.sq_rkey(dest),
                             laddr=rs.heap_base(pe) + mem.offset + 16 * 8, request_cqe=True)
            assert np.array_equal(rs.sq_image(pe, 0, 1)[0], exp)
