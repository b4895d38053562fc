"""ctypes front end of the CPU oracle (``oracle/*.c``).

Test infrastructure: only the tests, the smoke run and the benchmark's
CPU-baseline leg import this package.  The GPU library never does.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

SHORT, INT, LONG, LONGLONG, FLOAT, DOUBLE, BF16 = range(7)
SUM, MAX, MIN, PROD, AND, OR, XOR = range(7)


def build():
    """Compile liboracle.so with gcc (seconds)."""
    subprocess.run(["make", "-s", "-C", _HERE], check=True)


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    lib = C.CDLL(_LIB_PATH)
    vp, sz, i32, u64, u32 = C.c_void_p, C.c_size_t, C.c_int, C.c_uint64, C.c_uint32
    lib.orc_dtype_size.restype = sz
    lib.orc_dtype_size.argtypes = [i32]
    lib.orc_to_all.argtypes = [i32, i32, vp, sz, sz, sz, sz, i32, i32, i32]
    lib.orc_to_all_team.argtypes = [i32, i32, vp, sz, sz, sz, sz, i32, i32, i32]
    lib.orc_to_all_rounded_once.argtypes = [i32, i32, vp, sz, sz, sz, sz, i32, i32, i32]
    lib.orc_to_all_mt.argtypes = [i32, i32, vp, sz, sz, sz, sz, i32, i32, i32, i32]
    lib.orc_to_all_f64.argtypes = [i32, i32, vp, sz, sz, sz, i32, i32, i32, vp]
    lib.orc_abs_sum_f64.argtypes = [i32, vp, sz, sz, sz, i32, i32, i32, vp]
    lib.orc_float_to_bf16.restype = C.c_uint16
    lib.orc_float_to_bf16.argtypes = [C.c_float]
    lib.orc_bf16_to_float.restype = C.c_float
    lib.orc_bf16_to_float.argtypes = [C.c_uint16]
    for name in ("orc_put", "orc_get"):
        getattr(lib, name).restype = None
        getattr(lib, name).argtypes = [vp, sz, sz, sz, sz, i32, i32]
    lib.orc_broadcast.restype = None
    lib.orc_broadcast.argtypes = [vp, sz, sz, sz, sz, i32, i32, i32, i32]
    lib.orc_broadcast_team.restype = None
    lib.orc_broadcast_team.argtypes = [vp, sz, sz, sz, sz, i32, i32, i32, i32]
    for name in ("orc_alltoall", "orc_fcollect", "orc_alltoall_team", "orc_fcollect_team"):
        getattr(lib, name).restype = None
        getattr(lib, name).argtypes = [vp, sz, sz, sz, sz, i32, i32, i32]
    lib.orc_copy_mt.restype = None
    lib.orc_copy_mt.argtypes = [vp, vp, sz, i32]
    lib.orc_small_ops.argtypes = [vp, sz, vp, vp, sz, vp]
    lib.orc_wqe_build.restype = None
    lib.orc_wqe_build.argtypes = [vp, vp, u32, vp]
    lib.orc_sq_consume.restype = None
    lib.orc_sq_consume.argtypes = [vp, vp, u32, u32, vp, vp, vp, vp, vp, u32, vp, vp]
    lib.orc_ring_check.restype = C.c_long
    lib.orc_ring_check.argtypes = [vp, vp, u32, u32, vp, sz, vp, vp, i32, vp, vp, vp, vp]
    lib.orc_wqe_build_many.restype = None
    lib.orc_wqe_build_many.argtypes = [vp, vp, u32, vp, sz]
    lib.orc_small_ops_mt.argtypes = [vp, sz, vp, sz, vp, i32]
    lib.orc_wqe_index.restype = C.c_uint16
    lib.orc_wqe_index.argtypes = [vp]
    lib.orc_wqe_opcode.restype = C.c_uint8
    lib.orc_wqe_opcode.argtypes = [vp]
    lib.orc_wqe_raddr.restype = u64
    lib.orc_wqe_raddr.argtypes = [vp]
    lib.orc_doorbell.restype = None
    lib.orc_doorbell.argtypes = [vp, u32, vp]
    lib.orc_bswap16.restype = C.c_uint16
    lib.orc_bswap16.argtypes = [C.c_uint16]
    lib.orc_bswap32.restype = u32
    lib.orc_bswap32.argtypes = [u32]
    lib.orc_bswap64.restype = u64
    lib.orc_bswap64.argtypes = [u64]
    lib.orc_coalesce.restype = None
    lib.orc_coalesce.argtypes = [u64, vp, vp, vp, vp, vp, vp]
    lib.orc_fetch_incr.restype = None
    lib.orc_fetch_incr.argtypes = [u64, vp, vp]
    lib.orc_alloc_create.restype = vp
    lib.orc_alloc_create.argtypes = [sz]
    lib.orc_alloc_destroy.restype = None
    lib.orc_alloc_destroy.argtypes = [vp]
    lib.orc_alloc_alloc.restype = sz
    lib.orc_alloc_alloc.argtypes = [vp, sz]
    lib.orc_alloc_free.argtypes = [vp, sz]
    lib.orc_alloc_in_use.restype = sz
    lib.orc_alloc_in_use.argtypes = [vp]
    return lib


_lib = _load()

NP_DTYPE = {SHORT: np.int16, INT: np.int32, LONG: np.int64, LONGLONG: np.int64,
            FLOAT: np.float32, DOUBLE: np.float64, BF16: np.uint16}

SMALL_OP_DTYPE = np.dtype([("kind", "<u4"), ("pe", "<u4"), ("offset", "<u8"),
                           ("value", "<i8"), ("aux", "<i8")])
# Kinds of the small-operation stream (the codes of enum rsm_small_kind).
(OP_P64, OP_FADD64, OP_ADD64, OP_FINC64, OP_INC64, OP_CSWAP64, OP_FETCH64, OP_SET64, OP_SWAP64,
 OP_P32, OP_FADD32, OP_PUTMEM, OP_GETMEM, OP_FAND64, OP_FOR64, OP_FXOR64) = range(16)


def dtype_size(dtype):
    return int(_lib.orc_dtype_size(dtype))


class Heap:
    """All PE slices in one host buffer: slice p is ``buf[p*stride:(p+1)*stride]``."""

    def __init__(self, n_pes, stride, fill=0):
        self.n_pes = n_pes
        self.stride = stride
        self.buf = np.full(n_pes * stride, fill, dtype=np.uint8)

    @property
    def ptr(self):
        return self.buf.ctypes.data

    def view(self, pe, offset, count, np_dtype):
        start = pe * self.stride + offset
        nbytes = count * np.dtype(np_dtype).itemsize
        return self.buf[start:start + nbytes].view(np_dtype)


def to_all(heap, dtype, op, dest_off, src_off, n, pe_start=0, log_stride=0, pe_size=None,
           threads=1, pe_stride=None):
    """pe_stride: the team form, members pe_start + k * pe_stride (log_stride is then ignored)."""
    pe_size = heap.n_pes if pe_size is None else pe_size
    if pe_stride is not None:
        rc = _lib.orc_to_all_team(dtype, op, heap.ptr, heap.stride, dest_off, src_off, n, pe_start,
                                  pe_stride, pe_size)
    elif threads > 1:
        rc = _lib.orc_to_all_mt(dtype, op, heap.ptr, heap.stride, dest_off, src_off, n, pe_start,
                                log_stride, pe_size, threads)
    else:
        rc = _lib.orc_to_all(dtype, op, heap.ptr, heap.stride, dest_off, src_off, n, pe_start,
                             log_stride, pe_size)
    if rc != 0:
        raise ValueError("reduction not defined for this (dtype, op)")


def to_all_rounded_once(heap, dtype, op, dest_off, src_off, n, pe_start=0, log_stride=0, pe_size=None,
                        pe_stride=None):
    """The GPU library's floating-point contract (float sum/prod folded in double, bfloat16 sum in
    float, ascending member order, one rounding; everything else as ``to_all``): bit-exact
    expectation for its results."""
    pe_size = heap.n_pes if pe_size is None else pe_size
    stride = (1 << log_stride) if pe_stride is None else pe_stride
    rc = _lib.orc_to_all_rounded_once(dtype, op, heap.ptr, heap.stride, dest_off, src_off, n, pe_start,
                                      stride, pe_size)
    if rc != 0:
        raise ValueError("reduction not defined for this (dtype, op)")


def to_all_f64(heap, dtype, op, src_off, n, pe_start=0, log_stride=0, pe_size=None):
    pe_size = heap.n_pes if pe_size is None else pe_size
    out = np.empty(n, dtype=np.float64)
    rc = _lib.orc_to_all_f64(dtype, op, heap.ptr, heap.stride, src_off, n, pe_start, log_stride,
                             pe_size, out.ctypes.data)
    if rc != 0:
        raise ValueError("ground truth not defined for this (dtype, op)")
    return out


def abs_sum_f64(heap, dtype, src_off, n, pe_start=0, log_stride=0, pe_size=None):
    pe_size = heap.n_pes if pe_size is None else pe_size
    out = np.empty(n, dtype=np.float64)
    _lib.orc_abs_sum_f64(dtype, heap.ptr, heap.stride, src_off, n, pe_start, log_stride, pe_size,
                         out.ctypes.data)
    return out


def float_to_bf16(x):
    """Round float32 array to bfloat16 bit patterns (nearest even)."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    r = np.where(nan, (u >> 16) | 0x40, r)
    return r.astype(np.uint16)


def bf16_to_float(b):
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def put(heap, dest_off, src_off, nbytes, src_pe, dest_pe):
    _lib.orc_put(heap.ptr, heap.stride, dest_off, src_off, nbytes, src_pe, dest_pe)


def get(heap, dest_off, src_off, nbytes, my_pe, from_pe):
    _lib.orc_get(heap.ptr, heap.stride, dest_off, src_off, nbytes, my_pe, from_pe)


def broadcast(heap, dest_off, src_off, nbytes, root_idx, pe_start=0, log_stride=0, pe_size=None,
              pe_stride=None):
    pe_size = heap.n_pes if pe_size is None else pe_size
    if pe_stride is not None:
        _lib.orc_broadcast_team(heap.ptr, heap.stride, dest_off, src_off, nbytes, root_idx, pe_start,
                                pe_stride, pe_size)
        return
    _lib.orc_broadcast(heap.ptr, heap.stride, dest_off, src_off, nbytes, root_idx, pe_start,
                       log_stride, pe_size)


def alltoall(heap, dest_off, src_off, block_bytes, pe_start=0, log_stride=0, pe_size=None,
             pe_stride=None):
    pe_size = heap.n_pes if pe_size is None else pe_size
    if pe_stride is not None:
        _lib.orc_alltoall_team(heap.ptr, heap.stride, dest_off, src_off, block_bytes, pe_start,
                               pe_stride, pe_size)
        return
    _lib.orc_alltoall(heap.ptr, heap.stride, dest_off, src_off, block_bytes, pe_start, log_stride,
                      pe_size)


def fcollect(heap, dest_off, src_off, block_bytes, pe_start=0, log_stride=0, pe_size=None,
             pe_stride=None):
    pe_size = heap.n_pes if pe_size is None else pe_size
    if pe_stride is not None:
        _lib.orc_fcollect_team(heap.ptr, heap.stride, dest_off, src_off, block_bytes, pe_start,
                               pe_stride, pe_size)
        return
    _lib.orc_fcollect(heap.ptr, heap.stride, dest_off, src_off, block_bytes, pe_start, log_stride,
                      pe_size)


def copy_mt(dst, src, threads):
    assert dst.nbytes == src.nbytes
    _lib.orc_copy_mt(dst.ctypes.data, src.ctypes.data, src.nbytes, threads)


def small_ops(heap, ops, issuer_pe):
    ops = np.ascontiguousarray(ops, dtype=SMALL_OP_DTYPE)
    issuer = np.ascontiguousarray(issuer_pe, dtype=np.uint32)
    fetched = np.zeros(len(ops), dtype=np.int64)
    rc = _lib.orc_small_ops(heap.ptr, heap.stride, ops.ctypes.data, issuer.ctypes.data, len(ops),
                            fetched.ctypes.data)
    if rc != 0:
        raise ValueError("unknown small-op kind")
    return fetched


class Qp(C.Structure):
    _fields_ = [("ctrl_qp_sq", C.c_uint32), ("ctrl_sig", C.c_uint64), ("lkey", C.c_uint32),
                ("atomic_lkey", C.c_uint32), ("atomic_ret_base", C.c_uint64),
                ("max_nwqe", C.c_uint32)]


class WqeReq(C.Structure):
    _fields_ = [("opcode", C.c_uint8), ("size", C.c_uint32), ("raddr", C.c_uint64),
                ("rkey", C.c_uint32), ("laddr", C.c_uint64), ("atomic_data", C.c_uint64),
                ("atomic_cmp", C.c_uint64), ("inline_bytes", C.c_uint8 * 8),
                ("atomic_pos", C.c_uint32), ("request_cqe", C.c_int), ("form", C.c_int)]


OP_WRITE, OP_READ, OP_ATOMIC_CS, OP_ATOMIC_FA = 0x08, 0x10, 0x11, 0x12


def requests_cqe(sq_counter, max_nwqe, closes_post):
    """Whether the entry with running number ``sq_counter`` asks for a completion entry: the
    entry that closes a wave's post always does (multi-thread post policy, reference
    library/src/gpu_ib/thread_policy.cpp:170-216), and so does whatever lands in slot
    ``max_nwqe - 2`` of a lap (update_wqe_ce_single<false>, queue_pair.cpp:80-85)."""
    return bool(closes_post) or sq_counter % max_nwqe == max_nwqe - 2


WQE_DATA, WQE_ZERO_BYTE_READ, WQE_FLUSH_WRITE = range(3)


def wqe_build(slot, qp, sq_counter, opcode, size=0, raddr=0, rkey=0, laddr=0, atomic_data=0,
              atomic_cmp=0, inline=b"", atomic_pos=0, request_cqe=False, form=WQE_DATA):
    """Write one entry into ``slot`` (a 64-byte uint8 array view), in place."""
    assert slot.dtype == np.uint8 and slot.size == 64 and slot.flags["C_CONTIGUOUS"]
    rq = WqeReq()
    rq.opcode = opcode
    rq.size = size
    rq.raddr = raddr & 0xFFFFFFFFFFFFFFFF
    rq.rkey = rkey
    rq.laddr = laddr & 0xFFFFFFFFFFFFFFFF
    rq.atomic_data = atomic_data & 0xFFFFFFFFFFFFFFFF
    rq.atomic_cmp = atomic_cmp & 0xFFFFFFFFFFFFFFFF
    for i, b in enumerate(bytes(inline)[:8]):
        rq.inline_bytes[i] = b
    rq.atomic_pos = atomic_pos
    rq.request_cqe = 1 if request_cqe else 0
    rq.form = form
    _lib.orc_wqe_build(slot.ctypes.data, C.byref(qp), sq_counter & 0xFFFFFFFF, C.byref(rq))
    return slot


class Arena(C.Structure):
    _fields_ = [("heap_base0", C.c_uint64), ("slice_stride", C.c_uint64), ("heap_size", C.c_uint64),
                ("num_pes", C.c_int), ("rkeys", C.c_void_p), ("flush_base", C.c_uint64),
                ("flush_rkeys", C.c_void_p)]


class ConsumeTotals(C.Structure):
    _fields_ = [(n, C.c_uint64) for n in ("retired", "writes", "reads", "atomics", "bytes",
                                          "completions", "lost", "rejected", "local_skipped")]

    def as_dict(self):
        return {n: int(getattr(self, n)) for n, _ in self._fields_}


def sq_consume(qp, ring, consumed, published, heap_base0, slice_stride, heap_size, rkeys, target,
               sources, atomic_ret, cq, cq_producer=0, totals=None, flush_base=0, flush_rkeys=None):
    """Retire entries [consumed, published) of one ring image (uint8, max_nwqe*64) in order.

    ``target`` / ``sources``: uint8 images laid out like the arena (``target`` may be None).
    ``atomic_ret``: uint64[4096]; ``cq``: uint8 image of the completion queue.  Returns
    (new cq_producer, ConsumeTotals)."""
    rk = np.ascontiguousarray(rkeys, dtype=np.uint32)
    frk = None if flush_rkeys is None else np.ascontiguousarray(flush_rkeys, dtype=np.uint32)
    arena = Arena(heap_base0, slice_stride, heap_size, len(rk), rk.ctypes.data, flush_base,
                  None if frk is None else frk.ctypes.data)
    totals = totals if totals is not None else ConsumeTotals()
    prod = C.c_uint32(cq_producer)
    assert ring.dtype == np.uint8 and ring.flags["C_CONTIGUOUS"] and ring.size == qp.max_nwqe * 64
    assert cq.dtype == np.uint8 and cq.size % 64 == 0 and atomic_ret.dtype == np.uint64
    _lib.orc_sq_consume(C.byref(qp), ring.ctypes.data, consumed & 0xFFFFFFFF, published & 0xFFFFFFFF,
                        C.byref(arena), None if target is None else target.ctypes.data,
                        None if sources is None else sources.ctypes.data, atomic_ret.ctypes.data,
                        cq.ctypes.data, cq.size // 64, C.byref(prod), C.byref(totals))
    return prod.value, totals


WQE_EXPECT_DTYPE = np.dtype([("raddr", "<u8"), ("data", "<u8"), ("cmp", "<u8"),
                             ("opcode", "<u4"), ("size", "<u4")])
RING_CHECK_REASONS = {1: "index field", 2: "opcode", 3: "AMO return slot outside the window",
                      4: "not an inline write of 1..8 bytes", 5: "completion flag",
                      6: "no operation of this ring explains the entry (or it appears twice)",
                      7: "remote address outside the arena", 8: "bytes differ from the builder's"}


def sort_wqe_expect(expect):
    """Order the checker wants: ascending (opcode, raddr, data, cmp)."""
    order = np.lexsort((expect["cmp"], expect["data"], expect["raddr"], expect["opcode"]))
    return np.ascontiguousarray(expect[order])


def ring_check(image, qp, first_counter, count, expect_sorted, heap_base0, slice_stride, heap_size,
               rkeys, full_slot, flush_base=0, flush_rkeys=None):
    """Entries first_counter .. first_counter+count-1 of a ring image (uint8, max_nwqe*64)
    against wqe_build (see ringcheck.c).  Returns a dict: ok, position / reason of the first
    wrong entry, used (which operations were matched), pos_count (uint32[4096] AMO return
    positions), n_atomic, n_cqe."""
    image = np.ascontiguousarray(image, dtype=np.uint8).reshape(-1)
    assert image.size == qp.max_nwqe * 64 and expect_sorted.dtype == WQE_EXPECT_DTYPE
    rk = np.ascontiguousarray(rkeys, dtype=np.uint32)
    frk = None if flush_rkeys is None else np.ascontiguousarray(flush_rkeys, dtype=np.uint32)
    arena = Arena(heap_base0, slice_stride, heap_size, len(rk), rk.ctypes.data, flush_base,
                  None if frk is None else frk.ctypes.data)
    used = np.zeros(len(expect_sorted), dtype=np.uint8)
    pos_count = np.zeros(4096, dtype=np.uint32)
    n_atomic, n_cqe, why = C.c_uint32(0), C.c_uint32(0), C.c_int(0)
    rc = _lib.orc_ring_check(image.ctypes.data, C.byref(qp), first_counter & 0xFFFFFFFF, count,
                             expect_sorted.ctypes.data, len(expect_sorted), used.ctypes.data,
                             C.byref(arena), 1 if full_slot else 0, pos_count.ctypes.data,
                             C.byref(n_atomic), C.byref(n_cqe), C.byref(why))
    return {"ok": rc == 0, "position": rc - 1, "reason": RING_CHECK_REASONS.get(why.value, ""),
            "used": used, "pos_count": pos_count, "n_atomic": n_atomic.value, "n_cqe": n_cqe.value}


def wqe_build_many(ring, qp, first_counter, reqs):
    """The scalar builder over an array of WqeReq (ctypes array) into a ring image."""
    _lib.orc_wqe_build_many(ring.ctypes.data, C.byref(qp), first_counter & 0xFFFFFFFF, reqs, len(reqs))


def small_ops_mt(heap, ops, threads):
    """8-byte puts and 64-bit fetch-adds of ``ops`` applied by ``threads`` host threads with
    hardware atomics (the host-centric path's MPI_Put / MPI_Fetch_and_op on one node)."""
    ops = np.ascontiguousarray(ops, dtype=SMALL_OP_DTYPE)
    rc = _lib.orc_small_ops_mt(heap.buf.ctypes.data, heap.stride, ops.ctypes.data, len(ops), None, threads)
    if rc != 0:
        raise ValueError("small_ops_mt handles 8-byte puts and 64-bit fetch-adds only")


def wqe_index(slot):
    return int(_lib.orc_wqe_index(slot.ctypes.data))


def wqe_opcode(slot):
    return int(_lib.orc_wqe_opcode(slot.ctypes.data))


def wqe_raddr(slot):
    return int(_lib.orc_wqe_raddr(slot.ctypes.data))


def doorbell(last_slot, sq_counter_after):
    out = np.zeros(2, dtype=np.uint64)
    _lib.orc_doorbell(last_slot.ctypes.data, sq_counter_after & 0xFFFFFFFF, out.ctypes.data)
    return out


def bswap16(v):
    return int(_lib.orc_bswap16(v))


def bswap32(v):
    return int(_lib.orc_bswap32(v))


def bswap64(v):
    return int(_lib.orc_bswap64(v))


def coalesce(lane_mask, pe, src, dst, size):
    pe = np.ascontiguousarray(pe, dtype=np.int32)
    src = np.ascontiguousarray(src, dtype=np.uint64)
    dst = np.ascontiguousarray(dst, dtype=np.uint64)
    size = np.ascontiguousarray(size, dtype=np.uint64)
    must = np.zeros(64, dtype=np.uint8)
    out = np.zeros(64, dtype=np.uint64)
    _lib.orc_coalesce(lane_mask, pe.ctypes.data, src.ctypes.data, dst.ctypes.data,
                      size.ctypes.data, must.ctypes.data, out.ctypes.data)
    return must, out


def fetch_incr(lane_mask, counter):
    ctr = C.c_uint64(counter)
    out = np.zeros(64, dtype=np.uint64)
    _lib.orc_fetch_incr(lane_mask, C.byref(ctr), out.ctypes.data)
    return out, ctr.value


class Allocator:
    NONE = C.c_size_t(-1).value

    def __init__(self, heap_bytes):
        self._a = _lib.orc_alloc_create(heap_bytes)

    def alloc(self, n):
        return int(_lib.orc_alloc_alloc(self._a, n))

    def free(self, off):
        return int(_lib.orc_alloc_free(self._a, off))

    def in_use(self):
        return int(_lib.orc_alloc_in_use(self._a))

    def __del__(self):
        if getattr(self, "_a", None):
            _lib.orc_alloc_destroy(self._a)
            self._a = None
