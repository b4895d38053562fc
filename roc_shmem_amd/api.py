"""Host-side mirror of the reference's interface for the data path.

Names follow ``library/include/roc_shmem.hpp`` of the reference: ``roc_shmem_init``,
``roc_shmem_malloc``, ``roc_shmem_<T>_<op>_to_all`` ... with the single-process
meaning described in ``include/roc_shmem.hpp``.  Symmetric objects are plain
integer addresses (PE 0's address); ``SymArray`` wraps one with numpy I/O.
"""
import ctypes as C

import numpy as np

from . import _lib as L

__all__ = [
    "RocShmemError", "SymArray", "Launch", "Stream", "Graph",
    "roc_shmem_init", "roc_shmem_finalize", "roc_shmem_n_pes", "roc_shmem_malloc",
    "roc_shmem_free", "roc_shmem_ptr", "roc_shmem_team_world", "roc_shmem_team_split_strided",
    "roc_shmem_team_destroy", "roc_shmem_team_n_pes", "roc_shmem_team_translate_pe",
    "roc_shmem_barrier_all", "roc_shmem_to_all", "roc_shmem_to_all_noalloc", "roc_shmem_team_to_all",
    "roc_shmem_rma",
    "roc_shmem_broadcast", "roc_shmem_team_broadcast", "roc_shmem_alltoall",
    "roc_shmem_fcollect", "roc_shmem_wg_barrier_all", "roc_shmem_small_ops",
    "sq_reset", "sq_read", "sq_image", "sq_state", "sq_constants", "sq_rkey", "sq_flush_target",
    "sq_consume", "sq_set_mode", "sq_consumer_state", "sq_consumer_start", "sq_consumer_stop",
    "sq_consumer_running", "cq_reader_state", "cq_image", "atomic_ret_image", "arena",
    "read_device", "write_device",
    "kat_fetch_incr", "kat_coalesce", "take_status", "set_pacing", "get_pacing", "tune_reduce_pacing", "stream_probe", "STREAM_READ", "STREAM_WRITE", "STREAM_RUNTIME_FILL", "STREAM_RUNTIME_COPY", "STREAM_COPY", "synchronize", "heap_bytes_in_use",
    "sym_array", "Event", "device_array", "heap_base",
    "SHORT", "INT", "LONG", "LONGLONG", "FLOAT", "DOUBLE", "BF16",
    "SUM", "MAX", "MIN", "PROD", "AND", "OR", "XOR",
    "PUT", "GET", "PUT_NBI", "GET_NBI", "THREAD", "WAVE", "WG", "WG_SHARED",
    "SMALL_OP_DTYPE", "OP_P64", "OP_FADD64", "OP_ADD64", "OP_FINC64", "OP_INC64", "OP_CSWAP64",
    "OP_FETCH64", "OP_SET64", "OP_SWAP64", "OP_P32", "OP_FADD32", "OP_PUTMEM", "OP_GETMEM",
    "OP_FAND64", "OP_FOR64", "OP_FXOR64", "OP_NONE",
    "ROC_SHMEM_REDUCE_SYNC_SIZE", "ROC_SHMEM_BCAST_SYNC_SIZE", "NP_DTYPE",
]

SHORT, INT, LONG, LONGLONG, FLOAT, DOUBLE, BF16 = range(7)
SUM, MAX, MIN, PROD, AND, OR, XOR = range(7)
PUT, GET, PUT_NBI, GET_NBI = range(4)
STREAM_READ, STREAM_WRITE, STREAM_RUNTIME_FILL, STREAM_RUNTIME_COPY, STREAM_COPY = range(5)
THREAD, WAVE, WG, WG_SHARED = range(4)
(OP_P64, OP_FADD64, OP_ADD64, OP_FINC64, OP_INC64, OP_CSWAP64, OP_FETCH64, OP_SET64, OP_SWAP64,
 OP_P32, OP_FADD32, OP_PUTMEM, OP_GETMEM, OP_FAND64, OP_FOR64, OP_FXOR64) = range(16)
OP_NONE = 255
ROC_SHMEM_REDUCE_SYNC_SIZE = 256
ROC_SHMEM_BCAST_SYNC_SIZE = 256

NP_DTYPE = {SHORT: np.int16, INT: np.int32, LONG: np.int64, LONGLONG: np.int64,
            FLOAT: np.float32, DOUBLE: np.float64, BF16: np.uint16}

SMALL_OP_DTYPE = np.dtype([("kind", "<u4"), ("pe", "<u4"), ("offset", "<u8"),
                           ("value", "<i8"), ("aux", "<i8")])


class RocShmemError(RuntimeError):
    pass


def _check(rc):
    if rc != 0:
        raise RocShmemError(L.load().rsm_last_error().decode())


def Launch(wgs_per_pe=1, wg_size=256, tile=0, stream=None):
    return L.Launch(wgs_per_pe, wg_size, tile, getattr(stream, "h", stream))


def _launch(launch):
    return C.byref(launch if launch is not None else Launch())


# ---- lifecycle ---------------------------------------------------------------

def roc_shmem_init(num_pes=0, heap_size=0, num_blocks=0, sq_size=0):
    """reference: roc_shmem_init, library/src/roc_shmem.cpp:71-100.  Zero arguments
    fall back to ROC_SHMEM_NUM_PES / _HEAP_SIZE / _NUM_BLOCKS / _SQ_SIZE."""
    _check(L.load().rsm_init(num_pes, heap_size, num_blocks, sq_size))


def roc_shmem_finalize():
    _check(L.load().rsm_finalize())


def roc_shmem_n_pes():
    return L.load().rsm_n_pes()


def roc_shmem_malloc(nbytes):
    """Symmetric allocation; returns PE 0's address, or None (reference:
    roc_shmem_malloc, roc_shmem.cpp:118-126; power-of-two bins, 128-byte floor)."""
    p = L.load().rsm_malloc(nbytes)
    return p


def roc_shmem_free(addr):
    _check(L.load().rsm_free(addr))


def roc_shmem_ptr(addr, pe):
    return L.load().rsm_ptr(addr, pe)


def heap_base(pe):
    return L.load().rsm_heap_base(pe)


def heap_bytes_in_use():
    return L.load().rsm_heap_bytes_in_use()


def set_pacing(copy_bytes_per_tick=0, reduce_bytes_per_tick=0):
    """Lockstep pacing rates of large sharded copies / reductions (rsm_set_pacing); 0 = off."""
    _check(L.load().rsm_set_pacing(int(copy_bytes_per_tick), int(reduce_bytes_per_tick)))


def tune_reduce_pacing(dtype, op, dest, source, nreduce, PE_start, logPE_stride, PE_size, pSync, launch=None):
    """Measure and set the pacing rate of sharded reductions on this card, for this reduction
    (rsm_tune_reduce_pacing).  Returns {"rate", "free_ms", "paced_ms"}; rate 0 = pacing stays off."""
    rate, free_ms, paced_ms = C.c_uint(0), C.c_float(0), C.c_float(0)
    _check(L.load().rsm_tune_reduce_pacing(dtype, op, _addr(dest), _addr(source), nreduce, PE_start,
                                           logPE_stride, PE_size, _addr(pSync), _launch(launch),
                                           C.byref(rate), C.byref(free_ms), C.byref(paced_ms)))
    return {"rate": rate.value, "free_ms": free_ms.value, "paced_ms": paced_ms.value}


def get_pacing():
    a, b = C.c_uint(0), C.c_uint(0)
    _check(L.load().rsm_get_pacing(C.byref(a), C.byref(b)))
    return a.value, b.value


def take_status():
    return L.load().rsm_take_status()


def synchronize():
    _check(L.load().rsm_synchronize())


def roc_shmem_barrier_all():
    synchronize()


# ---- teams ----------------------------------------------------------------------

def roc_shmem_team_world():
    return L.load().rsm_team_world()


def roc_shmem_team_split_strided(parent, start, stride, size):
    """Returns (status, team): status 0 / -1 as the reference does
    (roc_shmem.cpp:216-297); team 0 stands for ROC_SHMEM_TEAM_INVALID."""
    out = C.c_uint64(0)
    rc = L.load().rsm_team_split_strided(parent, start, stride, size, C.byref(out))
    return (0 if rc == 0 else -1), out.value


def roc_shmem_team_destroy(team):
    _check(L.load().rsm_team_destroy(team))


def roc_shmem_team_n_pes(team):
    return L.load().rsm_team_n_pes(team)


def roc_shmem_team_translate_pe(src_team, src_pe, dst_team):
    return L.load().rsm_team_translate_pe(src_team, src_pe, dst_team)


# ---- symmetric arrays --------------------------------------------------------------

class SymArray:
    """A symmetric allocation of ``count`` elements of ``np_dtype`` in every PE's slice."""

    def __init__(self, count, np_dtype, fill=None):
        self.count = int(count)
        self.dtype = np.dtype(np_dtype)
        self.nbytes = self.count * self.dtype.itemsize
        self.addr = roc_shmem_malloc(max(self.nbytes, 1))
        if not self.addr:
            raise RocShmemError("symmetric heap exhausted (%d bytes)" % self.nbytes)
        if fill is not None:
            self.fill(fill)

    @property
    def offset(self):
        """Byte offset of the object inside every PE's slice."""
        return self.addr - heap_base(0)

    def pe_addr(self, pe):
        return roc_shmem_ptr(self.addr, pe)

    def write(self, pe, values, elem_offset=0):
        a = np.ascontiguousarray(values, dtype=self.dtype)
        assert elem_offset + a.size <= self.count
        _check(L.load().rsm_copy_to_device(self.pe_addr(pe) + elem_offset * self.dtype.itemsize,
                                           a.ctypes.data, a.nbytes))

    def read(self, pe, count=None, elem_offset=0):
        count = self.count - elem_offset if count is None else count
        out = np.empty(count, dtype=self.dtype)
        _check(L.load().rsm_copy_to_host(out.ctypes.data,
                                         self.pe_addr(pe) + elem_offset * self.dtype.itemsize,
                                         out.nbytes))
        return out

    def fill(self, byte_value, pe=None):
        pes = range(roc_shmem_n_pes()) if pe is None else [pe]
        for p in pes:
            _check(L.load().rsm_fill(self.pe_addr(p), byte_value, self.nbytes))

    def free(self):
        if self.addr:
            roc_shmem_free(self.addr)
            self.addr = None


def sym_array(count, np_dtype, fill=None):
    return SymArray(count, np_dtype, fill)


class device_array:
    """Ordinary (non-symmetric) device memory with numpy I/O."""

    def __init__(self, values=None, nbytes=None):
        if values is not None:
            a = np.ascontiguousarray(values)
            nbytes = a.nbytes
        self.nbytes = nbytes
        self.addr = L.load().rsm_device_alloc(max(nbytes, 1))
        if not self.addr:
            raise RocShmemError("device allocation failed")
        if values is not None:
            _check(L.load().rsm_copy_to_device(self.addr, a.ctypes.data, a.nbytes))

    def read(self, np_dtype, count):
        out = np.empty(count, dtype=np_dtype)
        _check(L.load().rsm_copy_to_host(out.ctypes.data, self.addr, out.nbytes))
        return out

    def fill(self, byte_value):
        _check(L.load().rsm_fill(self.addr, byte_value, self.nbytes))

    def free(self):
        if self.addr:
            _check(L.load().rsm_device_free(self.addr))
            self.addr = None


class Event:
    def __init__(self):
        self.h = L.load().rsm_event_create()

    def record(self, stream=None):
        _check(L.load().rsm_event_record(self.h, getattr(stream, "h", stream)))

    def elapsed_ms(self, stop):
        ms = C.c_float(0)
        _check(L.load().rsm_event_elapsed_ms(self.h, stop.h, C.byref(ms)))
        return ms.value

    def destroy(self):
        if self.h:
            L.load().rsm_event_destroy(self.h)
            self.h = None


class Stream:
    def __init__(self):
        self.h = L.load().rsm_stream_create()
        if not self.h:
            raise RocShmemError(L.load().rsm_last_error().decode())

    def synchronize(self):
        _check(L.load().rsm_stream_synchronize(self.h))

    def destroy(self):
        if self.h:
            L.load().rsm_stream_destroy(self.h)
            self.h = None


class Graph:
    """A recorded run of data-path calls: ``with Graph.capture(stream) as g:`` records every
    data-path call whose launch names ``stream``; ``g.launch(stream)`` replays them as one
    submission."""

    def __init__(self, stream):
        self.stream = stream
        self.h = None

    @classmethod
    def capture(cls, stream):
        return cls(stream)

    def __enter__(self):
        _check(L.load().rsm_capture_begin(self.stream.h))
        return self

    def __exit__(self, exc_type, exc, tb):
        self.h = L.load().rsm_capture_end(self.stream.h)
        if not self.h and exc_type is None:
            raise RocShmemError(L.load().rsm_last_error().decode())
        return False

    def launch(self, stream=None):
        _check(L.load().rsm_graph_launch(self.h, (stream or self.stream).h))

    def destroy(self):
        if self.h:
            L.load().rsm_graph_destroy(self.h)
            self.h = None


# ---- data path -------------------------------------------------------------------------

def _addr(x):
    return x.addr if hasattr(x, "addr") else x


def roc_shmem_to_all(dtype, op, dest, source, nreduce, PE_start, logPE_stride, PE_size, pWrk,
                     pSync, launch=None):
    """roc_shmem_ctx_<T>_<op>_wg_to_all over an active set (reference:
    roc_shmem.hpp:837-851), issued by ``launch.wgs_per_pe`` workgroups per PE."""
    _check(L.load().rsm_to_all(dtype, op, _addr(dest), _addr(source), nreduce, PE_start,
                               logPE_stride, PE_size, _addr(pWrk) if pWrk is not None else None,
                               _addr(pSync), _launch(launch)))


def roc_shmem_to_all_noalloc(dtype, op, dest, source, nreduce, PE_start, logPE_stride, PE_size,
                             launch=None):
    """The sharded form of roc_shmem_to_all without a caller-allocated pSync: the flags live in
    an array of the library's own and the call allocates nothing (rsm_to_all_noalloc)."""
    _check(L.load().rsm_to_all_noalloc(dtype, op, _addr(dest), _addr(source), nreduce, PE_start,
                                       logPE_stride, PE_size, _launch(launch)))


def roc_shmem_team_to_all(dtype, op, team, dest, source, nreduce, launch=None):
    _check(L.load().rsm_to_all_team(dtype, op, team, _addr(dest), _addr(source), nreduce,
                                    _launch(launch)))


def roc_shmem_rma(kind, granularity, dest, source, msg_bytes, n_msgs=1, dst_stride=None,
                  src_stride=None, pe_shift=1, launch=None):
    """roc_shmemx_ctx_{put,get}mem[_nbi]_{wg,wave} / roc_shmem_ctx_{put,get}mem[_nbi]
    from every PE p to PE (p + pe_shift) % n_pes."""
    dst_stride = msg_bytes if dst_stride is None else dst_stride
    src_stride = msg_bytes if src_stride is None else src_stride
    _check(L.load().rsm_rma(kind, granularity, _addr(dest), _addr(source), msg_bytes, n_msgs,
                            dst_stride, src_stride, pe_shift, _launch(launch)))


def stream_probe(kind, buf, bytes_per_pe, checksum=None, seed=0, launch=None):
    """Plain read-only / write-only stream over `buf` in every PE's slice (rsm_stream_probe)."""
    _check(L.load().rsm_stream_probe(kind, _addr(buf), bytes_per_pe, _addr(checksum) if checksum is not None else None,
                                     seed, _launch(launch)))


def roc_shmem_broadcast(elem_size, dest, source, nelem, PE_root, PE_start, logPE_stride, PE_size,
                        pSync, launch=None):
    _check(L.load().rsm_broadcast(elem_size, _addr(dest), _addr(source), nelem, PE_root, PE_start,
                                  logPE_stride, PE_size, _addr(pSync), _launch(launch)))


def roc_shmem_team_broadcast(elem_size, team, dest, source, nelem, PE_root, launch=None):
    _check(L.load().rsm_broadcast_team(elem_size, team, _addr(dest), _addr(source), nelem, PE_root,
                                       _launch(launch)))


def roc_shmem_alltoall(elem_size, team, dest, source, nelem, launch=None):
    _check(L.load().rsm_alltoall(elem_size, team, _addr(dest), _addr(source), nelem,
                                 _launch(launch)))


def roc_shmem_fcollect(elem_size, team, dest, source, nelem, launch=None):
    _check(L.load().rsm_fcollect(elem_size, team, _addr(dest), _addr(source), nelem,
                                 _launch(launch)))


def roc_shmem_wg_barrier_all(iterations=1, launch=None):
    _check(L.load().rsm_barrier_all(iterations, _launch(launch)))


def roc_shmem_small_ops(ops_dev, n_ops, fetched_dev=None, launch=None):
    _check(L.load().rsm_small_ops(_addr(ops_dev), n_ops,
                                  _addr(fetched_dev) if fetched_dev is not None else None,
                                  _launch(launch)))


# ---- send queues and wave-level drivers -----------------------------------------------------

def sq_reset():
    _check(L.load().rsm_sq_reset())


def sq_read(pe, block, index):
    out = np.zeros(8, dtype=np.uint64)
    _check(L.load().rsm_sq_read(pe, block, index, out.ctypes.data))
    return out


def sq_image(pe, block, entries):
    out = np.zeros(entries * 64, dtype=np.uint8)
    _check(L.load().rsm_sq_image(pe, block, out.ctypes.data, out.nbytes))
    return out.reshape(entries, 64)


def sq_state(pe, block):
    a, b, c = C.c_uint32(0), C.c_uint32(0), C.c_uint32(0)
    mailbox = np.zeros(2, dtype=np.uint64)
    _check(L.load().rsm_sq_state(pe, block, C.byref(a), C.byref(b), C.byref(c),
                                 mailbox.ctypes.data))
    return {"sq_counter": a.value, "published": b.value, "atomic_counter": c.value,
            "mailbox": mailbox}


def sq_constants(pe, block):
    qp, sig, lkey, alkey, base, n = (C.c_uint32(0), C.c_uint64(0), C.c_uint32(0), C.c_uint32(0),
                                     C.c_uint64(0), C.c_uint32(0))
    _check(L.load().rsm_sq_constants(pe, block, C.byref(qp), C.byref(sig), C.byref(lkey),
                                     C.byref(alkey), C.byref(base), C.byref(n)))
    return {"ctrl_qp_sq": qp.value, "ctrl_sig": sig.value, "lkey": lkey.value,
            "atomic_lkey": alkey.value, "atomic_ret_base": base.value, "max_nwqe": n.value}


def sq_rkey(dest_pe):
    k = C.c_uint32(0)
    _check(L.load().rsm_sq_rkey(dest_pe, C.byref(k)))
    return k.value


def sq_flush_target(pe):
    """(address, key) a fence's entry on a live queue names for PE ``pe`` (rsm_sq_flush_target)."""
    a, k = C.c_uint64(0), C.c_uint32(0)
    _check(L.load().rsm_sq_flush_target(pe, C.byref(a), C.byref(k)))
    return a.value, k.value


class ConsumeTotals(C.Structure):
    _fields_ = [(n, C.c_uint64) for n in ("retired", "writes", "reads", "atomics", "bytes",
                                          "completions", "lost", "rejected", "local_skipped")]

    def as_dict(self):
        return {n: int(getattr(self, n)) for n, _ in self._fields_}


def sq_consume(pe=-1, block=-1, target_arena=None):
    """Consumer pass over the rings of (pe, block), -1 = all (rsm_sq_consume): retire what
    they published, write completion entries and, when ``target_arena`` (a DeviceArray laid
    out like the arena) is given, execute every entry against it.  Returns the totals."""
    t = ConsumeTotals()
    _check(L.load().rsm_sq_consume(pe, block, _addr(target_arena) if target_arena is not None else None,
                                   C.byref(t)))
    return t.as_dict()


def sq_set_mode(queue):
    """False: rings are logs that wrap freely; True: slots are freed by sq_consume only."""
    _check(L.load().rsm_sq_set_mode(1 if queue else 0))


def sq_consumer_start():
    """Start the consumer that retires ring entries while producers post (rsm_sq_consumer_start)."""
    _check(L.load().rsm_sq_consumer_start())


def sq_consumer_stop():
    """Let the live consumer drain the rings and stop it; returns the totals of what it retired."""
    t = ConsumeTotals()
    rc = L.load().rsm_sq_consumer_stop(C.byref(t))
    _check(rc)
    return t.as_dict()


def sq_consumer_running():
    return bool(L.load().rsm_sq_consumer_running())


def cq_reader_state(pe, block):
    a, b, c = C.c_uint32(0), C.c_uint32(0), C.c_uint32(0)
    _check(L.load().rsm_cq_reader_state(pe, block, C.byref(a), C.byref(b), C.byref(c)))
    return {"cq_consumer": a.value, "quiet_counter": b.value, "cq_doorbell_record": c.value}


def sq_consumer_state(pe, block):
    a, b = C.c_uint32(0), C.c_uint32(0)
    _check(L.load().rsm_sq_consumer_state(pe, block, C.byref(a), C.byref(b)))
    return {"consumed": a.value, "cq_producer": b.value}


def cq_image(pe, block, entries):
    out = np.zeros(entries * 64, dtype=np.uint8)
    _check(L.load().rsm_cq_image(pe, block, out.ctypes.data, out.nbytes))
    return out.reshape(entries, 64)


def atomic_ret_image(pe, block, words=4096):
    out = np.zeros(words, dtype=np.uint64)
    _check(L.load().rsm_atomic_ret_image(pe, block, out.ctypes.data, out.nbytes))
    return out


def arena():
    """(base address, bytes, slice stride) of the arena that holds every PE slice."""
    base, nbytes, stride = C.c_void_p(0), C.c_size_t(0), C.c_size_t(0)
    _check(L.load().rsm_arena(C.byref(base), C.byref(nbytes), C.byref(stride)))
    return base.value, nbytes.value, stride.value


def read_device(addr, nbytes):
    """Bytes [addr, addr+nbytes) of device memory as a uint8 array."""
    out = np.empty(nbytes, dtype=np.uint8)
    _check(L.load().rsm_copy_to_host(out.ctypes.data, _addr(addr), nbytes))
    return out


def write_device(addr, values):
    a = np.ascontiguousarray(values)
    _check(L.load().rsm_copy_to_device(_addr(addr), a.ctypes.data, a.nbytes))


def kat_fetch_incr(lane_mask, n_wgs, wg_size):
    out = np.zeros(n_wgs * wg_size, dtype=np.uint64)
    ctr = C.c_uint64(0)
    _check(L.load().rsm_kat_fetch_incr(lane_mask, n_wgs, wg_size, out.ctypes.data, C.byref(ctr)))
    return out, ctr.value


def kat_coalesce(lane_mask, pe, src, dst, size):
    pe = np.ascontiguousarray(pe, dtype=np.int32)
    src = np.ascontiguousarray(src, dtype=np.uint64)
    dst = np.ascontiguousarray(dst, dtype=np.uint64)
    size = np.ascontiguousarray(size, dtype=np.uint64)
    must = np.zeros(64, dtype=np.uint8)
    out = np.zeros(64, dtype=np.uint64)
    _check(L.load().rsm_kat_coalesce(lane_mask, pe.ctypes.data, src.ctypes.data, dst.ctypes.data,
                                     size.ctypes.data, must.ctypes.data, out.ctypes.data))
    return must, out
