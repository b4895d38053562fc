"""rsm_to_all_noalloc (the reduction entry point that allocates nothing) against rsm_to_all.

The two entry points run the same sharded reduction; what differs is where the flag
barriers keep their flags: a caller-allocated symmetric pSync (rsm_to_all) or the
library's own file-scope device array (rsm_to_all_noalloc).  Results must be
bit-identical, and identical to the CPU oracle for integer types.  The array is
shared by all calls on the GPU and keeps the previous call's contents, so every case
makes two calls in a row, the second with a smaller input and another launch shape.
"""
import numpy as np
import pytest

import oracle
import roc_shmem_amd as rs
from helpers import random_values, runtime

pytestmark = pytest.mark.gpu


def both_ways(dtype, op, n_pes, n, seed, wgs, wg_size, pe_start=0, log_stride=0, pe_size=None):
    pe_size = n_pes if pe_size is None else pe_size
    npd = rs.NP_DTYPE[dtype]
    es = np.dtype(npd).itemsize
    src = rs.sym_array(n, npd)
    dst_ref = rs.sym_array(n, npd, fill=0x5A)
    dst_new = rs.sym_array(n, npd, fill=0x5A)
    psync = rs.sym_array(wgs * rs.ROC_SHMEM_REDUCE_SYNC_SIZE, np.int64, fill=0)
    heap = oracle.Heap(n_pes, 2 * n * es)
    for p in range(n_pes):
        vals = random_values(dtype, n, seed * 100 + p)
        src.write(p, vals)
        heap.view(p, 0, n, npd)[:] = vals
        heap.view(p, n * es, n, npd)[:] = np.frombuffer(b"\x5a" * (n * es), dtype=npd)
    launch = rs.Launch(wgs_per_pe=wgs, wg_size=wg_size)
    rs.roc_shmem_to_all(dtype, op, dst_ref, src, n, pe_start, log_stride, pe_size, None, psync, launch)
    rs.roc_shmem_to_all_noalloc(dtype, op, dst_new, src, n, pe_start, log_stride, pe_size, launch)
    rs.synchronize()
    oracle.to_all(heap, dtype, op, n * es, 0, n, pe_start, log_stride, pe_size)
    for p in range(n_pes):
        ref, new = dst_ref.read(p), dst_new.read(p)
        assert np.array_equal(ref.view(np.uint8), new.view(np.uint8)), \
            "PE %d: rsm_to_all_noalloc differs from rsm_to_all" % p
        if dtype not in (rs.FLOAT, rs.DOUBLE, rs.BF16):
            assert np.array_equal(new, heap.view(p, n * es, n, npd)), "PE %d differs from the oracle" % p
    for a in (psync, dst_new, dst_ref, src):
        a.free()


def test_two_calls_in_a_row_second_one_smaller():
    with runtime(8, heap_size=64 << 20):
        both_ways(rs.LONG, rs.SUM, 8, (1 << 18) + 37, seed=1, wgs=16, wg_size=512)
        both_ways(rs.LONG, rs.SUM, 8, 4099, seed=2, wgs=2, wg_size=256)
        both_ways(rs.FLOAT, rs.SUM, 8, 100003, seed=3, wgs=4, wg_size=1024)
        both_ways(rs.INT, rs.XOR, 8, 5, seed=4, wgs=1, wg_size=64)


def test_active_set_and_other_types():
    with runtime(8, heap_size=32 << 20):
        both_ways(rs.SHORT, rs.MAX, 8, 70001, seed=5, wgs=8, wg_size=256, pe_start=1, log_stride=1, pe_size=3)
        both_ways(rs.BF16, rs.SUM, 8, 33000, seed=6, wgs=3, wg_size=512, pe_start=0, log_stride=2, pe_size=2)
        both_ways(rs.DOUBLE, rs.MIN, 8, 1000, seed=7, wgs=1, wg_size=128)


def test_a_small_grid_after_a_large_one_shares_the_same_flag_array():
    # Slices of the flag array are handed out by (PE, workgroup) for the grid of the call, so a
    # call with another launch shape lays its slices over what the previous call used; the
    # entry point clears what it is going to use before the reduction starts.
    with runtime(4, heap_size=16 << 20):
        both_ways(rs.INT, rs.SUM, 4, 3000, seed=8, wgs=4, wg_size=256)
        n = 9000
        src = rs.sym_array(n, np.int32)
        dst = rs.sym_array(n, np.int32, fill=0)
        vals = [random_values(rs.INT, n, 900 + p) for p in range(4)]
        for p in range(4):
            src.write(p, vals[p])
        # a first reduction over many slices, then a smaller grid over the same array
        rs.roc_shmem_to_all_noalloc(rs.INT, rs.SUM, dst, src, n, 0, 0, 4, rs.Launch(32, 256))
        rs.roc_shmem_to_all_noalloc(rs.INT, rs.SUM, dst, src, n // 3, 0, 0, 4, rs.Launch(2, 64))
        rs.synchronize()
        want = vals[0] + vals[1] + vals[2] + vals[3]
        for p in range(4):
            assert np.array_equal(dst.read(p), want)
        dst.free()
        src.free()


def test_sizes_beyond_the_array_are_refused():
    with runtime(16, heap_size=8 << 20, num_blocks=4):
        src = rs.sym_array(1024, np.int64)
        dst = rs.sym_array(1024, np.int64, fill=0)
        for p in range(16):
            src.write(p, np.ones(1024, np.int64))
        with pytest.raises(rs.RocShmemError, match="exceed the 2048"):
            rs.roc_shmem_to_all_noalloc(rs.LONG, rs.SUM, dst, src, 1024, 0, 0, 16, rs.Launch(129, 64))
        with pytest.raises(rs.RocShmemError, match="tile must be 0"):
            rs.roc_shmem_to_all_noalloc(rs.LONG, rs.SUM, dst, src, 1024, 0, 0, 16, rs.Launch(2, 64, 256))
        # the largest grid the array has room for still works
        rs.roc_shmem_to_all_noalloc(rs.LONG, rs.SUM, dst, src, 1024, 0, 0, 16, rs.Launch(128, 64))
        rs.synchronize()
        for p in range(16):
            assert (dst.read(p) == 16).all()
        dst.free()
        src.free()


def _free_device_memory():
    """Free bytes of device memory as the HIP runtime reports them (hipMemGetInfo, straight from
    the runtime's library, which the data-path library has loaded already)."""
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")
    free, total = ctypes.c_size_t(0), ctypes.c_size_t(0)
    assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
    return free.value


def test_calls_allocate_nothing_and_can_be_recorded_in_a_graph():
    # What the entry point is for: callers that cannot allocate, a stream under capture among
    # them.  Two calls (the second smaller, another launch shape) are recorded into one graph and
    # replayed with new inputs, with eager work and synchronisations between the replays; every
    # replay is compared with the oracle, and neither the symmetric heap nor the device's free
    # memory moves across the calls.
    n_pes, n1, n2 = 8, 70001, 4099
    with runtime(n_pes, heap_size=32 << 20):
        stream = rs.Stream()
        src = rs.sym_array(n1, np.int64)
        dst1 = rs.sym_array(n1, np.int64, fill=0)
        dst2 = rs.sym_array(n2, np.int64, fill=0)
        big, small = rs.Launch(16, 512, 0, stream), rs.Launch(2, 256, 0, stream)

        def calls():
            rs.roc_shmem_to_all_noalloc(rs.LONG, rs.SUM, dst1, src, n1, 0, 0, n_pes, big)
            rs.roc_shmem_to_all_noalloc(rs.LONG, rs.XOR, dst2, src, n2, 0, 0, n_pes, small)

        def check(vals):
            want1 = np.sum(np.stack(vals), axis=0, dtype=np.int64)
            want2 = np.bitwise_xor.reduce(np.stack(vals)[:, :n2], axis=0)
            for p in range(n_pes):
                assert np.array_equal(dst1.read(p), want1), p
                assert np.array_equal(dst2.read(p), want2), p

        def new_inputs(seed):
            vals = [random_values(rs.LONG, n1, seed * 100 + p) for p in range(n_pes)]
            for p in range(n_pes):
                src.write(p, vals[p])
                dst1.fill(0, pe=p)
                dst2.fill(0, pe=p)
            return vals

        vals = new_inputs(1)
        calls()                                  # eager, also the first use on this device
        stream.synchronize()
        check(vals)
        heap_before, free_before = rs.heap_bytes_in_use(), _free_device_memory()
        for _ in range(20):
            calls()
        stream.synchronize()
        assert rs.heap_bytes_in_use() == heap_before
        assert _free_device_memory() == free_before, "a call changed the device's free memory"
        with rs.Graph.capture(stream) as graph:
            calls()
        # (the HIP runtime keeps device memory for an instantiated graph, the caller's, not the
        # entry point's: free memory is compared again from after the first replay)
        vals = new_inputs(9)
        graph.launch()
        stream.synchronize()
        check(vals)
        free_before = _free_device_memory()
        for seed in (2, 3, 4, 5):
            vals = new_inputs(seed)
            graph.launch()
            stream.synchronize()
            check(vals)
            # eager work of the same kind between the replays
            rs.roc_shmem_to_all_noalloc(rs.LONG, rs.MAX, dst2, src, n2, 0, 0, n_pes, small)
            stream.synchronize()
        assert rs.heap_bytes_in_use() == heap_before
        assert _free_device_memory() == free_before
        assert rs.take_status() == 0
        # a refused call queues nothing: the operator is not defined for the type
        with pytest.raises(rs.RocShmemError, match="operator not defined"):
            rs.roc_shmem_to_all_noalloc(rs.FLOAT, rs.XOR, dst2, src, n2, 0, 0, n_pes, small)
        graph.destroy()
        stream.destroy()
        for a in (dst2, dst1, src):
            a.free()
