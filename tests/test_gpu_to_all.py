"""Parity of roc_shmem_ctx_<T>_<op>_wg_to_all with the CPU oracle (C ABI path)."""
import numpy as np
import pytest

import oracle
import roc_shmem_amd as rs
from helpers import check_fp, random_values, runtime

pytestmark = pytest.mark.gpu

INT_TYPES = [rs.SHORT, rs.INT, rs.LONG, rs.LONGLONG]
INT_OPS = [rs.SUM, rs.MAX, rs.MIN, rs.PROD, rs.AND, rs.OR, rs.XOR]
FP_CASES = [(rs.FLOAT, op) for op in (rs.SUM, rs.MAX, rs.MIN, rs.PROD)] + \
           [(rs.DOUBLE, op) for op in (rs.SUM, rs.MAX, rs.MIN, rs.PROD)] + \
           [(rs.BF16, op) for op in (rs.SUM, rs.MAX, rs.MIN)]


def run_case(dtype, op, n_pes, n, seed, pe_start=0, log_stride=0, pe_size=None, wgs=1, wg_size=256,
             tile=0, kind="full", in_place=False, elem_shift=0, team=None):
    """Run one reduction on the GPU and on the oracle; returns (got per PE, oracle heap, offsets)."""
    pe_size = n_pes if pe_size is None else pe_size
    npd = rs.NP_DTYPE[dtype]
    es = np.dtype(npd).itemsize
    total = n + elem_shift
    src = rs.sym_array(total, npd)
    dst = src if in_place else rs.sym_array(total, npd)
    psync = rs.sym_array(wgs * rs.ROC_SHMEM_REDUCE_SYNC_SIZE, np.int64, fill=0)
    stride = 2 * total * es + 64
    heap = oracle.Heap(n_pes, stride)
    src_off, dst_off = 0, (0 if in_place else total * es)
    for p in range(n_pes):
        vals = random_values(dtype, total, seed * 1000 + p, kind)
        src.write(p, vals)
        heap.view(p, src_off, total, npd)[:] = vals
        if not in_place:
            guard = np.full(total, 0x5A5A5A5A5A5A5A5A, dtype=np.uint64).view(np.uint8)[:total * es].view(npd)
            dst.write(p, guard)
            heap.view(p, dst_off, total, npd)[:] = guard
    launch = rs.Launch(wgs_per_pe=wgs, wg_size=wg_size, tile=tile)
    d_addr = dst.addr + elem_shift * es
    s_addr = src.addr + elem_shift * es
    if team is not None:
        rs.roc_shmem_team_to_all(dtype, op, team, d_addr, s_addr, n, launch)
    else:
        rs.roc_shmem_to_all(dtype, op, d_addr, s_addr, n, pe_start, log_stride, pe_size, None, psync,
                            launch)
    rs.synchronize()
    truth = None
    if dtype in (rs.FLOAT, rs.DOUBLE, rs.BF16):
        truth = (oracle.to_all_f64(heap, dtype, op, src_off + elem_shift * es, n, pe_start, log_stride, pe_size),
                 oracle.abs_sum_f64(heap, dtype, src_off + elem_shift * es, n, pe_start, log_stride, pe_size))
    # The library's arithmetic, restated: in-type folds, except float sum/prod (folded in double)
    # and bfloat16 sum (folded in float), ascending members, rounded once.  Every comparison with
    # `expect` below is therefore bit for bit, floating point included.
    oracle.to_all_rounded_once(heap, dtype, op, dst_off + elem_shift * es, src_off + elem_shift * es, n,
                               pe_start, log_stride, pe_size)
    got = [dst.read(p) for p in range(n_pes)]
    # pSync must be back to ROC_SHMEM_SYNC_VALUE everywhere
    for p in range(n_pes):
        assert not psync.read(p).any(), "pSync not restored on PE %d" % p
    expect = [heap.view(p, dst_off, total, npd).copy() for p in range(n_pes)]
    src.free()
    if not in_place:
        dst.free()
    psync.free()
    return got, expect, truth


def members(n_pes, pe_start, log_stride, pe_size):
    return [pe_start + (k << log_stride) for k in range(pe_size)]


@pytest.mark.parametrize("dtype", INT_TYPES)
@pytest.mark.parametrize("op", INT_OPS)
def test_integer_ops_bit_exact(dtype, op):
    with runtime(4):
        got, expect, _ = run_case(dtype, op, 4, 4099, seed=11 + dtype * 7 + op)
        for p in range(4):
            assert np.array_equal(got[p], expect[p]), "PE %d differs" % p


@pytest.mark.parametrize("dtype,op", FP_CASES)
@pytest.mark.parametrize("kind", ["normal", "lognormal"])
def test_floating_point_within_tolerance(dtype, op, kind):
    with runtime(8):
        n = 6001
        got, expect, (ref64, abs64) = run_case(dtype, op, 8, n, seed=5 + dtype + op, kind=kind)
        for p in range(8):
            # bit-identical to the restated fold (exact selection for max / min, the wide fold
            # rounded once for sum / prod) ...
            assert np.array_equal(got[p].view(np.uint8), expect[p].view(np.uint8))
            # ... and within the stated tolerance of the long-double truth
            if op in (rs.MAX, rs.MIN):
                pass
            elif op == rs.SUM:
                check_fp(dtype, got[p], ref64, abs64)
            else:  # PROD: relative to the magnitude of the product itself
                check_fp(dtype, got[p], ref64, np.zeros_like(abs64))
            # every PE holds the same bits
            assert np.array_equal(got[p].view(np.uint8), got[0].view(np.uint8))


@pytest.mark.parametrize("n", [1, 2, 3, 15, 16, 17, 255, 1024, 1025])
def test_sizes_and_tails(n):
    with runtime(4):
        got, expect, _ = run_case(rs.INT, rs.SUM, 4, n, seed=n)
        for p in range(4):
            assert np.array_equal(got[p], expect[p])


def test_zero_elements_is_a_no_op():
    with runtime(4):
        dst = rs.sym_array(64, np.int64, fill=0x11)
        src = rs.sym_array(64, np.int64, fill=0x22)
        psync = rs.sym_array(256, np.int64, fill=0)
        rs.roc_shmem_to_all(rs.LONG, rs.SUM, dst, src, 0, 0, 0, 4, None, psync)
        rs.synchronize()
        for p in range(4):
            assert (dst.read(p).view(np.uint8) == 0x11).all()


@pytest.mark.parametrize("shift", [1, 3])
def test_arrays_shifted_alike_off_the_vector_boundary(shift):
    with runtime(4):
        got, expect, _ = run_case(rs.INT, rs.XOR, 4, 1000, seed=77, elem_shift=shift)
        for p in range(4):
            assert np.array_equal(got[p], expect[p])  # includes the untouched leading guard


@pytest.mark.parametrize("dtype,dst_shift,src_shift", [
    (rs.INT, 1, 2), (rs.INT, 0, 3), (rs.LONG, 1, 0), (rs.LONGLONG, 3, 6),
    (rs.SHORT, 2, 4),      # two-byte elements an even number apart: vector path
    (rs.SHORT, 1, 2),      # an odd number apart: element by element
    (rs.SHORT, 5, 0)])
@pytest.mark.parametrize("n,wgs", [(37, 1), (3000, 2), (70001, 3)])
def test_source_and_destination_shifted_differently(dtype, dst_shift, src_shift, n, wgs):
    # sizes below 4 KiB, below 64 KiB and above: the vector body starts at the destination's next
    # 16-byte, 128-byte and 1 KiB boundary; bytes around the destination stay as they were
    n_pes = 4
    npd = rs.NP_DTYPE[dtype]
    es = np.dtype(npd).itemsize
    total = n + 16
    with runtime(n_pes):
        src = rs.sym_array(total, npd)
        dst = rs.sym_array(total, npd)
        psync = rs.sym_array(wgs * rs.ROC_SHMEM_REDUCE_SYNC_SIZE, np.int64, fill=0)
        heap = oracle.Heap(n_pes, 2 * total * es + 64)
        for p in range(n_pes):
            vals = random_values(dtype, total, 900 + p)
            src.write(p, vals)
            heap.view(p, 0, total, npd)[:] = vals
            guard = np.full(total, 0x3C, np.uint8).repeat(es).view(npd)[:total]
            dst.write(p, guard)
            heap.view(p, total * es, total, npd)[:] = guard
        rs.roc_shmem_to_all(dtype, rs.SUM, dst.addr + dst_shift * es, src.addr + src_shift * es, n, 0, 0,
                            n_pes, None, psync, rs.Launch(wgs, 256))
        rs.synchronize()
        oracle.to_all(heap, dtype, rs.SUM, (total + dst_shift) * es, src_shift * es, n)
        for p in range(n_pes):
            assert np.array_equal(dst.read(p), heap.view(p, total * es, total, npd)), "PE %d" % p
            assert not psync.read(p).any()


def test_in_place():
    # reference: clients/sos_tests/reduce_in_place.cpp:58-69 (dest == source)
    with runtime(4):
        got, expect, _ = run_case(rs.LONG, rs.SUM, 4, 3000, seed=3, in_place=True)
        for p in range(4):
            assert np.array_equal(got[p], expect[p])


@pytest.mark.parametrize("pe_start,log_stride,pe_size", [(1, 0, 3), (0, 1, 4), (1, 1, 3), (2, 2, 2), (5, 0, 1)])
def test_active_sets(pe_start, log_stride, pe_size):
    # reference: clients/sos_tests/reduce_active_set.cpp:78-113; PEs outside the set keep their dest
    with runtime(8):
        got, expect, _ = run_case(rs.LONG, rs.MAX, 8, 2050, seed=21, pe_start=pe_start,
                                  log_stride=log_stride, pe_size=pe_size)
        for p in range(8):
            assert np.array_equal(got[p], expect[p]), "PE %d" % p


def test_tiled_over_many_workgroups_int64_c1_shape():
    # The int64 benchmark workload at reduced length: int64 sum, 4 slices,
    # values uniform in [-2^30, 2^30], dest pre-filled 0x5A.
    with runtime(4, heap_size=64 << 20):
        n = 1 << 18
        got, expect, _ = run_case(rs.LONG, rs.SUM, 4, n, seed=1, wgs=32, wg_size=256, kind="c1")
        for p in range(4):
            assert np.array_equal(got[p], expect[p])


@pytest.mark.parametrize("dtype,op,n,wgs,wg_size,shift,in_place", [
    (rs.INT, rs.XOR, 70001, 3, 128, 0, False),       # odd shard count, tail elements after the vectors
    (rs.SHORT, rs.SUM, 123457, 5, 64, 0, False),     # more passes than parts, 2-byte elements
    (rs.LONG, rs.MAX, 33333, 4, 256, 0, True),       # in place
    (rs.INT, rs.SUM, 50001, 4, 128, 1, False),       # unaligned arrays: the element path, cut into parts
    (rs.LONGLONG, rs.PROD, 9, 7, 64, 0, False),      # fewer elements than workgroups
    (rs.INT, rs.OR, 1 << 16, 6, 1024, 0, False)])    # fewer passes than parts
def test_one_reduction_shared_by_the_workgroups_of_a_pe(dtype, op, n, wgs, wg_size, shift, in_place):
    # roc_shmemx_ctx_<T>_<op>_wg_to_all_shard (extension): launch->tile == 0 and wgs_per_pe > 1
    with runtime(4):
        got, expect, _ = run_case(dtype, op, 4, n, seed=n, wgs=wgs, wg_size=wg_size, elem_shift=shift,
                                  in_place=in_place)
        for p in range(4):
            assert np.array_equal(got[p], expect[p]), "PE %d" % p


@pytest.mark.parametrize("dtype", [rs.FLOAT, rs.BF16, rs.DOUBLE])
def test_shared_reduction_floating_point_and_active_set(dtype):
    with runtime(8):
        got, expect, truth = run_case(dtype, rs.SUM, 8, 99991, seed=5, wgs=3, wg_size=256, pe_start=1,
                                      log_stride=1, pe_size=3, kind="lognormal")
        mem = members(8, 1, 1, 3)
        for p in range(8):
            if p in mem:
                check_fp(dtype, got[p], truth[0], truth[1])
                assert np.array_equal(got[p].view(np.uint8), got[mem[0]].view(np.uint8)), \
                    "every member holds the same bits"
            else:
                assert np.array_equal(got[p].view(np.uint8), expect[p].view(np.uint8)), "PE %d was written" % p


def test_arena_in_plain_device_memory():
    # ROC_SHMEM_HEAP_HOST_VISIBLE=0: hipMalloc instead of fine-grained memory; same results.
    import os
    os.environ["ROC_SHMEM_HEAP_HOST_VISIBLE"] = "0"
    try:
        with runtime(4):
            got, expect, _ = run_case(rs.LONG, rs.SUM, 4, 100003, seed=12, wgs=4, wg_size=256, kind="c1")
            for p in range(4):
                assert np.array_equal(got[p], expect[p])
            got, expect, truth = run_case(rs.FLOAT, rs.SUM, 4, 40000, seed=13, wgs=2)
            for p in range(4):
                check_fp(rs.FLOAT, got[p], truth[0], truth[1])
    finally:
        del os.environ["ROC_SHMEM_HEAP_HOST_VISIBLE"]


def test_repeated_tiles_reuse_one_psync_slice():
    with runtime(4):
        got, expect, _ = run_case(rs.INT, rs.SUM, 4, 40000, seed=9, wgs=2, wg_size=128, tile=1024)
        for p in range(4):
            assert np.array_equal(got[p], expect[p])


def test_team_form_world_and_split():
    with runtime(8):
        world = rs.roc_shmem_team_world()
        got, expect, _ = run_case(rs.INT, rs.SUM, 8, 5000, seed=4, team=world, wgs=4)
        for p in range(8):
            assert np.array_equal(got[p], expect[p])
        rc, team = rs.roc_shmem_team_split_strided(world, 1, 2, 3)
        assert rc == 0 and team
        got, expect, _ = run_case(rs.LONGLONG, rs.MIN, 8, 777, seed=8, team=team, pe_start=1,
                                  log_stride=1, pe_size=3, wgs=2)
        for p in range(8):
            assert np.array_equal(got[p], expect[p])
        rs.roc_shmem_team_destroy(team)


def test_closed_forms_of_the_reference_tests():
    # clients/sos_tests/to_all.cpp: sum of src=me -> npes(npes-1)/2 (:310-346);
    # max of src=me+i -> npes-1+i (:123-153); and of src=me -> 0 (:407-428);
    # or of (me+1)%4 -> 3 (:632,652); xor of me%2 -> (npes/2)%2 (:696-701);
    # prod of src=me+1 -> npes! (:471-503)
    npes, n = 8, 128
    with runtime(npes):
        src = rs.sym_array(n, np.int32)
        dst = rs.sym_array(n, np.int32)
        psync = rs.sym_array(256, np.int64, fill=0)
        i = np.arange(n, dtype=np.int32)

        def reduce(op, gen):
            for me in range(npes):
                src.write(me, gen(me))
            rs.roc_shmem_to_all(rs.INT, op, dst, src, n, 0, 0, npes, None, psync)
            rs.synchronize()
            return [dst.read(p) for p in range(npes)]

        for r in reduce(rs.SUM, lambda me: np.full(n, me, np.int32)):
            assert (r == npes * (npes - 1) // 2).all()
        for r in reduce(rs.MAX, lambda me: me + i):
            assert np.array_equal(r, npes - 1 + i)
        for r in reduce(rs.MIN, lambda me: me + i):
            assert np.array_equal(r, i)
        for r in reduce(rs.AND, lambda me: np.full(n, me, np.int32)):
            assert (r == 0).all()
        for r in reduce(rs.OR, lambda me: np.full(n, (me + 1) % 4, np.int32)):
            assert (r == 3).all()
        for r in reduce(rs.XOR, lambda me: np.full(n, me % 2, np.int32)):
            assert (r == (npes // 2) % 2).all()
        for r in reduce(rs.PROD, lambda me: np.full(n, me + 1, np.int32)):
            assert (r == 40320).all()
        # clients/functional_tests/tester.cpp:149-164: float sum of 1.0 over n PEs == n
        fsrc = rs.sym_array(512, np.float32)
        fdst = rs.sym_array(512, np.float32)
        for me in range(npes):
            fsrc.write(me, np.ones(512, np.float32))
        rs.roc_shmem_to_all(rs.FLOAT, rs.SUM, fdst, fsrc, 512, 0, 0, npes, None, psync)
        rs.synchronize()
        for p in range(npes):
            assert (fdst.read(p) == float(npes)).all()


@pytest.mark.parametrize("dtype", [rs.FLOAT, rs.LONG, rs.BF16])
def test_lds_staged_form_gives_the_same_bits(dtype):
    # ROC_SHMEM_REDUCE_LDS=1 sends float / long / bfloat16 sums of rsm_to_all (tile 0) through the
    # LDS-staged form of the sharded reduction: whole passes through LDS, the remainder the usual way.
    import os
    os.environ["ROC_SHMEM_REDUCE_LDS"] = "1"
    try:
        rs.roc_shmem_init(8, 64 << 20, 16, 1024)
    finally:
        del os.environ["ROC_SHMEM_REDUCE_LDS"]
    try:
        for n, wgs, wg_size, pe_size in (((1 << 20) + 4103, 4, 512, 8), (300001, 2, 1024, 8), (70000, 3, 256, 5),
                                         (4099, 1, 64, 8)):
            got, expect, _ = run_case(dtype, rs.SUM, 8, n, seed=31 + dtype, wgs=wgs, wg_size=wg_size,
                                      pe_size=pe_size)
            for p in range(8):
                assert np.array_equal(got[p].view(np.uint8), expect[p].view(np.uint8)), (n, wgs, wg_size, p)
        assert rs.take_status() == 0
    finally:
        rs.roc_shmem_finalize()
