"""Parity of the workgroup / wavefront / thread put and get with the CPU oracle."""
import numpy as np
import pytest

import oracle
import roc_shmem_amd as rs
from helpers import runtime

pytestmark = pytest.mark.gpu

GUARD = 0xA5


def run_rma(kind, gran, n_pes, msg_bytes, n_msgs, seed, pe_shift=1, src_mis=0, dst_mis=0, wgs=2,
            wg_size=256, stride_pad=0):
    """Every PE p moves n_msgs messages to/from PE (p+pe_shift)%n_pes; compares all slices."""
    msg_stride = msg_bytes + stride_pad
    span = msg_stride * n_msgs + 64
    src = rs.sym_array(span + 64, np.uint8)
    dst = rs.sym_array(span + 64, np.uint8)
    stride = 2 * (span + 64) + 256
    heap = oracle.Heap(n_pes, stride)
    s_off, d_off = 0, span + 64
    rng = np.random.default_rng(seed)
    for p in range(n_pes):
        payload = rng.integers(0, 256, size=span + 64, dtype=np.uint8)
        src.write(p, payload)
        heap.view(p, s_off, span + 64, np.uint8)[:] = payload
        dst.fill(GUARD, pe=p)
        heap.view(p, d_off, span + 64, np.uint8)[:] = GUARD
    rs.roc_shmem_rma(kind, gran, dst.addr + dst_mis, src.addr + src_mis, msg_bytes, n_msgs,
                     msg_stride, msg_stride, pe_shift, rs.Launch(wgs, wg_size))
    rs.synchronize()
    for p in range(n_pes):
        other = (p + pe_shift) % n_pes
        for m in range(n_msgs):
            if kind in (rs.PUT, rs.PUT_NBI):
                oracle.put(heap, d_off + dst_mis + m * msg_stride, s_off + src_mis + m * msg_stride,
                           msg_bytes, p, other)
            else:
                oracle.get(heap, d_off + dst_mis + m * msg_stride, s_off + src_mis + m * msg_stride,
                           msg_bytes, p, other)
    for p in range(n_pes):
        got = dst.read(p)
        exp = heap.view(p, d_off, span + 64, np.uint8)
        assert np.array_equal(got, exp), "PE %d: first difference at byte %d" % (
            p, int(np.argmax(got != exp)))
        assert np.array_equal(src.read(p), heap.view(p, s_off, span + 64, np.uint8))
    src.free()
    dst.free()


@pytest.mark.parametrize("kind", [rs.PUT, rs.GET, rs.PUT_NBI, rs.GET_NBI])
@pytest.mark.parametrize("gran", [rs.WG, rs.WAVE, rs.THREAD])
def test_kinds_and_granularities(kind, gran):
    with runtime(4):
        run_rma(kind, gran, 4, 1000, 9, seed=kind * 3 + gran)


@pytest.mark.parametrize("kind", [rs.PUT_NBI, rs.GET_NBI])
@pytest.mark.parametrize("gran,msg_bytes,wgs,wg_size,n_msgs", [
    # windows of 64 non-blocking calls and a quiet per workgroup (wave), as the reference's
    # message-rate kernel issues them (primitive_mr_tester.cpp:44-49): three whole windows per
    # workgroup (wave) and part of a fourth; 64 guard bytes between neighbouring messages
    (rs.WG, 4096, 4, 256, 64 * 4 * 3 + 7),
    (rs.WG, 65536, 4, 256, 64 * 4 * 3 + 7),
    (rs.WG, 4096, 3, 1024, 64 * 3 * 2 + 1),
    (rs.WAVE, 4096, 2, 256, 64 * 8 * 3 + 13),
    (rs.WAVE, 65536, 2, 128, 64 * 4 * 2 + 5),
    (rs.THREAD, 96, 1, 64, 64 * 64 * 2 + 9),
])
def test_windows_of_non_blocking_calls(kind, gran, msg_bytes, wgs, wg_size, n_msgs):
    # (the heap hands out powers of two: room for two arrays rounded up, and the library's own)
    with runtime(4, heap_size=4 << (n_msgs * (msg_bytes + 64) + 256).bit_length()):
        run_rma(kind, gran, 4, msg_bytes, n_msgs, seed=msg_bytes + gran + kind, wgs=wgs, wg_size=wg_size,
                stride_pad=64)


@pytest.mark.parametrize("msg_bytes", [8, 16, 32, 63, 64, 65, 100, 256, 1024, 4096, 65536, 1 << 20])
def test_message_size_sweep_wg(msg_bytes):
    # the put/get benchmark sweep at reduced heap size: 8 slices, powers of two from 8 B up
    with runtime(8):
        run_rma(rs.PUT, rs.WG, 8, msg_bytes, 3, seed=msg_bytes)
        run_rma(rs.GET, rs.WG, 8, msg_bytes, 3, seed=msg_bytes + 1)


@pytest.mark.parametrize("src_mis,dst_mis", [(0, 1), (1, 0), (4, 0), (0, 4), (8, 12), (12, 8), (1, 1),
                                             (3, 5), (5, 2), (7, 7)])
@pytest.mark.parametrize("msg_bytes", [67, 1000, 4096])
def test_misaligned_buffers(src_mis, dst_mis, msg_bytes):
    with runtime(4):
        for gran in (rs.WG, rs.WAVE, rs.THREAD):
            run_rma(rs.PUT, gran, 4, msg_bytes, 5, seed=src_mis * 16 + dst_mis, src_mis=src_mis,
                    dst_mis=dst_mis, stride_pad=29)


@pytest.mark.parametrize("kind", [rs.PUT, rs.GET])
@pytest.mark.parametrize("msg_bytes,src_mis,dst_mis,wgs,wg_size", [
    ((2 << 20) + 13, 0, 0, 4, 256),      # dealt pass by pass, tail bytes
    ((2 << 20) + 13, 4, 4, 3, 128),      # mutually aligned, 4 bytes past a 16-byte boundary: head bytes too
    ((1 << 20) + 5, 1, 7, 4, 256),       # misaligned against each other: one range per workgroup
    (1000, 3, 3, 4, 256),                # too small to deal
    (0, 0, 0, 2, 64)])
def test_one_transfer_shared_by_the_workgroups_of_a_pe(kind, msg_bytes, src_mis, dst_mis, wgs, wg_size):
    # roc_shmemx_ctx_{put,get}mem_wg_shard (extension)
    with runtime(4):
        run_rma(kind, rs.WG_SHARED, 4, msg_bytes, 2, seed=msg_bytes + src_mis, src_mis=src_mis,
                dst_mis=dst_mis, wgs=wgs, wg_size=wg_size, stride_pad=48 if msg_bytes else 0)


def test_zero_length_is_a_no_op():
    with runtime(4):
        run_rma(rs.PUT, rs.WG, 4, 0, 4, seed=1)
        run_rma(rs.GET, rs.THREAD, 4, 0, 4, seed=2)


def test_put_to_self_and_far_pe():
    with runtime(8):
        run_rma(rs.PUT, rs.WG, 8, 3000, 2, seed=4, pe_shift=0)
        run_rma(rs.PUT, rs.WAVE, 8, 3000, 2, seed=5, pe_shift=5)


def test_put_from_private_device_memory():
    # "source" of a put may be any device buffer of the calling PE, not only the heap
    with runtime(4):
        n = 5000
        payload = np.random.default_rng(3).integers(0, 256, size=n, dtype=np.uint8)
        local = rs.device_array(payload)
        dst = rs.sym_array(n, np.uint8, fill=GUARD)
        rs.roc_shmem_rma(rs.PUT, rs.WG, dst, local, n, 1, n, n, 1, rs.Launch(1, 256))
        rs.synchronize()
        for p in range(4):
            assert np.array_equal(dst.read(p), payload)
        local.free()
        dst.free()


def test_reference_fill_pattern():
    # clients/functional_tests/extended_primitives.cpp:87-119: sender '0', receiver pre-set '1'
    with runtime(2):
        n = 1 << 16
        s = rs.sym_array(n, np.uint8, fill=ord("0"))
        r = rs.sym_array(n, np.uint8, fill=ord("1"))
        rs.roc_shmem_rma(rs.PUT, rs.WG, r, s, n, 1, n, n, 1, rs.Launch(1, 64))
        rs.synchronize()
        assert (r.read(1) == ord("0")).all() and (r.read(0) == ord("0")).all()
        s.free()
        r.free()
