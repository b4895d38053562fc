"""Host-initiated data path and a user kernel built against the public header.

The C++ program tests/cxx/host_api_check.cpp uses the reference's host function
names (library/include/roc_shmem.hpp:907-1147) and checks every result against
a closed form, like the reference's testers do; it is compiled beforehand by
__graft_entry__.build().
"""
import os
import subprocess

import pytest

import glob

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
BINARY = os.path.join(HERE, "cxx", "host_api_check")
SOS_BINARY = os.path.join(HERE, "cxx", "sos_cases")
DEVICE_BINARY = os.path.join(HERE, "cxx", "device_api_cases")


def newest_header():
    pats = [os.path.join(ROOT, "include", "*.h*"),
            os.path.join(ROOT, "roc_shmem_amd", "csrc", "rocshmem_device", "*.hpp")]
    return max(os.path.getmtime(f) for p in pats for f in glob.glob(p))


def test_check_program_is_not_older_than_the_headers_it_inlines():
    # The device interface is header-only: a program built before a header changed carries
    # device code for the old state layout.  (The library refuses to initialise for such a
    # program; this catches it before anything runs.)
    for binary in (BINARY, SOS_BINARY, DEVICE_BINARY):
        if not os.path.exists(binary):
            pytest.skip("%s is not built yet" % binary)
        assert os.path.getmtime(binary) >= newest_header(), \
            "%s is stale: run __graft_entry__.build()" % binary


@pytest.mark.gpu
def test_host_api_program():
    if not os.path.exists(BINARY):
        pytest.fail("tests/cxx/host_api_check is not built: run __graft_entry__.build()")
    assert os.path.getmtime(BINARY) >= newest_header(), "stale check program: run __graft_entry__.build()"
    print("running", BINARY, flush=True)
    out = subprocess.run([BINARY], capture_output=True, text=True, timeout=100)
    tail = (out.stdout + out.stderr)[-3000:]
    assert out.returncode == 0, tail
    assert "HOST_API_OK" in out.stdout, tail


@pytest.mark.gpu
@pytest.mark.parametrize("num_pes", [2, 6])
def test_reference_host_programs_restated(num_pes):
    # tests/cxx/sos_cases.cpp: the reference's clients/sos_tests programs, one function each.
    if not os.path.exists(SOS_BINARY):
        pytest.fail("tests/cxx/sos_cases is not built: run __graft_entry__.build()")
    assert os.path.getmtime(SOS_BINARY) >= newest_header(), "stale check program: run __graft_entry__.build()"
    print("running", SOS_BINARY, "with", num_pes, "PEs", flush=True)
    env = dict(os.environ, ROC_SHMEM_NUM_PES=str(num_pes))
    out = subprocess.run([SOS_BINARY], capture_output=True, text=True, timeout=110, env=env)
    tail = (out.stdout + out.stderr)[-3000:]
    assert out.returncode == 0, tail
    assert "SOS_CASES_OK" in out.stdout, tail


@pytest.mark.gpu
@pytest.mark.parametrize("num_pes", [4, 8])
def test_reference_functional_testers_restated(num_pes):
    # tests/cxx/device_api_cases.cpp: user kernels in the style of clients/functional_tests.
    # With 8 PEs the members of every exchange sit on eight different XCDs.
    if not os.path.exists(DEVICE_BINARY):
        pytest.fail("tests/cxx/device_api_cases is not built: run __graft_entry__.build()")
    assert os.path.getmtime(DEVICE_BINARY) >= newest_header(), "stale check program: run __graft_entry__.build()"
    print("running", DEVICE_BINARY, "with", num_pes, "PEs", flush=True)
    env = dict(os.environ, ROC_SHMEM_NUM_PES=str(num_pes))
    out = subprocess.run([DEVICE_BINARY], capture_output=True, text=True, timeout=110, env=env)
    tail = (out.stdout + out.stderr)[-3000:]
    print(out.stdout[-1500:], flush=True)
    assert out.returncode == 0, tail
    assert "DEVICE_API_OK" in out.stdout, tail


@pytest.mark.gpu
def test_entry_points_called_from_several_host_threads():
    """The C ABI serialises its entry points: threads that allocate, launch, read back and free at
    the same time each get their own correct result (ctypes drops the interpreter lock during
    the calls, so they do overlap)."""
    import threading

    import numpy as np

    import roc_shmem_amd as rs

    n_pes, n, rounds = 4, 2000, 25
    rs.roc_shmem_init(n_pes, 64 << 20, 8, 1024)
    in_use_at_start = rs.heap_bytes_in_use()
    errors = []

    def worker(tid):
        try:
            rng = np.random.default_rng(tid)
            for r in range(rounds):
                src = rs.sym_array(n, np.int64)
                dst = rs.sym_array(n, np.int64, fill=0)
                psync = rs.sym_array(rs.ROC_SHMEM_REDUCE_SYNC_SIZE, np.int64, fill=0)
                host = [rng.integers(-1000, 1000, n, dtype=np.int64) + tid for _ in range(n_pes)]
                for p in range(n_pes):
                    src.write(p, host[p])
                rs.roc_shmem_to_all(rs.LONG, rs.SUM, dst, src, n, 0, 0, n_pes, None, psync)
                rs.synchronize()
                want = np.sum(np.stack(host), axis=0, dtype=np.int64)
                for p in range(n_pes):
                    if not np.array_equal(dst.read(p), want):
                        errors.append("thread %d round %d PE %d" % (tid, r, p))
                for a in (psync, dst, src):
                    a.free()
        except Exception as e:  # noqa: BLE001 - reported by the main thread
            errors.append("thread %d: %r" % (tid, e))

    try:
        threads = [threading.Thread(target=worker, args=(t,)) for t in range(6)]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        assert not errors, errors[:5]
        assert rs.take_status() == 0
        assert rs.heap_bytes_in_use() == in_use_at_start
    finally:
        rs.roc_shmem_finalize()
