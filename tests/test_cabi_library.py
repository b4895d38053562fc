"""The C-ABI library loads, exports every declared symbol, and fails loudly without a GPU."""
import os
import re

import pytest

from conftest import gpu_present

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "rocshmem_mi355x.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rsm_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound():
    from roc_shmem_amd import _lib
    lib = _lib.load()
    names = declared_symbols()
    assert len(names) >= 50
    for name in names:
        assert hasattr(lib, name), "library does not export %s" % name
        assert name in _lib.SIGNATURES, "no ctypes signature for %s" % name
    for name in _lib.SIGNATURES:
        assert name in names, "%s is bound but not declared in the header" % name


def test_each_kernel_unit_keeps_its_own_device_state():
    # One upload hook per translation unit that contains device code; a single shared hook
    # would leave the other units' kernels with a zeroed state.
    import glob
    from roc_shmem_amd import _lib
    csrc = os.path.join(ROOT, "roc_shmem_amd", "csrc")
    drivers = glob.glob(os.path.join(csrc, "cabi", "drv_*.hip"))
    # every driver unit, plus cabi.cpp and host/api_host.cpp, which include the device header too
    assert len(drivers) >= 5
    assert _lib.load().rsm_state_units() == len(drivers) + 2


@pytest.mark.skipif(gpu_present(), reason="checks the no-GPU error path")
def test_init_without_gpu_raises_instead_of_falling_back():
    import roc_shmem_amd as rs
    with pytest.raises(rs.RocShmemError):
        rs.roc_shmem_init(4, 1 << 20)
    assert rs.roc_shmem_n_pes() == -1
    with pytest.raises(rs.RocShmemError):
        rs.roc_shmem_to_all(rs.LONG, rs.SUM, 1, 2, 3, 0, 0, 4, None, 5)


def test_public_header_compiles_a_user_kernel(tmp_path):
    # A kernel written the way the reference's testers are (clients/functional_tests/
    # reduction_tester.cpp:74-104, primitive_tester.cpp:32-82) compiles against include/roc_shmem.hpp.
    src = tmp_path / "user_kernel.hip"
    src.write_text(r'''
#include "roc_shmem.hpp"
using namespace rocshmem;
__global__ void user(long *dest, long *src, long *pWrk, long *pSync, int n, roc_shmem_team_t team) {
  __shared__ roc_shmem_ctx_t ctx;
  roc_shmem_wg_init();
  roc_shmem_wg_ctx_create(ROC_SHMEM_CTX_WG_PRIVATE, &ctx);
  int n_pes = roc_shmem_ctx_n_pes(ctx);
  roc_shmem_ctx_long_sum_wg_to_all(ctx, dest, src, n, 0, 0, n_pes, pWrk, pSync);
  roc_shmem_ctx_long_max_wg_to_all(ctx, team, dest, src, n);
  roc_shmem_ctx_wg_barrier_all(ctx);
  roc_shmemx_ctx_putmem_wg(ctx, dest, src, n * sizeof(long), 1);
  roc_shmemx_ctx_getmem_nbi_wave(ctx, dest, src, n * sizeof(long), 1);
  roc_shmem_ctx_long_wg_broadcast(ctx, dest, src, n, 0, 0, 0, n_pes, pSync);
  roc_shmem_ctx_long_wg_alltoall(ctx, team, dest, src, n);
  roc_shmem_ctx_long_wg_fcollect(ctx, team, dest, src, n);
  if (threadIdx.x == 0) {
    roc_shmem_ctx_long_p(ctx, dest, 5L, 1);
    long v = roc_shmem_ctx_long_atomic_fetch_add(ctx, dest, 2L, 1);
    roc_shmem_ctx_int64_atomic_add(ctx, (int64_t *)dest, v, 0);
    roc_shmem_long_wait_until(dest, ROC_SHMEM_CMP_GE, 1L);
    roc_shmem_putmem(dest, src, 8, roc_shmem_my_pe());
  }
  roc_shmem_ctx_quiet(ctx);
  roc_shmem_wg_ctx_destroy(ctx);
  roc_shmem_wg_finalize();
}
int main() { roc_shmem_init(); void *p = roc_shmem_malloc(64); roc_shmem_free(p); roc_shmem_finalize(); }
''')
    import subprocess
    cmd = ["/opt/rocm/bin/hipcc", "-x", "hip", "--offload-arch=gfx950", "-std=c++17", "-DROCSHMEM_NO_MPI",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-I", os.path.join(ROOT, "include"), "-I", os.path.join(ROOT, "roc_shmem_amd", "csrc"),
           "-c", str(src), "-o", str(tmp_path / "user_kernel.o")]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]


def test_active_set_range_check_is_done_in_64_bits():
    # The check rsm_to_all / rsm_broadcast apply before they launch.  A 32-bit
    # (pe_size - 1) << log_pe_stride wraps for large strides (4 << 30 == 0, 2 << 30 == INT_MIN)
    # and would accept sets whose members lie far outside the arena.  No launch here.
    from roc_shmem_amd import _lib
    ok = _lib.load().rsm_host_active_set_in_range
    assert ok(0, 0, 8, 8) == 1
    assert ok(0, 0, 9, 8) == 0
    assert ok(1, 1, 4, 8) == 1          # 1, 3, 5, 7
    assert ok(1, 1, 5, 8) == 0          # ... 9
    assert ok(0, 2, 2, 8) == 1          # 0, 4
    assert ok(0, 3, 2, 8) == 0          # 0, 8
    assert ok(0, 6, 2, 128) == 1 and ok(0, 7, 2, 128) == 0
    assert ok(5, 0, 1, 8) == 1 and ok(8, 0, 1, 8) == 0 and ok(-1, 0, 1, 8) == 0
    for pe_size in (2, 3, 5, 128):
        for log in (29, 30, 31, 32, 40):
            assert ok(0, log, pe_size, 128) == 0, (pe_size, log)
    assert ok(0, 30, 1, 8) == 1 and ok(0, 31, 1, 8) == 0   # one member: any representable stride
    assert ok(0, -1, 2, 8) == 0 and ok(0, 0, 0, 8) == 0 and ok(0, 0, 129, 128) == 0
    # brute force against exact integers
    for num_pes in (1, 2, 7, 8, 128):
        for start in range(0, num_pes + 1):
            for log in range(0, 9):
                for size in (1, 2, 3, 4, 8, 16, 127, 128):
                    want = int(start < num_pes and start + (size - 1) * (1 << log) < num_pes)
                    assert ok(start, log, size, num_pes) == want, (start, log, size, num_pes)


def test_only_the_runtime_waits_for_the_whole_device():
    # A wait for the whole device while the live send-queue consumer runs lasts until the
    # consumer gives up by itself and leaves the queues without one.  Every such wait therefore
    # goes through Runtime::wait_for_device, which refuses while a persistent kernel is
    # registered: no other host source may call hipDeviceSynchronize itself.
    import glob
    import re
    csrc = os.path.join(ROOT, "roc_shmem_amd", "csrc")
    offenders = []
    for path in sorted(glob.glob(os.path.join(csrc, "**", "*.*"), recursive=True)):
        if os.sep + "build" + os.sep in path or not path.endswith((".cpp", ".hip", ".hpp")):
            continue
        text = open(path).read()
        for m in re.finditer(r"hipDeviceSynchronize\s*\(", text):
            line = text.count("\n", 0, m.start()) + 1
            if not path.endswith(os.path.join("host", "runtime.cpp")):
                offenders.append("%s:%d" % (os.path.relpath(path, ROOT), line))
    assert not offenders, offenders
    runtime = open(os.path.join(csrc, "host", "runtime.cpp")).read()
    # in the runtime: once at the end of init (nothing persistent can run yet) and in wait_for_device
    assert len(re.findall(r"hipDeviceSynchronize\s*\(", runtime)) == 2
    body = runtime[runtime.index("bool Runtime::wait_for_device()"):]
    assert "if (persistent_stop_) return false;" in body[:body.index("}")]
