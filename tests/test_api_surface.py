"""Every function the reference's public header declares exists here under the same name and on
the same side (host / device).  tests/golden/reference_api_names.json lists the reference's names
(written by tests/golden/make_api_names.py from library/include/roc_shmem.hpp); this repository's
headers are scanned the same way."""
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "tests", "golden"))
from api_names import names_of  # noqa: E402

HEADERS = [os.path.join(ROOT, "include", "roc_shmem.hpp"),
           os.path.join(ROOT, "include", "roc_shmem_host.hpp"),
           os.path.join(ROOT, "roc_shmem_amd", "csrc", "rocshmem_device", "api.hpp")]


def test_no_reference_function_is_missing_on_its_side():
    with open(os.path.join(ROOT, "tests", "golden", "reference_api_names.json")) as f:
        ref = json.load(f)
    assert len(ref["host"]) > 500 and len(ref["device"]) > 700      # the scan found the header
    host, device = names_of(HEADERS)
    assert sorted(set(ref["host"]) - set(host)) == []
    assert sorted(set(ref["device"]) - set(device)) == []


def test_the_scan_sees_macro_generated_names():
    host, device = names_of(HEADERS)
    for name in ("roc_shmem_ctx_float_sum_wg_to_all", "roc_shmemx_ctx_putmem_wg", "roc_shmem_ushort_wait_until",
                 "roc_shmem_ctx_bf16_sum_wg_to_all", "roc_shmem_ctx_int64_atomic_fetch_add"):
        assert name in device, name
    for name in ("roc_shmem_malloc", "roc_shmem_long_wait_until", "roc_shmem_uint64_atomic_fetch_xor",
                 "roc_shmem_ctx_double_prod_to_all"):
        assert name in host, name


def test_every_reference_declaration_resolves_with_its_exact_signature(tmp_path):
    """tests/golden/reference_api_signatures.json holds side, return type, name and parameter types
    of the reference header's 1454 declarations (tests/golden/make_api_signatures.py).  A program
    that initialises a function pointer of exactly that type from each name must compile against
    this repository's header, in a __device__ function for the device side and in a host function
    for the host side: a missing overload or a parameter of another type is a compile error."""
    import shutil
    import subprocess

    import pytest

    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not found")
    with open(os.path.join(ROOT, "tests", "golden", "reference_api_signatures.json")) as f:
        decls = json.load(f)["declarations"]
    assert len(decls) > 1400
    lines = ['#include "roc_shmem.hpp"', "using namespace rocshmem;"]
    for side, opener in (("device", "__device__ void device_side() {"), ("host", "void host_side() {")):
        lines.append(opener)
        for s, ret, name, params in decls:
            if s == side:
                lines.append("  { %s (*f)(%s) = %s; (void)f; }" % (ret, ", ".join(params), name))
        lines.append("}")
    src = tmp_path / "signatures.cpp"
    src.write_text("\n".join(lines) + "\n")
    cmd = [hipcc, "-x", "hip", "--offload-arch=gfx950", "-std=c++17", "-DROCSHMEM_NO_MPI", "-fsyntax-only",
           "-Wno-unused-command-line-argument", "-I", os.path.join(ROOT, "include"),
           "-I", os.path.join(ROOT, "roc_shmem_amd", "csrc"), str(src)]
    run = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    errors = [ln for ln in run.stderr.splitlines() if "error" in ln]
    assert run.returncode == 0 and not errors, "\n".join(errors[:20])
