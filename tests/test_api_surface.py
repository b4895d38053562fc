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
