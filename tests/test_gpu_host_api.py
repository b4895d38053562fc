"""Host-initiated data path and a user kernel built against the public header.

The C++ program tests/cxx/host_api_check.cpp uses the reference's host function
names (library/include/roc_shmem.hpp:907-1147) and checks every result against
a closed form, like the reference's testers do; it is compiled beforehand by
__graft_entry__.build().
"""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BINARY = os.path.join(HERE, "cxx", "host_api_check")


@pytest.mark.gpu
def test_host_api_program():
    if not os.path.exists(BINARY):
        pytest.fail("tests/cxx/host_api_check is not built: run __graft_entry__.build()")
    print("running", BINARY, flush=True)
    out = subprocess.run([BINARY], capture_output=True, text=True, timeout=100)
    tail = (out.stdout + out.stderr)[-3000:]
    assert out.returncode == 0, tail
    assert "HOST_API_OK" in out.stdout, tail
