#!/bin/bash
# Builds oracle/_ref/libref_alloc.so: the reference's own symmetric-heap allocator
# (header-only host code under /root/reference/library/src/memory), compiled where
# it lies with hipcc (its __device__ stubs need the HIP attribute), behind the C
# entry points of oracle/ref_alloc_wrapper.cpp.  The rest of the reference's path
# needs <infiniband/mlx5dv.h>, MPI, generated config.h or a GPU and is not built.
set -euo pipefail
HERE="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
REF="${ROC_SHMEM_REFERENCE:-/root/reference}"
mkdir -p "$HERE/_ref"
/opt/rocm/bin/hipcc -x hip --offload-arch=gfx950 -O2 -std=c++17 -fPIC -shared \
    -Wno-unused-command-line-argument -I "$REF/library" \
    "$HERE/ref_alloc_wrapper.cpp" -o "$HERE/_ref/libref_alloc.so"
echo "built $HERE/_ref/libref_alloc.so"
