"""Compile librocshmem_mi355x.so for gfx950 (hipcc, in-tree)."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "librocshmem_mi355x.so")


def build(jobs=8, force=False, isa=False):
    """Run the in-tree Makefile; returns the path of the shared library.  isa: also write the
    kernels' assembly under csrc/build/isa, which the check of the generated code reads."""
    if force:
        subprocess.run(["make", "-s", "-C", CSRC, "clean"], check=True)
    subprocess.run(["make", "-s", "-C", CSRC, "-j%d" % jobs, "all"] + (["isa"] if isa else []), check=True)
    if not os.path.exists(LIB_PATH):
        raise RuntimeError("build did not produce %s" % LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build())
