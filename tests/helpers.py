"""Shared pieces of the GPU parity tests."""
import contextlib

import numpy as np

import oracle
import roc_shmem_amd as rs


@contextlib.contextmanager
def runtime(num_pes, heap_size=64 << 20, num_blocks=16, sq_size=1024):
    """Bring the library up for one test and check the device status word on the way out."""
    rs.roc_shmem_init(num_pes, heap_size, num_blocks, sq_size)
    try:
        yield
        status = rs.take_status()
        assert status == 0, "device status word raised: %d" % status
    finally:
        rs.roc_shmem_finalize()


def splitmix64(seed, n):
    """Counter-based generator: n uint64 values from `seed`."""
    x = (np.arange(1, n + 1, dtype=np.uint64) * np.uint64(0x9E3779B97F4A7C15)) + np.uint64(seed)
    x ^= x >> np.uint64(30)
    x *= np.uint64(0xBF58476D1CE4E5B9)
    x ^= x >> np.uint64(27)
    x *= np.uint64(0x94D049BB133111EB)
    x ^= x >> np.uint64(31)
    return x


def random_values(dtype, n, seed, kind="full"):
    """Seeded inputs for a reduction of element type `dtype` (an rs/oracle dtype code)."""
    rng = np.random.default_rng(seed)
    npd = rs.NP_DTYPE[dtype]
    if dtype in (rs.SHORT, rs.INT, rs.LONG, rs.LONGLONG):
        if kind == "c1":  # uniform in [-2^30, 2^30]
            return rng.integers(-(1 << 30), (1 << 30) + 1, size=n, dtype=np.int64).astype(npd)
        info = np.iinfo(npd)
        return rng.integers(info.min, info.max, size=n, dtype=npd, endpoint=True)
    if kind == "lognormal":
        x = rng.choice([-1.0, 1.0], size=n) * np.exp(2.0 * rng.standard_normal(n))
    else:
        x = rng.standard_normal(n)
    if dtype == rs.BF16:
        return oracle.float_to_bf16(x.astype(np.float32))
    return x.astype(npd)


def as_float64(dtype, arr):
    if dtype == rs.BF16:
        return oracle.bf16_to_float(arr).astype(np.float64)
    return np.asarray(arr).astype(np.float64)


# Tolerances of the floating-point reductions against the long-double ground
# truth: |got - ref| <= tol * max(|ref|, eps * sum|x_p|).  float and bfloat16
# are folded in a wider type and rounded once, so eps is half an ulp of the
# result type relative to the terms.  double has no wider type on the GPU: each
# of the P-1 additions may round, which bounds the error by (P-1) * 2^-53 *
# sum|x_p| however much the terms cancel; tol * eps covers P <= 9.
FP_TOL = {rs.FLOAT: (1e-6, 2.0 ** -24), rs.BF16: (1e-2, 2.0 ** -8), rs.DOUBLE: (1e-12, 2.0 ** -10)}


def check_fp(dtype, got, ref64, abs_sum64):
    tol, eps = FP_TOL[dtype]
    g = as_float64(dtype, got)
    bound = tol * np.maximum(np.abs(ref64), eps * abs_sum64)
    bad = np.abs(g - ref64) > bound
    assert not bad.any(), "%d of %d elements outside tolerance; first at %d: got %r ref %r" % (
        bad.sum(), bad.size, int(np.argmax(bad)), g[np.argmax(bad)], ref64[np.argmax(bad)])
