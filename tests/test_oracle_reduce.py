"""Pins the oracle's reductions: closed forms held by the reference's own tests, a
brute-force fold, and exactly representable floating-point cases."""
import math

import numpy as np
import pytest

import oracle

INT_TYPES = [oracle.SHORT, oracle.INT, oracle.LONG, oracle.LONGLONG]
ALL_TYPES = INT_TYPES + [oracle.FLOAT, oracle.DOUBLE]
N = 128  # clients/sos_tests/to_all.cpp uses N = 128


def heap_with(npes, dtype, gen, n=N):
    npd = oracle.NP_DTYPE[dtype]
    es = np.dtype(npd).itemsize
    h = oracle.Heap(npes, 2 * n * es)
    for me in range(npes):
        h.view(me, 0, n, npd)[:] = gen(me).astype(npd)
    return h, npd, n * es


def results(h, dtype, op, n=N, **kw):
    npd = oracle.NP_DTYPE[dtype]
    es = np.dtype(npd).itemsize
    oracle.to_all(h, dtype, op, n * es, 0, n, **kw)
    return [h.view(p, n * es, n, npd).copy() for p in range(h.n_pes)]


@pytest.mark.parametrize("npes", [1, 2, 4, 7])
@pytest.mark.parametrize("dtype", ALL_TYPES)
def test_to_all_cpp_closed_forms(npes, dtype):
    i = np.arange(N)
    # max: src = me + i -> npes - 1 + i        (to_all.cpp:123-153)
    h, npd, _ = heap_with(npes, dtype, lambda me: me + i)
    for r in results(h, dtype, oracle.MAX):
        assert np.array_equal(r, (npes - 1 + i).astype(npd))
    # min: src = me + i -> i                    (to_all.cpp:213-251)
    for r in results(h, dtype, oracle.MIN):
        assert np.array_equal(r, i.astype(npd))
    # sum: src = me -> npes(npes-1)/2           (to_all.cpp:310-346)
    h, npd, _ = heap_with(npes, dtype, lambda me: np.full(N, me))
    for r in results(h, dtype, oracle.SUM):
        assert (r == npes * (npes - 1) // 2).all()
    # prod: src = me + 1 -> npes!               (to_all.cpp:471-503)
    h, npd, _ = heap_with(npes, dtype, lambda me: np.full(N, me + 1))
    for r in results(h, dtype, oracle.PROD):
        assert (r == math.factorial(npes)).all()


@pytest.mark.parametrize("npes", [1, 2, 4, 7])
@pytest.mark.parametrize("dtype", INT_TYPES)
def test_to_all_cpp_bitwise_closed_forms(npes, dtype):
    # and: src = me -> 0 for npes > 1 (to_all.cpp:407-428); or: (me+1)%4 -> 3, 1 if npes == 1
    # (:632,652); xor: me%2 -> (npes/2)%2 (:696-701)
    h, _, _ = heap_with(npes, dtype, lambda me: np.full(N, me))
    for r in results(h, dtype, oracle.AND):
        assert (r == 0).all()
    h, _, _ = heap_with(npes, dtype, lambda me: np.full(N, (me + 1) % 4))
    expect = 1 if npes == 1 else (3 if npes >= 2 else 0)
    if npes == 2:
        expect = 1 | 2
    for r in results(h, dtype, oracle.OR):
        assert (r == expect).all()
    h, _, _ = heap_with(npes, dtype, lambda me: np.full(N, me % 2))
    for r in results(h, dtype, oracle.XOR):
        assert (r == (npes // 2) % 2).all()


def test_float_sum_of_ones_and_team_reduce_forms():
    # clients/functional_tests/tester.cpp:149-164: float sum of 1.0 over n PEs == n
    # clients/sos_tests/shmem_team_reduce.cpp:88-101: src = 1: and/or/max/min/prod -> 1, sum -> npes, xor -> npes % 2
    for npes in (2, 3, 8):
        h, _, _ = heap_with(npes, oracle.FLOAT, lambda me: np.ones(512), n=512)
        for r in results(h, oracle.FLOAT, oracle.SUM, n=512):
            assert (r == float(npes)).all()
        h, _, _ = heap_with(npes, oracle.INT, lambda me: np.ones(N))
        for op, want in ((oracle.AND, 1), (oracle.OR, 1), (oracle.MAX, 1), (oracle.MIN, 1),
                         (oracle.PROD, 1), (oracle.SUM, npes), (oracle.XOR, npes % 2)):
            for r in results(h, oracle.INT, op):
                assert (r == want).all()


def test_big_reduction_and_in_place_and_active_set():
    # big_reduction.cpp:76-107 (long max, N = 128), reduce_in_place.cpp:58-69 (dest == source),
    # reduce_active_set.cpp:78-113 (PE_start = i, size = npes - i)
    npes = 6
    i = np.arange(N)
    h, npd, off = heap_with(npes, oracle.LONG, lambda me: me + i)
    oracle.to_all(h, oracle.LONG, oracle.MAX, 0, 0, N)          # in place
    for p in range(npes):
        assert np.array_equal(h.view(p, 0, N, npd), npes - 1 + i)
    for start in range(npes):
        h, npd, off = heap_with(npes, oracle.LONGLONG, lambda me: np.full(N, me))
        for p in range(npes):
            h.view(p, off, N, npd)[:] = -1
        oracle.to_all(h, oracle.LONGLONG, oracle.SUM, off, 0, N, pe_start=start, log_stride=0,
                      pe_size=npes - start)
        want = sum(range(start, npes))
        for p in range(npes):
            got = h.view(p, off, N, npd)
            assert (got == (want if p >= start else -1)).all()
    # strided set {1, 3, 5}
    h, npd, off = heap_with(npes, oracle.INT, lambda me: np.full(N, 1 << me))
    for p in range(npes):
        h.view(p, off, N, npd)[:] = 0
    oracle.to_all(h, oracle.INT, oracle.OR, off, 0, N, pe_start=1, log_stride=1, pe_size=3)
    for p in range(npes):
        assert (h.view(p, off, N, npd) == (0b101010 if p in (1, 3, 5) else 0)).all()


@pytest.mark.parametrize("dtype", INT_TYPES)
@pytest.mark.parametrize("op", range(7))
def test_integer_fold_matches_python_big_integers(dtype, op):
    npes, n = 5, 300
    npd = oracle.NP_DTYPE[dtype]
    bits = np.dtype(npd).itemsize * 8
    rng = np.random.default_rng(dtype * 10 + op)
    info = np.iinfo(npd)
    vals = [rng.integers(info.min, info.max, n, dtype=npd, endpoint=True) for _ in range(npes)]
    h, _, off = heap_with(npes, dtype, lambda me: vals[me], n=n)
    got = results(h, dtype, op, n=n)[3]
    fold = {0: lambda a, b: a + b, 1: max, 2: min, 3: lambda a, b: a * b, 4: lambda a, b: a & b,
            5: lambda a, b: a | b, 6: lambda a, b: a ^ b}[op]
    for k in range(n):
        acc = int(vals[0][k])
        for p in range(1, npes):
            acc = fold(acc, int(vals[p][k]))
            acc &= (1 << bits) - 1
            if acc >> (bits - 1):
                acc -= 1 << bits
        assert int(got[k]) == acc


def test_threaded_path_equals_the_single_threaded_one():
    rng = np.random.default_rng(1)
    h1, npd, off = heap_with(4, oracle.FLOAT, lambda me: rng.standard_normal(10001), n=10001)
    h2 = oracle.Heap(4, h1.stride)
    h2.buf[:] = h1.buf
    oracle.to_all(h1, oracle.FLOAT, oracle.SUM, off, 0, 10001)
    oracle.to_all(h2, oracle.FLOAT, oracle.SUM, off, 0, 10001, threads=5)
    assert np.array_equal(h1.buf, h2.buf)


def test_floating_point_ground_truth_and_in_type_fold():
    # exactly representable inputs: in-type fold, ground truth and numpy agree bit for bit
    npes, n = 8, 1000
    rng = np.random.default_rng(2)
    vals = [rng.integers(-1000, 1000, n).astype(np.float32) / 8 for _ in range(npes)]
    h, npd, off = heap_with(npes, oracle.FLOAT, lambda me: vals[me], n=n)
    truth = oracle.to_all_f64(h, oracle.FLOAT, oracle.SUM, 0, n)
    assert np.array_equal(truth, np.sum(np.stack(vals).astype(np.float64), axis=0))
    assert np.array_equal(results(h, oracle.FLOAT, oracle.SUM, n=n)[0].astype(np.float64), truth)
    assert np.array_equal(oracle.abs_sum_f64(h, oracle.FLOAT, 0, n),
                          np.sum(np.abs(np.stack(vals)).astype(np.float64), axis=0))
    # generic inputs: the long-double sum agrees with math.fsum (exact) to double rounding
    vals = [rng.standard_normal(200).astype(np.float32) for _ in range(npes)]
    h, _, _ = heap_with(npes, oracle.FLOAT, lambda me: vals[me], n=200)
    truth = oracle.to_all_f64(h, oracle.FLOAT, oracle.SUM, 0, 200)
    exact = np.array([math.fsum(float(v[k]) for v in vals) for k in range(200)])
    assert np.allclose(truth, exact, rtol=1e-15, atol=0)
    # max / min ignore NaN operands, as fmaxf / fminf do
    a = np.array([1.0, np.nan, -0.5, np.nan], np.float32)
    b = np.array([np.nan, 2.0, -0.25, np.nan], np.float32)
    h, _, off = heap_with(2, oracle.FLOAT, lambda me: (a, b)[me], n=4)
    mx = results(h, oracle.FLOAT, oracle.MAX, n=4)[0]
    mn = results(h, oracle.FLOAT, oracle.MIN, n=4)[1]
    assert mx[0] == 1.0 and mx[1] == 2.0 and mx[2] == -0.25 and np.isnan(mx[3])
    assert mn[0] == 1.0 and mn[1] == 2.0 and mn[2] == -0.5 and np.isnan(mn[3])


def test_bfloat16_rounding_known_answers():
    # round to nearest, ties to even, on the 16 dropped bits
    cases = {0x3F800000: 0x3F80,            # 1.0
             0x3F808000: 0x3F80,            # tie -> even (down)
             0x3F818000: 0x3F82,            # tie -> even (up)
             0x3F808001: 0x3F81,            # just above the tie
             0x3F807FFF: 0x3F80,            # just below the tie
             0x7F7FFFFF: 0x7F80,            # largest finite rounds to infinity
             0xFF800000: 0xFF80,            # -inf
             0x7FC00001: 0x7FC0,            # NaN stays NaN
             0x00000000: 0x0000, 0x80000000: 0x8000}
    bits = np.array(list(cases), dtype=np.uint32)
    got = oracle.float_to_bf16(bits.view(np.float32))
    assert [int(x) for x in got] == list(cases.values())
    back = oracle.bf16_to_float(np.array([0x3F80, 0xC000, 0x7F80], np.uint16))
    assert list(back) == [1.0, -2.0, np.inf]
    # bf16 sum ground truth: sums the rounded inputs exactly
    h = oracle.Heap(3, 64)
    for p, v in enumerate((1.0, 0.0078125, -1.0)):
        h.view(p, 0, 1, np.uint16)[:] = oracle.float_to_bf16(np.array([v], np.float32))
    assert oracle.to_all_f64(h, oracle.BF16, oracle.SUM, 0, 1)[0] == 0.0078125


def test_undefined_type_operator_pairs_are_refused():
    h = oracle.Heap(2, 256)
    for dtype, op in ((oracle.FLOAT, oracle.AND), (oracle.DOUBLE, oracle.XOR), (oracle.BF16, oracle.PROD)):
        with pytest.raises(ValueError):
            oracle.to_all(h, dtype, op, 64, 0, 4)


def test_rounded_once_fold_is_the_correctly_rounded_true_sum_where_the_wide_fold_is_exact():
    # float: eight N(0,1) terms lie within 2^26 of each other, so their double sum is exact and the
    # result must be the true sum rounded to float once; an in-type float fold (rounding after
    # every step) differs from it in a visible fraction of the elements, so a fold in the wrong
    # type would fail here.  math.fsum gives the exact sum independently of the oracle.
    npes, n = 8, 4000
    rng = np.random.default_rng(7)
    vals = [rng.standard_normal(n).astype(np.float32) for _ in range(npes)]
    h, _, off = heap_with(npes, oracle.FLOAT, lambda me: vals[me], n=n)
    oracle.to_all_rounded_once(h, oracle.FLOAT, oracle.SUM, off, 0, n)
    exact = np.array([math.fsum(float(v[k]) for v in vals) for k in range(n)])
    want = exact.astype(np.float32)
    for p in range(npes):
        assert np.array_equal(h.view(p, off, n, np.float32), want)
    assert np.array_equal(oracle.to_all_f64(h, oracle.FLOAT, oracle.SUM, 0, n).astype(np.float32), want)
    in_type = results(h, oracle.FLOAT, oracle.SUM, n=n)[0]
    assert (in_type != want).mean() > 0.05
    # prod of small exactly representable factors: exact in double, so equal to the exact product
    ints = [rng.integers(1, 8, n).astype(np.float32) / 2 for _ in range(npes)]
    h, _, off = heap_with(npes, oracle.FLOAT, lambda me: ints[me], n=n)
    oracle.to_all_rounded_once(h, oracle.FLOAT, oracle.PROD, off, 0, n)
    assert np.array_equal(h.view(3, off, n, np.float32),
                          np.prod(np.stack(ints).astype(np.float64), axis=0).astype(np.float32))
    # bfloat16: eight terms within 2^13 of each other sum exactly in float
    bvals = [oracle.float_to_bf16(rng.uniform(0.5, 4.0, n).astype(np.float32) * rng.choice([-1, 1], n).astype(np.float32))
             for _ in range(npes)]
    h, _, off = heap_with(npes, oracle.BF16, lambda me: bvals[me], n=n)
    oracle.to_all_rounded_once(h, oracle.BF16, oracle.SUM, off, 0, n)
    exact = np.array([math.fsum(float(oracle.bf16_to_float(v[k:k + 1])[0]) for v in bvals) for k in range(n)])
    want = oracle.float_to_bf16(exact.astype(np.float32))
    for p in range(npes):
        assert np.array_equal(h.view(p, off, n, np.uint16), want)
    in_type = results(h, oracle.BF16, oracle.SUM, n=n)[0]
    assert (in_type != want).mean() > 0.05
    # everything else is the in-type fold
    for dtype, op in ((oracle.FLOAT, oracle.MAX), (oracle.BF16, oracle.MIN), (oracle.DOUBLE, oracle.SUM),
                      (oracle.INT, oracle.PROD)):
        gen = (lambda me: bvals[me]) if dtype == oracle.BF16 else (lambda me: vals[me] * 1000)
        h1, _, off = heap_with(npes, dtype, gen, n=n)
        h2, _, _ = heap_with(npes, dtype, gen, n=n)
        oracle.to_all(h1, dtype, op, off, 0, n)
        oracle.to_all_rounded_once(h2, dtype, op, off, 0, n)
        assert np.array_equal(h1.buf, h2.buf)
    # active sets and teams address the same members as to_all
    h1, _, off = heap_with(npes, oracle.FLOAT, lambda me: vals[me], n=n)
    oracle.to_all_rounded_once(h1, oracle.FLOAT, oracle.SUM, off, 0, n, pe_start=1, log_stride=1, pe_size=3)
    want = (vals[1].astype(np.float64) + vals[3] + vals[5]).astype(np.float32)
    assert np.array_equal(h1.view(5, off, n, np.float32), want) and not h1.view(0, off, n, np.float32).any()
    h1, _, off = heap_with(npes, oracle.FLOAT, lambda me: vals[me], n=n)
    oracle.to_all_rounded_once(h1, oracle.FLOAT, oracle.SUM, off, 0, n, pe_start=0, pe_stride=3, pe_size=3)
    want = (vals[0].astype(np.float64) + vals[3] + vals[6]).astype(np.float32)
    assert np.array_equal(h1.view(6, off, n, np.float32), want)
