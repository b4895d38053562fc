"""Wave-level building blocks against the reference's unit-test expectations and the lane models."""
import numpy as np
import pytest

import oracle
import roc_shmem_amd as rs

pytestmark = pytest.mark.gpu

ALL = 0xFFFFFFFFFFFFFFFF


@pytest.mark.parametrize("mask,n_wgs,wg_size,total", [
    (0xA, 1, 64, 2),                       # clients/unit_tests/bitwise_gtest.cpp:1384-1408
    (ALL, 1, 64, 64),                      # :1410-1434
    (0xFFFFFFFF00000000, 1, 64, 32),       # :1436-1460
    (0xF0F0F0F0F0F0F0F0, 1, 64, 32),       # :1462-1486
    (ALL, 1024, 1024, 1048576),            # :1488-1500 (1024 x 1024 threads)
    (0x8000000000000001, 7, 256, 7 * 4 * 2),
])
def test_fetch_incr_known_answers(mask, n_wgs, wg_size, total):
    per_thread, counter = rs.kat_fetch_incr(mask, n_wgs, wg_size)
    assert counter == total
    lanes = np.arange(n_wgs * wg_size) % 64
    active = ((mask >> lanes.astype(np.uint64)) & 1).astype(bool) if False else \
        np.array([(mask >> int(l)) & 1 for l in range(64)], dtype=bool)[lanes]
    got = per_thread[active]
    # every active lane holds a distinct value and together they cover [0, total)
    assert np.array_equal(np.sort(got), np.arange(total, dtype=np.uint64))
    assert (per_thread[~active] == ALL).all()
    # inside each wave the values ascend with the lane index, one apart
    waves = per_thread.reshape(-1, 64)
    n_active = bin(mask).count("1")
    for w in waves[:64]:
        vals = w[[l for l in range(64) if (mask >> l) & 1]]
        assert np.array_equal(vals, vals[0] + np.arange(n_active, dtype=np.uint64))
        # logical lane 1 receives base + 1 (bitwise_gtest.cpp:1502-1526)
        assert vals[0] % n_active == 0


def test_fetch_incr_matches_lane_model():
    rng = np.random.default_rng(5)
    for _ in range(20):
        mask = int(rng.integers(1, 1 << 63, dtype=np.uint64)) | int(rng.integers(0, 2)) << 63
        got, counter = rs.kat_fetch_incr(mask, 1, 64)
        exp, exp_counter = oracle.fetch_incr(mask, 0)
        assert counter == exp_counter
        assert np.array_equal(got, exp)


def lanes_case(rng, size, runs):
    """Build 64 lanes out of (length, pe) runs of contiguous messages."""
    pe = np.zeros(64, np.int32)
    src = np.zeros(64, np.uint64)
    dst = np.zeros(64, np.uint64)
    sz = np.full(64, size, np.uint64)
    lane = 0
    base_s, base_d = 0x10000, 0x900000
    for length, p in runs:
        base_s += 4096
        base_d += 8192
        for k in range(length):
            if lane == 64:
                break
            pe[lane] = p
            src[lane] = base_s + k * size
            dst[lane] = base_d + k * size
            lane += 1
    return pe, src, dst, sz


def test_coalesce_reference_example():
    # library/src/wf_coal_policy.cpp:39-53: lanes 0-8 contiguous, lane 9 alone, lanes 10-63
    # contiguous -> three messages
    pe, src, dst, sz = lanes_case(None, 8, [(9, 1), (1, 1), (54, 1)])
    must, out = rs.kat_coalesce(ALL, pe, src, dst, sz)
    assert list(np.nonzero(must)[0]) == [0, 9, 10]
    assert out[0] == 9 * 8 and out[9] == 8 and out[10] == 54 * 8


def test_coalesce_matches_lane_model():
    rng = np.random.default_rng(17)
    for trial in range(60):
        runs = []
        left = 64
        while left > 0:
            length = int(rng.integers(1, 12))
            runs.append((length, int(rng.integers(0, 3))))
            left -= length
        size = int(rng.choice([1, 4, 8, 16, 64]))
        pe, src, dst, sz = lanes_case(rng, size, runs)
        if trial % 3 == 1:  # break size equality here and there
            sz[rng.integers(0, 64, 5)] = size * 2
        if trial % 3 == 2:  # make destinations discontiguous here and there
            dst[rng.integers(0, 64, 5)] += 8
        mask = ALL if trial % 2 == 0 else int(rng.integers(1, 1 << 63, dtype=np.uint64))
        must, out = rs.kat_coalesce(mask, pe, src, dst, sz)
        emust, eout = oracle.coalesce(mask, pe, src, dst, sz)
        active = np.array([(mask >> l) & 1 for l in range(64)], dtype=bool)
        assert np.array_equal(must[active], emust[active]), "trial %d" % trial
        assert np.array_equal(out[active], eout[active]), "trial %d" % trial
        # merged sizes of the senders account for every active lane's bytes
        assert out[active & (must == 1)].sum() == sz[active].sum()
