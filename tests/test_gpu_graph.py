"""A run of data-path calls recorded into a HIP graph and replayed: every replay is compared
with the CPU oracle on the inputs of that replay, with eager copies and synchronisation between
the replays."""
import numpy as np
import pytest

import oracle
import roc_shmem_amd as rs
from helpers import runtime

pytestmark = pytest.mark.gpu


def test_recorded_collectives_and_puts_replay_like_eager_calls():
    n_pes, n = 4, 5000
    with runtime(n_pes):
        stream = rs.Stream()
        src = rs.sym_array(n, np.int64)
        red = rs.sym_array(n, np.int64)
        bc = rs.sym_array(n, np.int64)
        ring = rs.sym_array(n, np.int64)
        psync_r = rs.sym_array(2 * rs.ROC_SHMEM_REDUCE_SYNC_SIZE, np.int64, fill=0)
        psync_b = rs.sym_array(2 * rs.ROC_SHMEM_BCAST_SYNC_SIZE, np.int64, fill=0)
        launch = rs.Launch(2, 256, 0, stream)

        def record():
            # sum over all PEs -> red; PE 1's red -> everybody else's bc; every PE's bc -> right neighbour's ring
            rs.roc_shmem_to_all(rs.LONG, rs.SUM, red, src, n, 0, 0, n_pes, None, psync_r, launch)
            rs.roc_shmem_broadcast(8, bc, red, n, 1, 0, 0, n_pes, psync_b, launch)
            rs.roc_shmem_rma(rs.PUT, rs.WG, ring, bc, n * 8, 1, None, None, 1, launch)

        with rs.Graph.capture(stream) as graph:
            record()

        rng = np.random.default_rng(11)
        for replay in range(4):
            # eager work of the program between the replays: new inputs, cleared outputs
            host = [rng.integers(-(1 << 40), 1 << 40, size=n, dtype=np.int64) for _ in range(n_pes)]
            for p in range(n_pes):
                src.write(p, host[p])
                bc.write(p, np.full(n, -3 - replay, np.int64))
                ring.write(p, np.full(n, -5, np.int64))
            rs.synchronize()
            if replay == 3:
                record()            # the same calls made eagerly on the stream
            else:
                graph.launch()
            rs.synchronize()
            total = np.sum(np.stack(host), axis=0, dtype=np.int64)
            for p in range(n_pes):
                assert np.array_equal(red.read(p), total), "replay %d: sum on PE %d" % (replay, p)
                want_bc = np.full(n, -3 - replay, np.int64) if p == 1 else total
                assert np.array_equal(bc.read(p), want_bc), "replay %d: broadcast on PE %d" % (replay, p)
                left = (p - 1) % n_pes
                want_ring = np.full(n, -3 - replay, np.int64) if left == 1 else total
                assert np.array_equal(ring.read(p), want_ring), "replay %d: ring on PE %d" % (replay, p)
                assert not psync_r.read(p).any() and not psync_b.read(p).any()
            assert rs.take_status() == 0
        # the oracle agrees with the closed form used above
        heap = oracle.Heap(n_pes, 2 * n * 8)
        for p in range(n_pes):
            heap.view(p, 0, n, np.int64)[:] = host[p]
        oracle.to_all(heap, rs.LONG, rs.SUM, n * 8, 0, n)
        assert np.array_equal(heap.view(2, n * 8, n, np.int64), total)
        graph.destroy()
        stream.destroy()


def test_capture_on_the_default_stream_is_refused():
    with runtime(2):
        class Null:
            h = None
        with pytest.raises(rs.RocShmemError):
            rs.Graph.capture(Null()).__enter__()
