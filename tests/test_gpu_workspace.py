"""The split-KV workspace of the backend and the graphs that captured its address."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_graph_replay_survives_a_workspace_that_grew_meanwhile(backend, gda, oracle):
    """A captured sdpa_decode holds the address of the partial-result workspace of its capture.  A later, larger
    call on the same backend replaces the workspace; the old block must stay allocated while the graph lives, so a
    replay afterwards still gives the eager result."""
    arena = backend.buffer(128 << 20)
    try:
        B, H, D, Tmax = 2, 4, 64, 4096
        q = oracle.normal_f16((B, 1, H, D), 5100)
        k = oracle.normal_f16((B, Tmax, H, D), 5101)
        v = oracle.normal_f16((B, Tmax, H, D), 5102)
        pos = np.array([4095, 2100], np.int32)
        tq, tk, tv, tp = arena.from_numpy(q), arena.from_numpy(k), arena.from_numpy(v), arena.from_numpy(pos)
        eager, replay = arena.alloc(q.shape, gda.F16), arena.alloc(q.shape, gda.F16)
        backend.sdpa_decode_positions(tq, tk, tv, tp, eager, 0.125)  # sizes the workspace for this shape
        want = eager.read()
        backend.scope_begin()
        backend.graph_begin_capture()
        backend.sdpa_decode_positions(tq, tk, tv, tp, replay, 0.125)
        graph = backend.graph_end_capture()
        backend.fence_wait(backend.record_fence())
        try:
            # a call with more (row, head, split) slots than any before: the workspace grows
            B2, H2, T2 = 3, 16, 8192
            q2 = arena.alloc((B2, 1, H2, D), gda.F16)
            k2 = arena.alloc((B2, T2, H2, D), gda.F16)
            v2 = arena.alloc((B2, T2, H2, D), gda.F16)
            o2 = arena.alloc((B2, 1, H2, D), gda.F16)
            for t in (q2, k2, v2):
                backend.rand_uniform(t, 7, -1.0, 1.0)
            p2 = arena.from_numpy(np.full(B2, T2 - 1, np.int32))
            backend.set_tunable("sdpa_chunk", 64)
            try:
                backend.sdpa_decode_positions(q2, k2, v2, p2, o2, 0.125)
            finally:
                backend.set_tunable("sdpa_chunk", 0)
            for _ in range(3):
                backend.fill(replay, 0)
                backend.scope_begin()
                backend.graph_launch(graph)
                backend.fence_wait(backend.record_fence())
                assert np.array_equal(replay.read().view(np.uint16), want.view(np.uint16))
        finally:
            backend.graph_destroy(graph)
    finally:
        backend.free(arena)


def test_many_queued_graph_launches_stay_bounded_and_ordered(backend, gda):
    """200 replays of a small graph queued without a wait in between (the backend bounds the number in flight):
    each replay adds 1 to a counter, the result counts them all."""
    arena = backend.buffer(1 << 20)
    try:
        c = arena.from_numpy(np.zeros(64, np.int32))
        backend.scope_begin()
        backend.graph_begin_capture()
        backend.add_scalar_i32(c, c, 1)
        graph = backend.graph_end_capture()
        try:
            for _ in range(200):
                backend.graph_launch(graph)
            backend.fence_wait(backend.record_fence())
            assert np.all(c.read() == 200)
        finally:
            backend.graph_destroy(graph)
    finally:
        backend.free(arena)
