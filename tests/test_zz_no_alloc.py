"""gd_backend_sdpa_decode_positions_noalloc: the split-KV decode entry point that allocates nothing.

It shares the kernels of gd_backend_sdpa_decode_positions, so its output must equal that entry point's bit
for bit; its split-KV partial results live in one fixed device array that keeps the previous call's contents,
so the cases run back to back, the second smaller than the first.  Named so that it is collected last.
"""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _bits(a):
    return np.ascontiguousarray(a).view(np.uint16)


def _pair(backend, arena, oracle, B, H, Hkv, D, Tmax, pos, seed, window=0, prefix=0):
    """Runs the no-alloc entry point and the regular one on the same inputs; returns both outputs."""
    q = oracle.normal_f16((B, 1, H, D), seed)
    k = oracle.normal_f16((B, Tmax, Hkv, D), seed + 1)
    v = oracle.normal_f16((B, Tmax, Hkv, D), seed + 2)
    sentinel = np.full(q.shape, 7.0, np.float16)
    tq, tk, tv = arena.from_numpy(q), arena.from_numpy(k), arena.from_numpy(v)
    tp = arena.from_numpy(np.asarray(pos, np.int32))
    out_n, out_r = arena.from_numpy(sentinel), arena.from_numpy(sentinel)
    scale = 1.0 / np.sqrt(D)
    backend.sdpa_decode_positions_noalloc(tq, tk, tv, tp, out_n, scale, window, prefix)
    backend.sdpa_decode_positions(tq, tk, tv, tp, out_r, scale, window, prefix)
    want = oracle.sdpa_decode(q, k, v, pos, scale, window, prefix, out_init=sentinel.astype(np.float32))
    return out_n.read(), out_r.read(), want


def test_noalloc_equals_the_allocating_entry_point_on_two_calls_in_a_row(backend, gda, oracle):
    arena = backend.buffer(256 << 20)
    try:
        # first call: 4 rows x 8 heads over up to 6000 keys -> the key range is split (partials in the scratch);
        # one row is untouched (negative position), one is shorter than a split
        pos = [5999, 3000, -1, 17]
        a_n, a_r, a_w = _pair(backend, arena, oracle, 4, 8, 8, 64, 6000, pos, 4100)
        assert np.array_equal(_bits(a_n), _bits(a_r))
        assert np.abs(a_n.astype(np.float64) - a_w).max() < 2e-3
        # second call, smaller (fewer rows, fewer splits, grouped heads, head size 128): stale partials of the
        # first call lie in every slot it uses and beyond
        arena.reset()
        pos = [1500, 2047]
        b_n, b_r, b_w = _pair(backend, arena, oracle, 2, 8, 4, 128, 2048, pos, 4200)
        assert np.array_equal(_bits(b_n), _bits(b_r))
        assert np.abs(b_n.astype(np.float64) - b_w).max() < 2e-3
        # third: window + prefix (the two-run walk), a single row
        arena.reset()
        c_n, c_r, c_w = _pair(backend, arena, oracle, 1, 4, 4, 64, 4096, [4000], 4300, window=1500, prefix=64)
        assert np.array_equal(_bits(c_n), _bits(c_r))
        assert np.abs(c_n.astype(np.float64) - c_w).max() < 2e-3
    finally:
        backend.free(arena)


def test_noalloc_without_a_split_and_generic_shapes(backend, gda, oracle):
    """Shapes that need no partial results: one workgroup per (row, head), and the generic kernel (F32 tensors with
    two query tokens per row)."""
    arena = backend.buffer(256 << 20)
    try:
        pos = list(oracle.uniform_i32(64, 4400, 1, 511))
        n, r, w = _pair(backend, arena, oracle, 64, 8, 8, 64, 512, pos, 4401)
        assert "split_kernel" in backend.sdpa_decode_last_kernel()
        assert np.array_equal(_bits(n), _bits(r))
        assert np.abs(n.astype(np.float64) - w).max() < 2e-3
        arena.reset()
        B, Tq, H, Hkv, D, Tmax = 3, 2, 4, 2, 40, 70
        q = oracle.normal_f16((B, Tq, H, D), 4410).astype(np.float32)
        k = oracle.normal_f16((B, Tmax, Hkv, D), 4411).astype(np.float32)
        v = oracle.normal_f16((B, Tmax, Hkv, D), 4412).astype(np.float32)
        pos = np.array([0, 33, 60], np.int32)
        tq, tk, tv, tp = (arena.from_numpy(a) for a in (q, k, v, pos))
        out_n, out_r = arena.from_numpy(np.zeros(q.shape, np.float32)), arena.from_numpy(np.zeros(q.shape, np.float32))
        backend.sdpa_decode_positions_noalloc(tq, tk, tv, tp, out_n, 0.2)
        assert "generic" in backend.sdpa_decode_last_kernel()
        backend.sdpa_decode_positions(tq, tk, tv, tp, out_r, 0.2)
        assert np.array_equal(out_n.read().view(np.uint32), out_r.read().view(np.uint32))
        want = oracle.sdpa_decode(q.astype(np.float16), k.astype(np.float16), v.astype(np.float16), pos, 0.2)
        assert np.abs(out_n.read().astype(np.float64) - want).max() < 1e-5
    finally:
        backend.free(arena)


def test_noalloc_ragged_rows_in_pieces_and_under_graph_capture(backend, gda, oracle):
    """The form that cuts the rows of a ragged batch into pieces keeps its arrival counters and partial results in
    the fixed array too (counters are back at zero after every launch).  Then the entry point is captured into a
    graph, as a caller that cannot allocate would use it, and replayed three times with eager calls of other sizes
    in between: every replay must give the bits of the eager call."""
    arena = backend.buffer(256 << 20)
    try:
        B, H, D, Tmax = 40, 8, 64, 1100
        pos = oracle.uniform_i32(B, 4500, 0, Tmax - 1)
        pos[3], pos[7] = -1, Tmax + 3
        for _ in range(2):
            arena.reset()
            n, r, w = _pair(backend, arena, oracle, B, H, H, D, Tmax, pos, 4501)
            if B * H >= backend.device_info()[1]:
                assert "rows merged by the last piece" in backend.sdpa_decode_last_kernel()
            assert np.array_equal(_bits(n), _bits(r))
            assert np.abs(n.astype(np.float64) - w).max() < 2e-3
        arena.reset()
        # split partials (4 rows x 8 heads over 6000 keys) under capture
        q = oracle.normal_f16((4, 1, 8, 64), 4600)
        k, v = oracle.normal_f16((4, 6000, 8, 64), 4601), oracle.normal_f16((4, 6000, 8, 64), 4602)
        tq, tk, tv = arena.from_numpy(q), arena.from_numpy(k), arena.from_numpy(v)
        tp = arena.from_numpy(np.array([5999, 3000, -1, 17], np.int32))
        eager, out = arena.from_numpy(np.full(q.shape, 7.0, np.float16)), arena.from_numpy(np.full(q.shape, 7.0, np.float16))
        backend.sdpa_decode_positions_noalloc(tq, tk, tv, tp, eager, 0.125)
        assert "combine kernel" in backend.sdpa_decode_last_kernel()
        backend.scope_begin()
        backend.graph_begin_capture()
        backend.sdpa_decode_positions_noalloc(tq, tk, tv, tp, out, 0.125)
        graph = backend.graph_end_capture()
        try:
            for i in range(3):
                backend.fill(out, 0x4700)
                backend.graph_launch(graph)
                backend.fence_wait(backend.record_fence())
                assert np.array_equal(_bits(out.read()), _bits(eager.read())), i
                # an eager call of another size dirties the shared array between the replays
                other = arena.from_numpy(np.zeros((2, 1, 8, 64), np.float16))
                backend.sdpa_decode_positions_noalloc(arena.from_numpy(q[:2]), arena.from_numpy(k[:2, :3000]),
                                                      arena.from_numpy(v[:2, :3000]),
                                                      arena.from_numpy(np.array([2999, 100], np.int32)), other, 0.125)
                backend.scope_begin()
        finally:
            backend.fence_wait(backend.record_fence())
            backend.graph_destroy(graph)
    finally:
        backend.free(arena)


def test_noalloc_rejects_what_the_fixed_scratch_cannot_hold(backend, gda):
    """A launch whose partial results would need more than the fixed array is refused with GD_ERR_OUT_OF_MEMORY
    before anything is launched; the output stays untouched."""
    B, H, D, Tmax = 2, 8, 128, 65536
    arena = backend.buffer((2 * B * Tmax * H * D + 4 * B * H * D) * 2 + (1 << 20))
    try:
        q = arena.alloc((B, 1, H, D), gda.F16)
        k = arena.alloc((B, Tmax, H, D), gda.F16)
        v = arena.alloc((B, Tmax, H, D), gda.F16)
        out = arena.alloc((B, 1, H, D), gda.F16)
        backend.fill(out, 0x4700)
        pos = arena.from_numpy(np.full(B, Tmax - 1, np.int32))
        a = gda.SdpaDecodeArgs(0.1, 0, 0, 0)
        backend.set_tunable("sdpa_chunk", 32)  # 2048 splits x 16 (row, head) pairs x 130 floats = 17 MB
        backend.set_tunable("sdpa_merge", 0)   # (rows merged inside the kernel are cut into 16 pieces at most)
        try:
            st = backend.call("gd_backend_sdpa_decode_positions_noalloc", q.view(), k.view(), v.view(), pos.view(),
                              out.view(), C.byref(a))
        finally:
            backend.set_tunable("sdpa_chunk", 0)
            backend.set_tunable("sdpa_merge", 1)
        assert st == -2  # GD_ERR_OUT_OF_MEMORY
        assert np.all(out.read().view(np.uint16) == 0x4700)
        # bad arguments are still bad arguments
        bad = gda.SdpaDecodeArgs(float("nan"), 0, 0, 0)
        assert backend.call("gd_backend_sdpa_decode_positions_noalloc", q.view(), k.view(), v.view(), pos.view(),
                            out.view(), C.byref(bad)) == gda.INVALID_ARGUMENT
    finally:
        backend.free(arena)
