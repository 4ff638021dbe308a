"""Parity of every HIP operator against the CPU oracle, through the C-ABI.

Bars (BASELINE.json north_star): cache append, gathers, argmax ids and index maps are
bit-exact; sdpa_decode, projections and rms_norm are within rtol 2e-3 / atol 1e-3 of the
oracle in F16.  Inputs come from the oracle's splitmix64 + Box-Muller generator, seeded.
"""
import ctypes as C
import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
RTOL, ATOL = 2e-3, 1e-3


def _golden(name):
    with open(os.path.join(GOLDEN, name)) as f:
        return json.load(f)


def _close(got, want, rtol=RTOL, atol=ATOL, through=None):
    """`through`: an intermediate the result was formed from by an F16 add; its magnitude, not the
    (possibly cancelled) result's, sets the size of one rounding step."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    err = np.abs(got - want)
    bound = atol + rtol * np.abs(want)
    if through is not None:
        bound = bound + rtol * np.abs(np.asarray(through, np.float64))
    if not np.all(err <= bound):
        at = np.unravel_index(np.argmax(err - bound), err.shape)
        raise AssertionError(f"max err {err.max():.3e}, worst excess {(err - bound).max():.3e} at {at}: got {got[at]!r} "
                             f"want {want[at]!r} bound {bound[at]:.3e}")


def _bits(a):
    return np.ascontiguousarray(a).view(np.uint16 if a.dtype == np.float16 else np.uint32)


@pytest.fixture()
def arena(backend):
    buf = backend.buffer(512 << 20)
    yield buf
    backend.free(buf)


# ---- lifecycle -------------------------------------------------------------------------

def test_backend_identity_and_scope_rules(backend, gda):
    assert backend.name.startswith("hip:")
    assert gda.lib().gd_backend_kind_query(backend.handle) == 2
    backend.scope_begin()
    assert backend.call("gd_backend_scope_begin") == gda.BAD_STATE  # nested scope
    f = backend.record_fence()
    backend.fence_wait(f)
    name, cus, mem = backend.device_info()
    assert cus > 0 and mem > (1 << 30)


def test_upload_download_fill(backend, arena, gda):
    rng = np.random.default_rng(0)
    a = rng.integers(0, 255, 100003, dtype=np.uint8)
    t = arena.from_numpy(a)
    assert np.array_equal(t.read(), a)
    h = arena.alloc((1001,), gda.F16)
    backend.fill(h, 0x3c00)
    assert np.all(h.read() == np.float16(1.0))
    w = arena.alloc((77,), gda.I32)
    backend.fill(w, 0xdeadbeef)
    assert np.all(w.read().view(np.uint32) == 0xdeadbeef)
    b = arena.alloc((13,), gda.U8)
    backend.fill(b, 0x5a)
    assert np.all(b.read() == 0x5a)
    # queued work is visible to a download inside a scope (program order)
    backend.scope_begin()
    backend.fill(h, 0x4000)
    assert np.all(h.read() == np.float16(2.0))
    backend.fence_wait(backend.record_fence())


# ---- A1 kv_cache_append -------------------------------------------------------------------

@pytest.mark.parametrize("np_dtype", [np.float32, np.float16])
def test_append_reference_golden_vectors(backend, arena, gda, np_dtype):
    g = _golden("kv_cache_append_vectors.json")
    c = g["at"]
    k = arena.from_numpy(np.zeros(c["cache_shape"], np_dtype))
    v = arena.from_numpy(np.zeros(c["cache_shape"], np_dtype))
    kn = arena.from_numpy(np.array(c["k_new"], np_dtype).reshape(c["new_shape"]))
    vn = arena.from_numpy(np.array(c["v_new"], np_dtype).reshape(c["new_shape"]))
    backend.kv_cache_append_at(k, v, c["cache_pos"], kn, vn)
    assert np.array_equal(k.read().ravel(), np.array(c["expect_k"], np_dtype))
    assert np.array_equal(v.read().ravel(), np.array(c["expect_v"], np_dtype))
    c = g["positions"]
    k = arena.from_numpy(np.zeros(c["cache_shape"], np_dtype))
    v = arena.from_numpy(np.zeros(c["cache_shape"], np_dtype))
    kn = arena.from_numpy(np.array(c["k_new"], np_dtype).reshape(c["new_shape"]))
    vn = arena.from_numpy(np.array(c["v_new"], np_dtype).reshape(c["new_shape"]))
    pos = arena.from_numpy(np.array(c["cache_pos"], np.int32))
    backend.kv_cache_append_positions(k, v, pos, kn, vn)
    assert np.array_equal(k.read().ravel(), np.array(c["expect_k"], np_dtype))
    assert np.array_equal(v.read().ravel(), np.array(c["expect_v"], np_dtype))
    c = g["packed"]
    k = arena.from_numpy(np.zeros(c["cache_shape"], np_dtype))
    v = arena.from_numpy(np.zeros(c["cache_shape"], np_dtype))
    kn = arena.from_numpy(np.array(c["k_new"], np_dtype).reshape(c["new_shape"]))
    vn = arena.from_numpy(np.array(c["v_new"], np_dtype).reshape(c["new_shape"]))
    pos = arena.from_numpy(np.array(c["cache_pos"], np.int32))
    cu = arena.from_numpy(np.array(c["cu_seqlens"], np.int32))
    backend.kv_cache_append_packed(k, v, pos, cu, kn, vn)
    assert np.array_equal(k.read().ravel(), np.array(c["expect_k"], np_dtype))
    assert np.array_equal(v.read().ravel(), np.array(c["expect_v"], np_dtype))


def test_append_positions_bit_exact_with_skips(backend, arena, oracle):
    B, Tmax, H, D = 32, 300, 8, 64
    k0, v0 = oracle.normal_f16((B, Tmax, H, D), 11), oracle.normal_f16((B, Tmax, H, D), 12)
    kn, vn = oracle.normal_f16((B, 1, H, D), 13), oracle.normal_f16((B, 1, H, D), 14)
    pos = oracle.uniform_i32(B, 15, 0, Tmax - 1)
    pos[3], pos[7], pos[9] = -1, Tmax, Tmax - 1  # skipped, skipped, last valid slot
    k, v = arena.from_numpy(k0), arena.from_numpy(v0)
    backend.kv_cache_append_positions(k, v, arena.from_numpy(pos), arena.from_numpy(kn), arena.from_numpy(vn))
    wk, wv = k0.copy(), v0.copy()
    oracle.kv_cache_append(wk, wv, kn, vn, pos)
    assert np.array_equal(_bits(k.read()), _bits(wk)) and np.array_equal(_bits(v.read()), _bits(wv))


@pytest.mark.parametrize("D,tnew", [(64, 3), (6, 2), (5, 1)])  # 16-, 4- and 1-byte copy units
def test_append_copy_units_and_multi_token(backend, arena, oracle, D, tnew):
    B, Tmax, H = 3, 9, 2
    k0, v0 = oracle.normal_f16((B, Tmax, H, D), 21), oracle.normal_f16((B, Tmax, H, D), 22)
    kn, vn = oracle.normal_f16((B, tnew, H, D), 23), oracle.normal_f16((B, tnew, H, D), 24)
    pos = np.array([0, 4, Tmax - tnew], np.int32)
    k, v = arena.from_numpy(k0), arena.from_numpy(v0)
    backend.kv_cache_append_positions(k, v, arena.from_numpy(pos), arena.from_numpy(kn), arena.from_numpy(vn))
    wk, wv = k0.copy(), v0.copy()
    oracle.kv_cache_append(wk, wv, kn, vn, pos)
    assert np.array_equal(_bits(k.read()), _bits(wk)) and np.array_equal(_bits(v.read()), _bits(wv))


def test_append_packed_bit_exact_with_skips(backend, arena, oracle):
    B, Tmax, H, D = 6, 40, 4, 32
    lens = np.array([7, 0, 40, 13, 5, 9], np.int32)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    pos = np.array([0, 3, 0, 30, -2, 31], np.int32)  # seq 3 overflows (30+13), seq 4 negative, seq 5 fits exactly
    N = int(cu[-1]) + 3
    k0, v0 = oracle.normal_f16((B, Tmax, H, D), 31), oracle.normal_f16((B, Tmax, H, D), 32)
    kn, vn = oracle.normal_f16((N, H, D), 33), oracle.normal_f16((N, H, D), 34)
    k, v = arena.from_numpy(k0), arena.from_numpy(v0)
    backend.kv_cache_append_packed(k, v, arena.from_numpy(pos), arena.from_numpy(cu), arena.from_numpy(kn),
                                   arena.from_numpy(vn))
    wk, wv = k0.copy(), v0.copy()
    oracle.kv_cache_append_packed(wk, wv, kn, vn, pos, cu)
    assert np.array_equal(_bits(k.read()), _bits(wk)) and np.array_equal(_bits(v.read()), _bits(wv))


def test_append_rejects_bad_arguments(backend, arena, gda):
    k = arena.alloc((2, 5, 1, 8), gda.F16)
    v = arena.alloc((2, 5, 1, 8), gda.F16)
    kn = arena.alloc((2, 2, 1, 8), gda.F16)
    vn = arena.alloc((2, 2, 1, 8), gda.F16)
    bad_d = arena.alloc((2, 2, 1, 4), gda.F16)
    for cache_pos in (-1, 4, 6):  # negative, span passes Tmax, beyond Tmax
        a = gda.KvAppendArgs(cache_pos)
        st = backend.call("gd_backend_kv_cache_append_at", k.view(), v.view(), kn.view(), vn.view(), C.byref(a))
        assert st == gda.INVALID_ARGUMENT
    a = gda.KvAppendArgs(0)
    assert backend.call("gd_backend_kv_cache_append_at", k.view(), v.view(), bad_d.view(), bad_d.view(),
                        C.byref(a)) == gda.INVALID_ARGUMENT
    pos3 = arena.alloc((3,), gda.I32)
    assert backend.call("gd_backend_kv_cache_append_positions", k.view(), v.view(), pos3.view(), kn.view(),
                        vn.view(), C.byref(a)) == gda.INVALID_ARGUMENT


# ---- A2 sdpa_decode -------------------------------------------------------------------------

def test_decode_reference_test_case(backend, arena, oracle):
    """tests/test_sdpa_varlen.c:679-719 of the reference: Tq=2, GQA 2:1, Dh=4, rank-0 position tensor."""
    c = _golden("reference_test_cases.json")["sdpa_decode_test_decode"]
    B, Tq, Tmax, Hq, Hkv, D = (c[x] for x in ("B", "Tq", "Tmax", "Hq", "Hkv", "Dh"))
    q = oracle.fill_tokens(B * Tq * Hq * D, c["q_base"]).reshape(B, Tq, Hq, D)
    k = oracle.fill_tokens(B * Tmax * Hkv * D, c["k_base"]).reshape(B, Tmax, Hkv, D)
    v = oracle.fill_tokens(B * Tmax * Hkv * D, c["v_base"]).reshape(B, Tmax, Hkv, D)
    tq, tk, tv = arena.from_numpy(q), arena.from_numpy(k), arena.from_numpy(v)
    pos = arena.from_numpy(np.array([c["cache_pos"]], np.int32))
    out = arena.from_numpy(np.zeros(q.shape, np.float16))
    backend.sdpa_decode(tq, tk, tv, pos, out, c["scale"])
    want = oracle.sdpa_decode(q, k, v, [c["cache_pos"]], c["scale"])
    assert np.abs(out.read().astype(np.float32) - want).max() < c["tol_abs"]


def test_decode_positions_equals_scalar_f32(backend, arena, oracle, gda):
    """tests/test_kv_cache_decode.c:181-303 of the reference: three position forms agree (F32 tensors)."""
    c = _golden("reference_test_cases.json")["sdpa_decode_positions_vs_scalar"]
    qs, ks = c["q_shape"], c["kv_shape"]
    i = np.arange(int(np.prod(qs)), dtype=np.float32)
    q = ((i - 7.0) * 0.03).astype(np.float32).reshape(qs)
    j = np.arange(int(np.prod(ks)), dtype=np.float32)
    k = ((j - 11.0) * 0.02).astype(np.float32).reshape(ks)
    v = ((j + 3.0) * -0.015).astype(np.float32).reshape(ks)
    tq, tk, tv = arena.from_numpy(q), arena.from_numpy(k), arena.from_numpy(v)
    pos = arena.from_numpy(np.array(c["cache_pos"], np.int32))
    out = arena.from_numpy(np.zeros(qs, np.float32))
    backend.sdpa_decode_positions(tq, tk, tv, pos, out, c["scale"])
    got = out.read()
    for b in range(qs[0]):
        ob = arena.from_numpy(np.zeros([1] + qs[1:], np.float32))
        backend.sdpa_decode_at(tq.rows(b, 1), tk.rows(b, 1), tv.rows(b, 1), c["cache_pos"][b], ob, c["scale"])
        assert np.abs(ob.read()[0] - got[b]).max() < c["tol_abs"]
        p0 = arena.from_numpy(np.array([c["cache_pos"][b]], np.int32))
        ot = arena.from_numpy(np.zeros([1] + qs[1:], np.float32))
        backend.sdpa_decode(tq.rows(b, 1), tk.rows(b, 1), tv.rows(b, 1), p0, ot, c["scale"])
        assert np.abs(ot.read()[0] - got[b]).max() < c["tol_abs"]
    _close(got, oracle.sdpa_decode(q, k, v, c["cache_pos"], c["scale"]), 1e-5, 1e-6)


def _split_kernel_args(name):
    """Template arguments of the split-KV kernel as gd_backend_sdpa_decode_last_kernel prints them: head size, query
    heads per kv head, wavefronts, trip length, streaming loads[, prefix[, pieces, first rows ahead of the position]]."""
    assert name.startswith("gd_sdpa_decode_split_kernel<"), name
    return name[name.index("<") + 1:name.index(">")].split(",")


def _decode_case(backend, arena, oracle, B, H, Hkv, D, Tmax, pos, scale, window=0, seed=100, chunk=0):
    q = oracle.normal_f16((B, 1, H, D), seed)
    k = oracle.normal_f16((B, Tmax, Hkv, D), seed + 1)
    v = oracle.normal_f16((B, Tmax, Hkv, D), seed + 2)
    sentinel = np.full(q.shape, 7.0, np.float16)
    tq, tk, tv = arena.from_numpy(q), arena.from_numpy(k), arena.from_numpy(v)
    tp, out = arena.from_numpy(np.asarray(pos, np.int32)), arena.from_numpy(sentinel)
    backend.set_tunable("sdpa_chunk", chunk)
    try:
        backend.sdpa_decode_positions(tq, tk, tv, tp, out, scale, window)
    finally:
        backend.set_tunable("sdpa_chunk", 0)
    want = oracle.sdpa_decode(q, k, v, pos, scale, window, out_init=sentinel.astype(np.float32))
    _close(out.read(), want)
    return out.read()


@pytest.mark.parametrize("chunk", [0, 64, 1024])
def test_decode_isolated_config_shape(backend, arena, oracle, chunk):
    """BASELINE config 1 at a length the oracle finishes in seconds: B=32, H=8, DH=64, ragged lengths,
    append one token then decode over L+1 keys, scale 1/8."""
    B, H, D, Tmax = 32, 8, 64, 1025
    L = oracle.uniform_i32(B, 1001, 1, Tmax - 1)
    k0, v0 = oracle.normal_f16((B, Tmax, H, D), 1002), oracle.normal_f16((B, Tmax, H, D), 1003)
    q, kn, vn = (oracle.normal_f16((B, 1, H, D), s) for s in (1004, 1005, 1006))
    tk, tv, tp = arena.from_numpy(k0), arena.from_numpy(v0), arena.from_numpy(L)
    backend.kv_cache_append_positions(tk, tv, tp, arena.from_numpy(kn), arena.from_numpy(vn))
    wk, wv = k0.copy(), v0.copy()
    oracle.kv_cache_append(wk, wv, kn, vn, L)
    assert np.array_equal(_bits(tk.read()), _bits(wk)) and np.array_equal(_bits(tv.read()), _bits(wv))
    out = arena.alloc(q.shape, 1)
    backend.set_tunable("sdpa_chunk", chunk)
    try:
        backend.sdpa_decode_positions(arena.from_numpy(q), tk, tv, tp, out, 0.125)
    finally:
        backend.set_tunable("sdpa_chunk", 0)
    _close(out.read(), oracle.sdpa_decode(q, wk, wv, L, 0.125))


def test_decode_isolated_config_full_size(backend, oracle):
    """BASELINE config 1 at its full size: B=32, H=8, DH=64, caches of 4097 rows, lengths uniform in [1, 4096]; one
    token appended per sequence (bit-exact), then the decode over L+1 keys against the oracle.  At this size (275 MB
    of caches) the dispatch marks the K/V loads streaming and cuts long rows into pieces that the last piece to arrive
    merges; with that switched off it picks the 8-wavefront form, one workgroup per (row, head): neither is reached
    by a smaller case."""
    B, H, D, Tmax = 32, 8, 64, 4097
    big = backend.buffer(640 << 20)
    try:
        L = oracle.uniform_i32(B, 1101, 1, 4096)
        k0, v0 = oracle.normal_f16((B, Tmax, H, D), 1102), oracle.normal_f16((B, Tmax, H, D), 1103)
        q, kn, vn = (oracle.normal_f16((B, 1, H, D), sd) for sd in (1104, 1105, 1106))
        tk, tv, tp = big.from_numpy(k0), big.from_numpy(v0), big.from_numpy(L)
        backend.kv_cache_append_positions(tk, tv, tp, big.from_numpy(kn), big.from_numpy(vn))
        oracle.kv_cache_append(k0, v0, kn, vn, L)
        assert np.array_equal(_bits(tk.read()), _bits(k0)) and np.array_equal(_bits(tv.read()), _bits(v0))
        want = oracle.sdpa_decode(q, k0, v0, L, 0.125)
        tq = big.from_numpy(q)
        for merge, form in ((1, "rows merged by the last piece"), (0, "<64,1,8,")):
            out = big.from_numpy(np.full(q.shape, 7.0, np.float16))
            backend.set_tunable("sdpa_merge", merge)
            try:
                backend.sdpa_decode_positions(tq, tk, tv, tp, out, 0.125)
            finally:
                backend.set_tunable("sdpa_merge", 1)
            name = backend.sdpa_decode_last_kernel()
            assert form in name and _split_kernel_args(name)[4] == "true", name
            _close(out.read(), want)
    finally:
        backend.free(big)


@pytest.mark.parametrize("H,Hkv,D", [(8, 8, 64), (16, 4, 128), (6, 3, 64)])
def test_decode_long_rows_in_pieces_merged_in_the_kernel(backend, arena, oracle, H, Hkv, D):
    """Rows cut into pieces whose partial results the last piece to arrive merges (one launch), against the oracle and
    against the form with a combine kernel behind the split kernel: a ragged batch (one-key rows, full rows, a row
    past the cache end, untouched rows, NaN behind every live range), cut at 64, 96 and 1024 keys; then the dispatch's
    own choice on 40 x Hkv (row, head) pairs with 1100-row caches, which is the merging form when there is a pair for
    every compute unit: ragged rows are cut at 256 keys, rows of about one length stay whole or are halved."""
    B, Tmax = 40, 1100
    rng = np.random.default_rng(77 + H)
    pos = rng.integers(0, Tmax, B).astype(np.int32)
    pos[[0, 1, 2, 3, 4, 5]] = [-1, 0, Tmax - 1, Tmax + 7, 255, 256]
    pos[B - 1] = -5
    q = oracle.normal_f16((B, 1, H, D), 70)
    k, v = oracle.normal_f16((B, Tmax, Hkv, D), 71), oracle.normal_f16((B, Tmax, Hkv, D), 72)
    kd, vd = k.copy(), v.copy()
    for b in range(B):
        if 0 <= pos[b] < Tmax - 1:
            kd[b, pos[b] + 1:] = np.nan
            vd[b, pos[b] + 1:] = np.nan
    sentinel = np.full(q.shape, 7.0, np.float16)
    tq, tk, tv = arena.from_numpy(q), arena.from_numpy(kd), arena.from_numpy(vd)
    scale = 1.0 / np.sqrt(D)

    def run(positions, merge, chunk, caches=None):
        out = arena.from_numpy(sentinel)
        ck, cv = caches or (tk, tv)
        backend.set_tunable("sdpa_merge", merge)
        backend.set_tunable("sdpa_chunk", chunk)
        try:
            backend.sdpa_decode_positions(tq, ck, cv, arena.from_numpy(positions), out, scale)
        finally:
            backend.set_tunable("sdpa_merge", 1)
            backend.set_tunable("sdpa_chunk", 0)
        return out.read(), backend.sdpa_decode_last_kernel()

    want = oracle.sdpa_decode(q, k, v, pos, scale, out_init=sentinel.astype(np.float32))
    for chunk in (64, 96, 1024):
        merged, name = run(pos, 2, chunk)
        assert "rows merged by the last piece" in name, name
        combined, name = run(pos, 0, chunk)
        assert "combine kernel" in name, name
        for got in (merged, combined):
            assert np.isfinite(got.astype(np.float32)).all()
            assert (got[0] == 7.0).all() and (got[B - 1] == 7.0).all()
            _close(got, want)
        assert np.abs(merged.astype(np.float32) - combined.astype(np.float32)).max() < 1e-3
    # twice in a row: the arrival counters are back at zero after a launch
    for _ in range(2):
        got, name = run(pos, 1, 0)
        assert ("rows merged by the last piece" in name) == (B * Hkv >= backend.device_info()[1]), name
        _close(got, want)
    even = rng.integers(1000, Tmax, B).astype(np.int32)
    even[7] = -1
    got, _ = run(even, 1, 0, (arena.from_numpy(k), arena.from_numpy(v)))
    _close(got, oracle.sdpa_decode(q, k, v, even, scale, out_init=sentinel.astype(np.float32)))


@pytest.mark.parametrize("D,chunk", [(64, 0), (64, 32), (128, 0), (128, 64)])
def test_decode_ignores_rows_behind_the_live_range(backend, arena, oracle, D, chunk):
    """Cache rows behind a sequence's last live key may hold anything (another request's rows, NaN, infinities): the
    result must not depend on them.  Every row from position + 1 on is filled with NaN (K) and infinities (V); rows
    with 1, 2, 7, 33 and 300 live keys plus a full one, so that the first loads of a workgroup reach behind the
    range in every way."""
    B, H, Tmax = 6, 4, 384
    pos = np.array([0, 1, 6, 32, 299, Tmax - 1], np.int32)
    q = oracle.normal_f16((B, 1, H, D), 50)
    k, v = oracle.normal_f16((B, Tmax, H, D), 51), oracle.normal_f16((B, Tmax, H, D), 52)
    kd, vd = k.copy(), v.copy()
    for b in range(B):
        kd[b, pos[b] + 1:] = np.nan
        vd[b, pos[b] + 1:] = np.inf
        vd[b, pos[b] + 1::2] = -np.inf
    out = arena.from_numpy(np.full(q.shape, 7.0, np.float16))
    backend.set_tunable("sdpa_chunk", chunk)
    try:
        backend.sdpa_decode_positions(arena.from_numpy(q), arena.from_numpy(kd), arena.from_numpy(vd),
                                      arena.from_numpy(pos), out, 1.0 / np.sqrt(D))
    finally:
        backend.set_tunable("sdpa_chunk", 0)
    got = out.read()
    assert np.isfinite(got.astype(np.float32)).all()
    _close(got, oracle.sdpa_decode(q, k, v, pos, 1.0 / np.sqrt(D)))


def test_decode_full_size_long_context_sampled(backend, oracle):
    """BASELINE config 3's attention at its full size (B=16, 16 heads of 128, 4096-row caches, live lengths in
    [1024, 4096]: 537 MB of cache filled on the device), checked on sampled batch rows against a float64 softmax of
    the downloaded rows, and for independence from the split of the key range (size-independent property)."""
    B, H, D, T = 16, 16, 128, 4096
    big = backend.buffer(640 << 20)
    try:
        k, v = big.alloc((B, T, H, D), 1), big.alloc((B, T, H, D), 1)
        backend.rand_uniform(k, 9001, -1.0, 1.0)
        backend.rand_uniform(v, 9002, -1.0, 1.0)
        q = oracle.normal_f16((B, 1, H, D), 9003)
        pos = oracle.uniform_i32(B, 9004, 1023, 4095)
        tq, tp, out = big.from_numpy(q), big.from_numpy(pos), big.alloc((B, 1, H, D), 1)
        scale = 1.0 / np.sqrt(D)
        results = []
        for chunk in (0, 512, 2048):
            backend.set_tunable("sdpa_chunk", chunk)
            try:
                backend.sdpa_decode_positions(tq, k, v, tp, out, scale)
            finally:
                backend.set_tunable("sdpa_chunk", 0)
            results.append(out.read().astype(np.float32))
        assert np.abs(results[0] - results[1]).max() < 1e-3 and np.abs(results[0] - results[2]).max() < 1e-3
        for b in (0, 7, 15):
            n = int(pos[b]) + 1
            kb = k.rows(b, 1).read()[0, :n].astype(np.float64)  # [n, H, D]
            vb = v.rows(b, 1).read()[0, :n].astype(np.float64)
            sc = np.einsum("hd,nhd->hn", q[b, 0].astype(np.float64), kb) * scale
            w = np.exp(sc - sc.max(axis=1, keepdims=True))
            want = np.einsum("hn,nhd->hd", w / w.sum(axis=1, keepdims=True), vb)
            got = results[0][b, 0]
            assert np.all(np.abs(got - want) <= 1e-3 + 2e-3 * np.abs(want)), b
    finally:
        backend.free(big)


# query heads per kv head: 1, 4, 8, 2, 3, 6 (the split-KV kernel) and 5 (the generic kernel)
@pytest.mark.parametrize("H,Hkv,D", [(8, 8, 64), (16, 16, 128), (8, 2, 64), (8, 1, 128), (6, 3, 64), (6, 2, 64),
                                     (12, 2, 128), (6, 1, 64), (10, 2, 64)])
def test_decode_head_layouts(backend, arena, oracle, H, Hkv, D):
    pos = np.array([0, 1, 63, 64, 200, 299, -1, 31], np.int32)
    _decode_case(backend, arena, oracle, 8, H, Hkv, D, 300, pos, 1.0 / np.sqrt(D), seed=200 + H + D, chunk=96)


@pytest.mark.parametrize("H,Hkv,D", [(8, 8, 64), (16, 16, 128), (8, 2, 64), (6, 1, 64)])
@pytest.mark.parametrize("waves", [4, 8])
def test_decode_streaming_loads_give_the_same_bits(backend, arena, oracle, H, Hkv, D, waves):
    """The instantiations with streaming (non-temporal) K/V loads, which the dispatch picks by itself only above
    128 MiB of caches, forced on at a size the oracle covers: within the bar of the oracle, and the same bits as the
    cacheable form (the hint changes the cache policy of a load, not its value)."""
    pos = np.array([0, 1, 63, 64, 200, 299, -1, 31], np.int32)
    backend.set_tunable("sdpa_waves", waves)
    try:
        plain = _decode_case(backend, arena, oracle, 8, H, Hkv, D, 300, pos, 1.0 / np.sqrt(D), seed=230 + H + D, chunk=96)
        assert _split_kernel_args(backend.sdpa_decode_last_kernel())[4] == "false"
        backend.set_tunable("sdpa_nontemporal", 1)
        try:
            hinted = _decode_case(backend, arena, oracle, 8, H, Hkv, D, 300, pos, 1.0 / np.sqrt(D), seed=230 + H + D, chunk=96)
            name = backend.sdpa_decode_last_kernel()
        finally:
            backend.set_tunable("sdpa_nontemporal", -1)
    finally:
        backend.set_tunable("sdpa_waves", 0)
    args = _split_kernel_args(name)
    assert args[4] == "true" and (H != Hkv or args[2] == str(waves)) and args[-1] == "true", name   # ..., no window: first rows ahead
    assert np.array_equal(_bits(plain), _bits(hinted))


@pytest.mark.parametrize("window", [1, 7, 256, 1000])
def test_decode_sliding_window(backend, arena, oracle, window):
    pos = np.array([0, 5, 255, 256, 257, 511, 400, 100], np.int32)
    _decode_case(backend, arena, oracle, 8, 8, 8, 64, 512, pos, 0.125, window, seed=300 + window, chunk=64)


def test_decode_position_past_cache_end_clamps(backend, arena, oracle):
    _decode_case(backend, arena, oracle, 2, 4, 4, 64, 40, np.array([40, 100], np.int32), 0.125, seed=400)


@pytest.mark.parametrize("H,Hkv,D", [(8, 8, 64), (4, 1, 128), (6, 3, 64)])
@pytest.mark.parametrize("window,prefix", [(0, 5), (16, 4), (7, 40), (300, 64), (1, 1), (64, 700)])
def test_decode_prefix_and_window(backend, arena, oracle, H, Hkv, D, window, prefix):
    """Always-visible prefix in front of a sliding window (reference mask metal_sdpa_decode.metal:25-52, range helpers
    :55-84): queries inside the prefix, on its edge, behind it, far behind it (prefix and window apart) and past the
    end of the cache; head layouts of the split-KV kernel and one of the generic kernel; with and without a split of
    the visible keys."""
    Tmax = 700
    pos = np.array([0, 2, prefix - 1, prefix, prefix + 1, prefix + window, 333, 698, 699, 705, -1], np.int32)
    pos = np.clip(pos, -1, 705)
    B = pos.size
    q = oracle.normal_f16((B, 1, H, D), 4100 + window)
    k = oracle.normal_f16((B, Tmax, Hkv, D), 4101 + prefix)
    v = oracle.normal_f16((B, Tmax, Hkv, D), 4102)
    sentinel = np.full(q.shape, 7.0, np.float16)
    tq, tk, tv, tp = arena.from_numpy(q), arena.from_numpy(k), arena.from_numpy(v), arena.from_numpy(pos)
    want = oracle.sdpa_decode(q, k, v, pos, 0.11, window, prefix, out_init=sentinel.astype(np.float32))
    for chunk in (0, 32, 96):
        out = arena.from_numpy(sentinel)
        backend.set_tunable("sdpa_chunk", chunk)
        try:
            backend.sdpa_decode_positions(tq, tk, tv, tp, out, 0.11, window, prefix)
        finally:
            backend.set_tunable("sdpa_chunk", 0)
        _close(out.read(), want)
    # the prefix really is visible: a key inside it with a huge score owns the output of a row far behind it
    if prefix >= 2 and window > 0 and prefix + window < 333:
        k2 = k.copy()
        k2[6, 1] = (q[6, 0, :Hkv] * 40).astype(np.float16) if H == Hkv else k2[6, 1]
        out = arena.from_numpy(sentinel)
        backend.sdpa_decode_positions(tq, arena.from_numpy(k2), tv, tp, out, 0.11, window, prefix)
        _close(out.read(), oracle.sdpa_decode(q, k2, v, pos, 0.11, window, prefix, out_init=sentinel.astype(np.float32)))


def test_decode_generic_paths(backend, arena, oracle):
    """Tq > 1, odd head sizes and F32 caches take the generic kernel (prefix masks too when the head size is odd)."""
    rng_seed = 500
    for (Tq, D, window, prefix) in [(1, 64, 0, 3), (1, 64, 4, 2), (3, 64, 0, 0), (2, 40, 5, 0), (1, 72, 0, 0)]:
        B, H, Hkv, Tmax = 3, 4, 2, 70
        q = oracle.normal_f16((B, Tq, H, D), rng_seed)
        k = oracle.normal_f16((B, Tmax, Hkv, D), rng_seed + 1)
        v = oracle.normal_f16((B, Tmax, Hkv, D), rng_seed + 2)
        pos = np.array([0, 33, 66], np.int32)
        out = arena.from_numpy(np.zeros(q.shape, np.float16))
        backend.sdpa_decode_positions(arena.from_numpy(q), arena.from_numpy(k), arena.from_numpy(v),
                                      arena.from_numpy(pos), out, 0.2, window, prefix)
        _close(out.read(), oracle.sdpa_decode(q, k, v, pos, 0.2, window, prefix))
        rng_seed += 10


def test_decode_closed_forms(backend, arena, oracle):
    B, H, D, Tmax = 4, 8, 64, 130
    q = oracle.normal_f16((B, 1, H, D), 600)
    v = oracle.normal_f16((B, Tmax, H, D), 601)
    k = np.broadcast_to(oracle.normal_f16((1, 1, H, D), 602), (B, Tmax, H, D)).copy()
    pos = np.array([129, 64, 0, 17], np.int32)
    out = arena.alloc(q.shape, 1)
    backend.sdpa_decode_positions(arena.from_numpy(q), arena.from_numpy(k), arena.from_numpy(v),
                                  arena.from_numpy(pos), out, 0.125)
    got = out.read().astype(np.float64)
    for b in range(B):  # equal keys -> mean of the visible values; one key -> that value
        _close(got[b, 0], v[b, : pos[b] + 1].astype(np.float64).mean(0))
    assert np.array_equal(_bits(out.read()[2, 0]), _bits(v[2, 0]))


def test_decode_rejects_bad_arguments(backend, arena, gda):
    q = arena.alloc((2, 1, 4, 64), gda.F16)
    k = arena.alloc((2, 16, 2, 64), gda.F16)
    out = arena.alloc((2, 1, 4, 64), gda.F16)
    pos = arena.alloc((2,), gda.I32)
    a = gda.SdpaDecodeArgs(0.125, 0, 0, 0)
    ok = backend.call("gd_backend_sdpa_decode_positions", q.view(), k.view(), k.view(), pos.view(), out.view(), C.byref(a))
    assert ok == gda.GD_OK
    bad_scale = gda.SdpaDecodeArgs(0.0, 0, 0, 0)
    assert backend.call("gd_backend_sdpa_decode_positions", q.view(), k.view(), k.view(), pos.view(), out.view(),
                        C.byref(bad_scale)) == gda.INVALID_ARGUMENT
    bad_prefix = gda.SdpaDecodeArgs(0.125, 0, 17, 0)
    assert backend.call("gd_backend_sdpa_decode_positions", q.view(), k.view(), k.view(), pos.view(), out.view(),
                        C.byref(bad_prefix)) == gda.INVALID_ARGUMENT
    k3 = arena.alloc((2, 16, 3, 64), gda.F16)  # 4 query heads over 3 kv heads
    assert backend.call("gd_backend_sdpa_decode_positions", q.view(), k3.view(), k3.view(), pos.view(), out.view(),
                        C.byref(a)) == gda.INVALID_ARGUMENT
    at = gda.SdpaDecodeArgs(0.125, 0, 0, 16)  # Tq does not fit after position 16
    assert backend.call("gd_backend_sdpa_decode_at", q.view(), k.view(), k.view(), out.view(), C.byref(at)) == gda.INVALID_ARGUMENT


# ---- A11 sdpa_varlen ----------------------------------------------------------------------------

@pytest.mark.parametrize("H,Hkv,D,window,prefix", [(4, 4, 64, 0, 0), (4, 2, 128, 0, 0), (4, 4, 64, 5, 0), (2, 1, 32, 3, 4)])
def test_varlen_matches_oracle(backend, arena, oracle, H, Hkv, D, window, prefix):
    lens = np.array([70, 1, 0, 129, 33], np.int32)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    N = int(cu[-1])
    q, k, v = oracle.normal_f16((N, H, D), 700), oracle.normal_f16((N, Hkv, D), 701), oracle.normal_f16((N, Hkv, D), 702)
    out = arena.from_numpy(np.zeros(q.shape, np.float16))
    backend.sdpa_varlen(arena.from_numpy(q), arena.from_numpy(k), arena.from_numpy(v), arena.from_numpy(cu), out,
                        0.15, True, window, prefix, 256)
    _close(out.read(), oracle.sdpa_varlen(q, k, v, cu, 0.15, True, window, prefix, 256))


@pytest.mark.parametrize("H,Hkv,D,causal,window,prefix", [
    (4, 4, 64, True, 0, 0), (4, 2, 128, True, 0, 0), (2, 2, 128, True, 100, 0), (4, 1, 64, True, 70, 0),
    (2, 1, 128, True, 40, 150), (2, 2, 64, True, 0, 200), (2, 2, 64, False, 0, 0), (2, 1, 128, False, 90, 0)])
def test_varlen_many_blocks_matches_oracle(backend, arena, oracle, H, Hkv, D, causal, window, prefix):
    """Segments longer than the 128-row query block and the 64-key block of the matrix-core kernel: block
    edges, windows and prefixes that cross them, a segment that ends exactly on a block edge."""
    lens = np.array([300, 128, 1, 577, 64, 65], np.int32)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    N = int(cu[-1])
    q, k, v = oracle.normal_f16((N, H, D), 720), oracle.normal_f16((N, Hkv, D), 721), oracle.normal_f16((N, Hkv, D), 722)
    out = arena.from_numpy(np.zeros(q.shape, np.float16))
    scale = float(1.0 / np.sqrt(D))
    backend.sdpa_varlen(arena.from_numpy(q), arena.from_numpy(k), arena.from_numpy(v), arena.from_numpy(cu), out,
                        scale, causal, window, prefix, 0)
    _close(out.read(), oracle.sdpa_varlen(q, k, v, cu, scale, causal, window, prefix, 0))


@pytest.mark.parametrize("H,Hkv,D,causal,window,prefix", [(4, 2, 64, True, 0, 0), (2, 2, 128, True, 9, 3), (3, 1, 20, False, 0, 0),
                                                          (2, 1, 32, True, 40, 0)])
def test_varlen_f32_tensors(backend, arena, oracle, H, Hkv, D, causal, window, prefix):
    """F32 q/k/v/out (the reference accepts F16 and F32: src/ops/sdpa_varlen/core_sdpa_varlen.c:12-122).  Two checks:
    inputs that are exactly representable in F16 against the oracle (which then computes the same problem), and
    arbitrary F32 inputs against a float64 softmax over the visible set, the in-test model of the reference
    (tests/test_sdpa_varlen.c:158-230); bar 1e-5 relative + 2e-6 absolute, F32 accumulation."""
    lens = np.array([70, 1, 0, 131, 33], np.int32)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    N = int(cu[-1])
    qh, kh, vh = oracle.normal_f16((N, H, D), 760), oracle.normal_f16((N, Hkv, D), 761), oracle.normal_f16((N, Hkv, D), 762)
    tcu = arena.from_numpy(cu)
    out = arena.from_numpy(np.full(qh.shape, 3.0, np.float32))
    backend.sdpa_varlen(arena.from_numpy(qh.astype(np.float32)), arena.from_numpy(kh.astype(np.float32)),
                        arena.from_numpy(vh.astype(np.float32)), tcu, out, 0.15, causal, window, prefix, 0)
    _close(out.read(), oracle.sdpa_varlen(qh, kh, vh, cu, 0.15, causal, window, prefix, 0), 2e-5, 4e-6)
    rng = np.random.default_rng(763)
    q, k, v = (rng.standard_normal(sh).astype(np.float32) for sh in ((N, H, D), (N, Hkv, D), (N, Hkv, D)))
    out = arena.from_numpy(np.full(q.shape, 3.0, np.float32))
    backend.sdpa_varlen(arena.from_numpy(q), arena.from_numpy(k), arena.from_numpy(v), tcu, out, 0.15, causal, window, prefix, 0)
    got = out.read()
    want = np.zeros(q.shape, np.float64)
    for b in range(len(lens)):
        s0, T = int(cu[b]), int(lens[b])
        i, j = np.arange(T)[:, None], np.arange(T)[None, :]
        vis = np.ones((T, T), bool)   # the mask of tests/test_sdpa_varlen.c:122-148 of the reference, as array logic
        if causal:
            vis &= np.where(i < prefix, j < prefix, j <= i) if prefix > 0 else (j <= i)
        if window > 0:
            vis &= ~((i >= prefix) & (j >= prefix) & (i - j >= window)) if prefix > 0 else (i - j < window)
        for h in range(H):
            sc = q[s0:s0 + T, h].astype(np.float64) @ k[s0:s0 + T, h // (H // Hkv)].astype(np.float64).T * 0.15
            sc = np.where(vis, sc, -np.inf)
            w = np.exp(sc - sc.max(axis=1, keepdims=True)) if T else sc
            want[s0:s0 + T, h] = (w / w.sum(axis=1, keepdims=True)) @ v[s0:s0 + T, h // (H // Hkv)].astype(np.float64)
    _close(got, want, 2e-5, 4e-6)


def test_varlen_many_segments(backend, arena, oracle):
    """150 segments of 0..200 tokens (empty ones among them, some longer than a 128-row query block): a workgroup
    finds its segment by a search over runs of 64 segments, so the segment index crosses two run boundaries."""
    lens = oracle.uniform_i32(150, 741, 0, 201)
    lens[[0, 63, 64, 127, 128, 149]] = [0, 130, 0, 129, 200, 1]
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    N = int(cu[-1])
    q, k, v = (oracle.normal_f16((N, 2, 64), sd) for sd in (742, 743, 744))
    out = arena.from_numpy(np.full(q.shape, 5.0, np.float16))
    backend.sdpa_varlen(arena.from_numpy(q), arena.from_numpy(k), arena.from_numpy(v), arena.from_numpy(cu), out,
                        0.125, True, 0, 0, 0)
    _close(out.read(), oracle.sdpa_varlen(q, k, v, cu, 0.125, True, 0, 0, 0))


def test_varlen_ignores_values_of_the_next_segment(backend, arena, oracle):
    """Keys past a segment's end are never used, even if the neighbouring segment holds infinities."""
    cu = np.array([0, 70, 140], np.int32)
    q, k, v = (oracle.normal_f16((140, 2, 64), s) for s in (730, 731, 732))
    v[70:] = np.inf
    k[70:] = np.nan
    out = arena.from_numpy(np.zeros(q.shape, np.float16))
    backend.sdpa_varlen(arena.from_numpy(q), arena.from_numpy(k), arena.from_numpy(v), arena.from_numpy(cu), out,
                        0.125, False, 0, 0, 0)
    got = out.read()
    assert np.all(np.isfinite(got[:70]))
    kk, vv = k.copy(), v.copy()
    kk[70:], vv[70:] = 0, 0
    _close(got[:70], oracle.sdpa_varlen(q, kk, vv, cu, 0.125, False, 0, 0, 0)[:70])


@pytest.mark.parametrize("H,Hkv,D,causal,window,prefix", [
    (4, 4, 64, True, 0, 0), (4, 2, 128, True, 0, 0), (2, 2, 128, True, 100, 0), (2, 1, 128, True, 40, 150),
    (2, 2, 64, False, 0, 0)])
def test_varlen_reads_keys_and_values_from_the_caches(backend, arena, oracle, gda, H, Hkv, D, causal, window, prefix):
    """gd_backend_sdpa_varlen_cached (token t of segment b in row t of cache b) against gd_backend_sdpa_varlen on packed
    rows holding the same keys and values: the same kernel on the same numbers, so bit for bit, and against the oracle.
    Cache rows behind a segment's length hold NaN keys and infinite values and must not leak; a segment that fills
    its cache to the last row; an empty segment; a segment longer than the cache leaves its rows of out untouched."""
    lens = np.array([300, 128, 0, 577, 64, 65, 1], np.int32)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    B, N, Tmax = len(lens), int(cu[-1]), 577
    q, k, v = oracle.normal_f16((N, H, D), 770), oracle.normal_f16((N, Hkv, D), 771), oracle.normal_f16((N, Hkv, D), 772)
    kc = np.full((B, Tmax, Hkv, D), np.nan, np.float16)
    vc = np.full((B, Tmax, Hkv, D), np.inf, np.float16)
    for b in range(B):
        kc[b, :lens[b]], vc[b, :lens[b]] = k[cu[b]:cu[b + 1]], v[cu[b]:cu[b + 1]]
    scale = float(1.0 / np.sqrt(D))
    tq, tcu = arena.from_numpy(q), arena.from_numpy(cu)
    packed = arena.from_numpy(np.zeros(q.shape, np.float16))
    backend.sdpa_varlen(tq, arena.from_numpy(k), arena.from_numpy(v), tcu, packed, scale, causal, window, prefix, 0)
    cached = arena.from_numpy(np.zeros(q.shape, np.float16))
    backend.sdpa_varlen_cached(tq, arena.from_numpy(kc), arena.from_numpy(vc), tcu, cached, scale, causal, window, prefix, 0)
    got = cached.read()
    assert np.array_equal(_bits(got), _bits(packed.read()))
    _close(got, oracle.sdpa_varlen(q, k, v, cu, scale, causal, window, prefix, 0))
    # a cache of 400 rows cannot hold the segment of 577: its rows stay as they were, all others are computed
    short = arena.from_numpy(np.full(q.shape, 5.0, np.float16))
    backend.sdpa_varlen_cached(tq, arena.from_numpy(np.ascontiguousarray(kc[:, :400])),
                               arena.from_numpy(np.ascontiguousarray(vc[:, :400])), tcu, short, scale, causal, window, prefix, 0)
    got_short = short.read()
    assert np.all(got_short[cu[3]:cu[4]] == 5.0)
    keep = np.r_[0:cu[3], cu[4]:N]
    assert np.array_equal(_bits(got_short[keep]), _bits(got[keep]))
    # F32 tensors, other head sizes and a batch that is not the number of segments are refused, not mis-run
    a = gda.SdpaVarlenArgs(scale, 1, 0, 0, 0, 0)
    k5 = arena.alloc((B + 1, 8, Hkv, D), gda.F16)
    assert backend.call("gd_backend_sdpa_varlen_cached", tq.view(), k5.view(), k5.view(), tcu.view(), cached.view(),
                        C.byref(a)) == gda.INVALID_ARGUMENT
    k32 = arena.alloc((B, 8, Hkv, D), gda.F32)
    assert backend.call("gd_backend_sdpa_varlen_cached", tq.view(), k32.view(), k32.view(), tcu.view(), cached.view(),
                        C.byref(a)) == gda.UNSUPPORTED


def test_varlen_max_seqlen_truncates(backend, arena, oracle):
    cu = np.array([0, 50, 60], np.int32)
    q, k, v = (oracle.normal_f16((60, 2, 64), s) for s in (710, 711, 712))
    out = arena.from_numpy(np.full(q.shape, 3.0, np.float16))
    backend.sdpa_varlen(arena.from_numpy(q), arena.from_numpy(k), arena.from_numpy(v), arena.from_numpy(cu), out,
                        0.125, True, 0, 0, 32)
    got = out.read()
    _close(got, oracle.sdpa_varlen(q, k, v, cu, 0.125, True, 0, 0, 32))
    assert np.all(got[32:50] == 0)


# ---- A3 rms_norm ---------------------------------------------------------------------------------------

@pytest.mark.parametrize("rows,cols", [(64, 512), (16, 2048), (3, 100), (1, 8200), (5, 7)])
def test_rms_norm_f16(backend, arena, oracle, rows, cols):
    x = oracle.normal_f16((rows, cols), 800 + cols, 1.5)
    w = (1.0 + 0.1 * oracle.normal_f16((cols,), 801).astype(np.float32)).astype(np.float16)
    out = arena.alloc((rows, cols), 1)
    backend.rms_norm_forward(arena.from_numpy(x), arena.from_numpy(w), out, 1e-5)
    _close(out.read(), oracle.rms_norm(x, w, 1e-5))


def test_rms_norm_f32_reference_case(backend, arena, oracle, gda):
    c = _golden("reference_test_cases.json")["rms_norm_f32_2x4"]
    x = np.array(c["x"], np.float32).reshape(2, 4)
    w = np.array(c["w"], np.float32)
    out = arena.alloc((2, 4), gda.F32)
    backend.rms_norm_forward(arena.from_numpy(x), arena.from_numpy(w), out, c["eps"])
    assert np.abs(out.read() - oracle.rms_norm(x, w, c["eps"])).max() < c["tol_abs"]
    a = gda.RmsNormArgs(rows=2, cols=4, eps=0.0)
    assert backend.call("gd_backend_rms_norm_forward", out.view(), arena.from_numpy(w).view(), out.view(),
                        C.byref(a)) == gda.INVALID_ARGUMENT


# ---- A4 qkv_split_rope -------------------------------------------------------------------------------------

@pytest.mark.parametrize("N,H,D,interleaved", [(64, 8, 64, False), (16, 16, 128, False), (5, 3, 24, False),
                                               (7, 2, 64, True), (4, 2, 6, True)])
def test_qkv_split_rope(backend, arena, oracle, N, H, D, interleaved):
    qkv = oracle.normal_f16((N, 3 * H * D), 900 + D)
    pos = oracle.uniform_i32(N, 901, 0, 4095)
    pos[0] = 0
    q, k, v = (arena.alloc((N, H, D), 1) for _ in range(3))
    backend.qkv_split_rope_forward(arena.from_numpy(qkv), arena.from_numpy(pos), q, k, v, H, D, 10000.0, interleaved)
    wq, wk, wv = oracle.qkv_split_rope(qkv, pos, H, D, 10000.0, interleaved)
    assert np.array_equal(_bits(v.read()), _bits(wv))  # v and the index map: bit-exact
    _close(q.read(), wq)
    _close(k.read(), wk)
    # position 0 is the identity, bit for bit
    src = qkv.reshape(N, 3, H, D)
    assert np.array_equal(_bits(q.read()[0]), _bits(src[0, 0])) and np.array_equal(_bits(k.read()[0]), _bits(src[0, 1]))


def test_qkv_split_rope_rejects_partial_rotation(backend, arena, gda):
    qkv = arena.alloc((2, 3 * 2 * 8), gda.F16)
    pos = arena.alloc((2,), gda.I32)
    o = arena.alloc((2, 2, 8), gda.F16)
    a = gda.RopeArgs(10000.0, 4, 0)  # n_dims != head_dim
    assert backend.call("gd_backend_qkv_split_rope_forward", qkv.view(), pos.view(), o.view(), o.view(), o.view(),
                        2, 8, C.byref(a)) == gda.INVALID_ARGUMENT


# ---- A5/A6/A7 projections ------------------------------------------------------------------------------------

@pytest.mark.parametrize("M,K,N", [(64, 512, 1536), (1, 512, 2048), (16, 2048, 96), (33, 136, 50), (64, 1536, 512),
                                   (130, 64, 48), (3, 20, 7)])
def test_linear_nt_and_bias_roundings(backend, arena, oracle, M, K, N):
    x = oracle.normal_f16((M, K), 1000 + K, 1.0)
    w = oracle.normal_f16((N, K), 1001 + N, 0.05)
    bias = oracle.normal_f16((N,), 1002, 0.5)
    tx, tw, tb = arena.from_numpy(x), arena.from_numpy(w), arena.from_numpy(bias)
    y = arena.alloc((M, N), 1)
    backend.matmul_nt(tx, tw, y)
    _close(y.read(), oracle.linear_nt(x, w))
    backend.linear_nt(tx, tw, tb, y)
    _close(y.read(), oracle.linear_nt(x, w, bias))


@pytest.mark.parametrize("M,K,N", [(64, 1536, 512), (16, 352, 2048), (1, 64, 40), (70, 24, 33), (2, 9, 5)])
def test_linear_kn_and_swiglu_fusion(backend, arena, oracle, M, K, N):
    x = oracle.normal_f16((M, K), 1100 + K, 1.0)
    w = oracle.normal_f16((K, N), 1101 + N, 0.05)
    bias = oracle.normal_f16((N,), 1102, 0.5)
    tx, tw, tb = arena.from_numpy(x), arena.from_numpy(w), arena.from_numpy(bias)
    y = arena.alloc((M, N), 1)
    backend.matmul(tx, tw, y)
    _close(y.read(), oracle.linear(x, w))
    backend.linear(tx, tw, tb, y)
    _close(y.read(), oracle.linear(x, w, bias))
    x12 = oracle.normal_f16((M, 2 * K), 1103, 1.0)
    backend.swiglu_split_linear(arena.from_numpy(x12), tw, tb, y)
    _close(y.read(), oracle.swiglu_split_linear(x12, w, bias))
    backend.swiglu_split_linear(arena.from_numpy(x12), tw, None, y)
    _close(y.read(), oracle.swiglu_split_linear(x12, w))


def test_linear_reference_fill_values_and_strided_rows(backend, arena, oracle):
    """Inputs of the reference's tests/test_linear.c (fill_values) and a row-strided x view."""
    c = _golden("reference_test_cases.json")["linear_f16"]
    M, K, N = 4, 16, 8
    x = oracle.fill_values(M * K, 0.01, -0.1).astype(np.float16).reshape(M, K)
    w = oracle.fill_values(K * N, 0.02, -0.3).astype(np.float16).reshape(K, N)
    b = oracle.fill_values(N, 0.05, -0.5).astype(np.float16)
    y = arena.alloc((M, N), 1)
    backend.linear(arena.from_numpy(x), arena.from_numpy(w), arena.from_numpy(b), y)
    want = x.astype(np.float64) @ w.astype(np.float64) + b.astype(np.float64)
    assert np.abs(y.read().astype(np.float64) - want).max() < c["tol_abs"]
    wide = oracle.normal_f16((M, 2 * K), 1200)
    tw = arena.from_numpy(wide)
    import ctypes
    xm = tw.matrix(rows=M, cols=K, row_elems=2 * K)  # left half of every row
    st = backend.call("gd_backend_matmul", ctypes.byref(xm), arena.from_numpy(w).matrix(), y.matrix())
    assert st == 0
    _close(y.read(), oracle.linear(wide[:, :K], w))


def test_linear_rejects_bad_arguments(backend, arena, gda):
    x = arena.alloc((4, 16), gda.F16)
    w = arena.alloc((16, 8), gda.F16)
    y = arena.alloc((4, 8), gda.F16)
    bad_w = arena.alloc((15, 8), gda.F16)
    f32 = arena.alloc((4, 16), gda.F32)
    assert backend.call("gd_backend_matmul", x.matrix(), bad_w.matrix(), y.matrix()) == gda.INVALID_ARGUMENT
    assert backend.call("gd_backend_matmul", f32.matrix(), w.matrix(), y.matrix()) == gda.UNSUPPORTED
    assert backend.call("gd_backend_matmul_nt", x.matrix(), w.matrix(), y.matrix()) == gda.INVALID_ARGUMENT


# ---- A8 add, swiglu_split, A9 embedding, A10 argmax, gather ----------------------------------------------------

def test_add_residual_bias_and_broadcast(backend, arena, oracle):
    a = oracle.normal_f16((64, 512), 1300, 30.0)
    b = oracle.normal_f16((64, 512), 1301, 0.3)
    out = arena.alloc((64, 512), 1)
    backend.add(arena.from_numpy(a), arena.from_numpy(b), out)
    assert np.array_equal(_bits(out.read()), _bits(a + b))
    bias = oracle.normal_f16((512,), 1302)
    backend.add(arena.from_numpy(a), arena.from_numpy(bias), out)
    assert np.array_equal(_bits(out.read()), _bits(a + bias))
    backend.add(arena.from_numpy(bias), arena.from_numpy(a), out)
    assert np.array_equal(_bits(out.read()), _bits(a + bias))
    x = oracle.normal_f16((3, 1, 5), 1303)
    y = oracle.normal_f16((4, 1), 1304)
    o = arena.alloc((3, 4, 5), 1)
    backend.add(arena.from_numpy(x), arena.from_numpy(y), o)
    assert np.array_equal(_bits(o.read()), _bits(x + y))
    odd = oracle.normal_f16((7, 3), 1305)
    o2 = arena.alloc((7, 3), 1)
    backend.add(arena.from_numpy(odd), arena.from_numpy(odd), o2)
    assert np.array_equal(_bits(o2.read()), _bits(odd + odd))


def test_add_rejects_incompatible_shapes(backend, arena, gda):
    x, y, o = arena.alloc((4, 6), gda.F16), arena.alloc((5,), gda.F16), arena.alloc((4, 6), gda.F16)
    assert backend.call("gd_backend_add", x.view(), y.view(), o.view()) == gda.INVALID_ARGUMENT


@pytest.mark.parametrize("rows,H", [(64, 1536), (3, 4), (2, 8), (5, 13)])
def test_swiglu_split(backend, arena, oracle, rows, H):
    x12 = oracle.normal_f16((rows, 2 * H), 1400 + H, 2.0)
    out = arena.alloc((rows, H), 1)
    backend.swiglu_split_forward(arena.from_numpy(x12), out)
    _close(out.read(), oracle.swiglu_split(x12))


def test_embedding_bit_exact_and_nan_rows(backend, arena, oracle, gda):
    table = oracle.normal_f16((2048, 512), 1500, 0.02)
    ids = oracle.uniform_i32(64, 1501, 0, 2047)
    ids[5], ids[9] = -1, 2048
    out = arena.alloc((64, 512), 1)
    backend.embedding_forward(arena.from_numpy(table), arena.from_numpy(ids), out)
    assert np.array_equal(_bits(out.read()), _bits(oracle.embedding(table, ids)))
    t32 = oracle.fill_normal(10 * 3, 1502, 1.0).reshape(10, 3)
    ids = np.array([9, 0, 11], np.int32)
    o32 = arena.alloc((3, 3), gda.F32)
    backend.embedding_forward(arena.from_numpy(t32), arena.from_numpy(ids), o32)
    got = o32.read()
    assert np.array_equal(got[:2], t32[[9, 0]]) and np.all(np.isnan(got[2]))


def test_argmax_rows(backend, arena, oracle, gda):
    logits = oracle.normal_f16((64, 2048), 1600, 3.0)
    logits[1, 100] = logits[1, 1900] = np.float16(60.0)  # tie -> lowest index
    logits[2, :] = np.nan
    logits[3, 7] = np.inf
    logits[4, :] = -np.inf
    logits[4, 2047] = np.float16(-5.0)
    ids, gap = arena.alloc((64,), gda.I32), arena.alloc((64,), gda.F32)
    backend.argmax_rows(arena.from_numpy(logits), ids, gap)
    want_ids, want_gap = oracle.argmax_rows(logits)
    assert np.array_equal(ids.read(), want_ids)
    assert np.array_equal(gap.read(), want_gap)
    wide = oracle.normal_f16((16, 32768), 1601, 3.0)
    ids2 = arena.alloc((16,), gda.I32)
    backend.argmax_rows(arena.from_numpy(wide), ids2)
    assert np.array_equal(ids2.read(), oracle.argmax_rows(wide)[0])


def test_gather_rows_and_position_increment(backend, arena, oracle, gda):
    src = oracle.normal_f16((100, 512), 1700)
    rows = np.array([99, 0, 42, 42, 100], np.int32)  # last one is out of range: row untouched
    out = arena.from_numpy(np.full((5, 512), 9.0, np.float16))
    backend.gather_rows(arena.from_numpy(src), arena.from_numpy(rows), out)
    got = out.read()
    assert np.array_equal(_bits(got[:4]), _bits(src[[99, 0, 42, 42]])) and np.all(got[4] == 9.0)
    p = arena.from_numpy(np.arange(64, dtype=np.int32))
    backend.add_scalar_i32(p, p, 1)
    assert np.array_equal(p.read(), np.arange(1, 65))


def test_rand_uniform_matches_the_counter_based_stream(backend, arena, oracle, gda):
    n = 100003
    want = oracle.rand_uniform_f32(n, 1234, -1.0, 1.0)
    f32 = arena.alloc((n,), gda.F32)
    backend.rand_uniform(f32, 1234, -1.0, 1.0)
    assert np.array_equal(_bits(f32.read()), _bits(want))
    f16 = arena.alloc((n,), gda.F16)
    backend.rand_uniform(f16, 1234, -1.0, 1.0)
    assert np.array_equal(_bits(f16.read()), _bits(want.astype(np.float16)))
    odd = arena.alloc((1000,), gda.F32)  # a span that is not a power of two: the multiply-add rounds once
    backend.rand_uniform(odd, 99, 0.25, 7.5)
    assert np.array_equal(_bits(odd.read()), _bits(oracle.rand_uniform_f32(1000, 99, 0.25, 7.5)))
    i32 = arena.alloc((8,), gda.I32)
    st = gda.lib().gd_backend_rand_uniform(backend.handle, i32.buffer.handle, i32.offset, i32.count, i32.dtype, 1, 0.0, 1.0)
    assert st == gda.UNSUPPORTED
    st = gda.lib().gd_backend_rand_uniform(backend.handle, f32.buffer.handle, f32.offset, f32.count, f32.dtype, 1, 2.0, 1.0)
    assert st == gda.INVALID_ARGUMENT


@pytest.mark.parametrize("dtype", [np.float16, np.int32, np.uint8])
def test_concat_to_full_places_slices_bit_exact(backend, arena, gda, dtype):
    """np.concatenate is the reference: two slices along the middle axis, then along axis 0."""
    rng = np.random.default_rng(5)
    a = rng.integers(0, 200, (3, 2, 7)).astype(dtype)
    b = rng.integers(0, 200, (3, 5, 7)).astype(dtype)
    full = arena.from_numpy(np.zeros((3, 7, 7), dtype))
    backend.concat_to_full(arena.from_numpy(a), full, 1, 0)
    backend.concat_to_full(arena.from_numpy(b), full, 1, 2)
    assert np.array_equal(full.read(), np.concatenate([a, b], axis=1))
    rows = arena.from_numpy(np.zeros((6, 2, 7), dtype))
    backend.concat_to_full(arena.from_numpy(a), rows, 0, 3)
    got = rows.read()
    assert np.array_equal(got[3:], a) and not got[:3].any()
    bad = gda.ConcatArgs(a.size, 7, 2, 7, 6)  # slice would run past the end of the axis
    assert backend.call("gd_backend_concat_to_full", arena.from_numpy(a).view(), full.view(), C.byref(bad)) == gda.INVALID_ARGUMENT


# ---- fused operators (same rounding points as the separate ones) -----------------------------------------------

@pytest.mark.parametrize("M,K,N", [(64, 512, 1536), (16, 2048, 96), (5, 136, 50), (70, 512, 64)])
def test_fused_linear_rms_prologue_and_residual(backend, arena, oracle, M, K, N):
    x = oracle.normal_f16((M, K), 2000 + K, 1.3)
    nw = (1.0 + 0.1 * oracle.normal_f16((K,), 2001).astype(np.float32)).astype(np.float16)
    w = oracle.normal_f16((N, K), 2002 + N, 0.05)
    bias = oracle.normal_f16((N,), 2003, 0.5)
    res = oracle.normal_f16((M, N), 2004, 1.0)
    y = arena.alloc((M, N), 1)
    tx, tw, tb, tr, tn = (arena.from_numpy(a) for a in (x, w, bias, res, nw))
    backend.fused_linear(tx, tw, tb, None, tn, y, True, 2, 2, 1e-5)
    want = oracle.linear_nt(oracle.rms_norm(x, nw, 1e-5), w, bias)
    _close(y.read(), want)
    backend.fused_linear(tx, tw, tb, tr, None, y, True, 2, 0)
    want = oracle.add(res, oracle.linear_nt(x, w, bias))
    _close(y.read(), want, through=res)  # the sum may cancel: one rounding step is the residual's size
    backend.fused_linear(tx, tw, None, tr, tn, y, True, 0, 2, 1e-5)
    _close(y.read(), oracle.add(res, oracle.linear_nt(oracle.rms_norm(x, nw, 1e-5), w)), through=res)


@pytest.mark.parametrize("M,K,N,nk", [(64, 1536, 512, True), (64, 1536, 512, False), (16, 352, 2048, True), (3, 24, 33, False)])
def test_fused_linear_swiglu_prologue_both_layouts(backend, arena, oracle, M, K, N, nk):
    x12 = oracle.normal_f16((M, 2 * K), 2100 + K, 1.0)
    w_kn = oracle.normal_f16((K, N), 2101 + N, 0.05)
    bias = oracle.normal_f16((N,), 2102, 0.5)
    res = oracle.normal_f16((M, N), 2103, 1.0)
    w = np.ascontiguousarray(w_kn.T) if nk else w_kn
    y = arena.alloc((M, N), 1)
    backend.fused_linear(arena.from_numpy(x12), arena.from_numpy(w), arena.from_numpy(bias), arena.from_numpy(res), None, y,
                         nk, 1, 1)
    _close(y.read(), oracle.add(res, oracle.swiglu_split_linear(x12, w_kn, bias)))


# Many-row (prefill) projections: the LDS-tiled matrix-core kernel.  (300, 136, 200) runs the 128 x 128 tile
# with ragged edges in all three dimensions, (2100, 200, 8200) the 256 x 256 tile (9 x 33 tiles), ragged too;
# (640, 160, 384) and (2304, 160, 8192) are whole tiles with K a multiple of 32, which take the path that
# stages operands straight into LDS (5 K tiles: pipeline fill, two steady-state tiles, drain).
TILE_SHAPES = [(300, 136, 200), (128, 64, 128), (2100, 200, 8200), (640, 160, 384), (2304, 160, 8192), (256, 96, 256)]


@pytest.mark.parametrize("M,K,N", TILE_SHAPES)
@pytest.mark.parametrize("nk", [True, False])
def test_many_row_projection_plain_and_bias_modes(backend, arena, oracle, M, K, N, nk):
    x = oracle.normal_f16((M, K), 2300 + K, 1.0)
    w_kn = oracle.normal_f16((K, N), 2301 + N, 0.05)
    bias = oracle.normal_f16((N,), 2302, 0.5)
    res = oracle.normal_f16((M, N), 2303, 1.0)
    w = np.ascontiguousarray(w_kn.T) if nk else w_kn
    w_nk = np.ascontiguousarray(w_kn.T)
    tx, tw, tb, tr = (arena.from_numpy(a) for a in (x, w, bias, res))
    y = arena.alloc((M, N), 1)
    backend.fused_linear(tx, tw, None, None, None, y, nk, 0, 0)
    _close(y.read(), oracle.linear_nt(x, w_nk))
    backend.fused_linear(tx, tw, tb, None, None, y, nk, 1, 0)  # bias added in F32
    _close(y.read(), oracle.linear(x, w_kn, bias))
    backend.fused_linear(tx, tw, tb, tr, None, y, nk, 2, 0)  # bias added after the F16 rounding, then the residual
    inter = oracle.linear_nt(x, w_nk, bias)
    _close(y.read(), oracle.add(res, inter), through=inter)


@pytest.mark.parametrize("M,K,N", TILE_SHAPES)
@pytest.mark.parametrize("nk", [True, False])
def test_many_row_projection_prologues(backend, arena, oracle, M, K, N, nk):
    x12 = oracle.normal_f16((M, 2 * K), 2400 + K, 1.0)
    x = np.ascontiguousarray(x12[:, :K])
    nw = (1.0 + 0.1 * oracle.normal_f16((K,), 2401).astype(np.float32)).astype(np.float16)
    w_kn = oracle.normal_f16((K, N), 2402 + N, 0.05)
    bias = oracle.normal_f16((N,), 2403, 0.5)
    w = np.ascontiguousarray(w_kn.T) if nk else w_kn
    tw, tb = arena.from_numpy(w), arena.from_numpy(bias)
    y = arena.alloc((M, N), 1)
    backend.fused_linear(arena.from_numpy(x12), tw, tb, None, None, y, nk, 1, 1)
    _close(y.read(), oracle.swiglu_split_linear(x12, w_kn, bias))
    backend.fused_linear(arena.from_numpy(x), tw, tb, None, arena.from_numpy(nw), y, nk, 1, 2, 1e-5)
    _close(y.read(), oracle.linear(oracle.rms_norm(x, nw, 1e-5), w_kn, bias))


@pytest.mark.parametrize("K", [128, 192])
def test_many_row_projection_tail_in_192_row_tiles(backend, arena, oracle, K):
    """13,192 rows onto 2048 columns of an [N,K] weight: 52 x 8 tiles of 256 x 256 are 1.6 rounds on 256 compute units;
    the first round's 8,192 rows run in those tiles, the 5,000 rows behind them (640 tiles of 128 x 128 would need more
    than one round of them) in one launch of 27 x 8 tiles of 192 x 256, three row tiles per wavefront, the last row tile
    ragged.  Whole output against the oracle, plain, with bias, and with bias and residual."""
    M, N = 13192, 2048
    x = oracle.normal_f16((M, K), 2500 + K, 1.0)
    w = oracle.normal_f16((N, K), 2501, 0.05)
    bias = oracle.normal_f16((N,), 2502, 0.5)
    res = oracle.normal_f16((M, N), 2503, 1.0)
    tx, tw, tb, tr = (arena.from_numpy(a) for a in (x, w, bias, res))
    y = arena.alloc((M, N), 1)
    backend.fused_linear(tx, tw, None, None, None, y, True, 0, 0)
    _close(y.read(), oracle.linear_nt(x, w))
    backend.fused_linear(tx, tw, tb, tr, None, y, True, 2, 0)
    inter = oracle.linear_nt(x, w, bias)
    got = y.read()
    _close(got, oracle.add(res, inter), through=inter)
    # the 192-row launch starts at row 13192 - 27 * 192 = 8008: rows 8008..8191 are rows of the first launch computed
    # once more.  The same rows from a call over the first 8,192 rows alone (whole 256 x 256 tiles only): same bits
    y_head = arena.alloc((8192, N), 1)
    backend.fused_linear(tx.rows(0, 8192), tw, tb, tr.rows(0, 8192), None, y_head, True, 2, 0)
    assert np.array_equal(_bits(y_head.read()), _bits(got[:8192]))


def test_many_row_projection_full_size_sampled(backend, oracle):
    """The packed-prefill projections of BASELINE config 4 at full size (30,229 rows): the qkv projection ([N,K]
    weight, bias added after the F16 rounding) and the down projection ([K,N] weight, F32 bias, residual), operands
    filled on the device, sampled rows (first, last, both sides of every kind of tile edge) against float64; and the
    attention projection with its residual on an [N,K] weight, whose 5,653 rows behind the last whole round of 256 x 256
    tiles go to one launch of 192 x 256 tiles (rows 24,576 on; tile edges every 192 rows, the last tile ragged)."""
    M = 30229
    big = backend.buffer(900 << 20)
    try:
        for (K, N, nk) in ((2048, 6144, True), (5632, 2048, False), (2048, 2048, True)):
            big.reset()
            x, w = big.alloc((M, K), 1), big.alloc((N, K) if nk else (K, N), 1)
            backend.rand_uniform(x, 9101 + K, -1.0, 1.0)
            backend.rand_uniform(w, 9102 + K, -0.05, 0.05)
            bias = oracle.normal_f16((N,), 9103, 0.5)
            res = big.alloc((M, N), 1)
            backend.rand_uniform(res, 9104, -1.0, 1.0)
            y = big.alloc((M, N), 1)
            with_res = not nk or N == 2048
            backend.fused_linear(x, w, big.from_numpy(bias), res if with_res else None, None, y, nk, 2 if nk else 1, 0)
            wf = w.read().astype(np.float64)
            wf = wf.T if nk else wf
            for r in (0, 1, 255, 256, 4095, 4096, 17000, 24575, 24576, 24767, 24768, 30143, 30144, 30207, 30208, 30228):
                xr = x.rows(r, 1).read()[0].astype(np.float64)
                t = xr @ wf
                if nk:
                    want = (t.astype(np.float16).astype(np.float32) + bias.astype(np.float32)).astype(np.float16)
                    if with_res:
                        want = (res.rows(r, 1).read()[0].astype(np.float32) + want.astype(np.float32)).astype(np.float16)
                else:
                    u = (t + bias.astype(np.float64)).astype(np.float16)
                    want = (res.rows(r, 1).read()[0].astype(np.float32) + u.astype(np.float32)).astype(np.float16)
                got = y.rows(r, 1).read()[0].astype(np.float32)
                scale_ = np.abs(t) + np.abs(bias.astype(np.float64)) + 1.0
                assert np.all(np.abs(got - want.astype(np.float32)) <= 1e-3 + 2e-3 * scale_), (K, N, r)
    finally:
        backend.free(big)


def test_varlen_full_size_sampled(backend, oracle):
    """The packed causal prefill attention of BASELINE config 4 at full size: 32 sequences of 64..2048 tokens, 16
    heads of 128; sampled query rows (first and last of a sequence, both sides of 64-key block edges and of
    128-row workgroup edges) against a float64 softmax over the visible keys."""
    H, D = 16, 128
    lens = oracle.uniform_i32(32, 9201, 64, 2048)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    n = int(cu[-1])
    big = backend.buffer(640 << 20)
    try:
        q, k, v, out = (big.alloc((n, H, D), 1) for _ in range(4))
        for t, seed in ((q, 9202), (k, 9203), (v, 9204)):
            backend.rand_uniform(t, seed, -1.0, 1.0)
        scale = 1.0 / np.sqrt(D)
        backend.sdpa_varlen(q, k, v, big.from_numpy(cu), out, scale)
        for s in (0, 5, 17, 31):
            base, L = int(cu[s]), int(lens[s])
            ks = k.rows(base, L).read().astype(np.float64)
            vs = v.rows(base, L).read().astype(np.float64)
            for i in sorted({0, 1, 63, 64, 127, 128, L // 2, L - 2, L - 1}):
                if i >= L:
                    continue
                qi = q.rows(base + i, 1).read()[0].astype(np.float64)  # [H, D]
                sc = np.einsum("hd,nhd->hn", qi, ks[:i + 1]) * scale
                wgt = np.exp(sc - sc.max(axis=1, keepdims=True))
                want = np.einsum("hn,nhd->hd", wgt / wgt.sum(axis=1, keepdims=True), vs[:i + 1])
                got = out.rows(base + i, 1).read()[0].astype(np.float32)
                assert np.all(np.abs(got - want) <= 1e-3 + 2e-3 * np.abs(want)), (s, i)
    finally:
        backend.free(big)


def test_many_row_projection_row_pitches_and_unaligned_output(backend, arena, oracle, gda):
    """Row-strided x / y views (slices of wider matrices) and an output whose rows are not 16-byte aligned."""
    M, K, N = 200, 96, 136
    xw = oracle.normal_f16((M, K + 40), 2500)
    w = oracle.normal_f16((N, K), 2501, 0.05)
    tx = arena.from_numpy(xw)
    ty = arena.from_numpy(np.full((M, N + 3), 7.0, np.float16))
    xv = gda.MatrixView(tx.buffer.handle, tx.offset, M, K, (K + 40) * 2, gda.F16)
    yv = gda.MatrixView(ty.buffer.handle, ty.offset + 2, M, N, (N + 3) * 2, gda.F16)
    tw = arena.from_numpy(w)
    assert backend.call("gd_backend_matmul_nt", C.byref(xv), tw.matrix(), C.byref(yv)) == 0
    backend.flush()
    got = ty.read()
    _close(got[:, 1:N + 1], oracle.linear_nt(np.ascontiguousarray(xw[:, :K]), w))
    assert np.all(got[:, 0] == 7.0) and np.all(got[:, N + 1:] == 7.0)


@pytest.mark.parametrize("M,K,H", [(64, 512, 1536), (16, 2048, 5632), (5, 136, 24), (33, 64, 40),
                                   (1024, 512, 1536), (512, 256, 384), (300, 200, 200), (257, 128, 136),
                                   (2304, 160, 4096), (2100, 96, 4100)])
def test_fused_linear_swiglu_epilogue(backend, arena, oracle, gda, M, K, H):
    """rms_norm -> up/gate projection (+ F16 bias) -> swiglu_split in one launch equals the three separate operators."""
    x = oracle.normal_f16((M, K), 2600 + K, 1.3)
    nw = (1.0 + 0.1 * oracle.normal_f16((K,), 2601).astype(np.float32)).astype(np.float16)
    w = oracle.normal_f16((2 * H, K), 2602 + H, 0.05)
    bias = oracle.normal_f16((2 * H,), 2603, 0.5)
    y = arena.alloc((M, H), 1)
    tx, tw, tb, tn = (arena.from_numpy(a) for a in (x, w, bias, nw))
    backend.fused_linear(tx, tw, tb, None, tn, y, True, 2, 2, 1e-5, epilogue=1)
    def scale(u, b):
        # one rounding step of the value (before its bias was added: the sum may cancel) times the gate, or of
        # the gate times the value
        u, b = u.astype(np.float64), b.astype(np.float64)
        return (np.abs(u[:, :H]) + np.abs(b[:H])) * (1.0 + np.abs(u[:, H:]) + np.abs(b[H:]))

    u = oracle.linear_nt(oracle.rms_norm(x, nw, 1e-5), w, bias)
    _close(y.read(), oracle.swiglu_split(u), through=scale(u, bias))
    backend.fused_linear(tx, tw, None, None, None, y, True, 0, 0, 0.0, epilogue=1)
    u = oracle.linear_nt(x, w)
    _close(y.read(), oracle.swiglu_split(u), through=scale(u, np.zeros_like(bias)))
    a = gda.FusedLinearArgs(0, 0, 0, 0.0, 1)  # the gated epilogue needs the [N,K] weight layout
    wk = arena.alloc((K, 2 * H), gda.F16)
    assert backend.call("gd_backend_fused_linear", tx.matrix(), wk.matrix(), None, None, None, y.matrix(), C.byref(a)) == gda.UNSUPPORTED


def test_few_row_projection_over_weights_on_both_sides_of_a_2_gib_boundary(backend, oracle, gda):
    """The kernels that stream large weight matrices through LDS take the matrix's address as a scalar base plus
    32-bit lane offsets.  The same matrix placed twice, 2 GiB apart: one of the two copies has an address whose low
    word has its top bit set (a sign extension of that word once sent the loads of such a copy to invalid
    addresses).  rms_norm + up/gate + swiglu (the persistent form) and projection + residual (one tile per
    workgroup), both copies against the oracle and against each other to the bit."""
    M, K, H = 16, 2048, 1024
    big = backend.buffer((2 << 30) + (96 << 20))
    try:
        x = oracle.normal_f16((M, K), 3100, 1.3)
        nw = (1.0 + 0.1 * oracle.normal_f16((K,), 3101).astype(np.float32)).astype(np.float16)
        w = oracle.normal_f16((2 * H, K), 3102, 0.05)
        bias = oracle.normal_f16((2 * H,), 3103, 0.5)
        res = oracle.normal_f16((M, 2 * H), 3104, 1.0)
        tx, tn, tb, tr = (big.from_numpy(a) for a in (x, nw, bias, res))
        y1, y2 = big.alloc((M, H), gda.F16), big.alloc((M, 2 * H), gda.F16)
        first = big.alloc((2 * H, K), gda.F16).write(w)
        second = gda.Tensor(big, first.offset + (2 << 30), (2 * H, K), gda.F16).write(w)
        backend.set_tunable("linear_wide", 1)
        got = []
        for tw in (first, second):
            backend.fill(y1, 0x7e00)
            backend.fill(y2, 0x7e00)
            backend.fused_linear(tx, tw, tb, None, tn, y1, True, 2, 2, 1e-5, epilogue=1)
            backend.fused_linear(tx, tw, tb, tr, None, y2, True, 2, 0)
            got.append((y1.read(), y2.read()))
        assert np.array_equal(_bits(got[0][0]), _bits(got[1][0])) and np.array_equal(_bits(got[0][1]), _bits(got[1][1]))
        u = oracle.linear_nt(oracle.rms_norm(x, nw, 1e-5), w, bias)
        through = (np.abs(u[:, :H].astype(np.float64)) + np.abs(bias[:H].astype(np.float64))) * \
                  (1.0 + np.abs(u[:, H:].astype(np.float64)) + np.abs(bias[H:].astype(np.float64)))
        _close(got[0][0], oracle.swiglu_split(u), through=through)
        _close(got[0][1], oracle.add(res, oracle.linear_nt(x, w, bias)), through=res)
    finally:
        backend.set_tunable("linear_wide", -1)
        backend.free(big)


@pytest.mark.parametrize("M,K,N", [(16, 2048, 2048), (16, 5632, 2048), (5, 1152, 1024), (1, 384, 264), (16, 128, 2048)])
def test_few_row_projection_onto_narrow_outputs(backend, arena, oracle, gda, M, K, N):
    """Up to 16 rows onto an output with fewer 16-column tiles than the chip has compute units: 8 columns per workgroup
    (K in pieces of 128 dealt to the eight wavefronts: 16, 44, 9, 3 and 1 pieces here, so wavefronts with one piece more
    than others and wavefronts with none).  All bias modes, with and without the residual, against the oracle; the
    16-column form (tunable linear_tiles = 1) must meet the same bar."""
    x = oracle.normal_f16((M, K), 3300 + K, 1.0)
    w = oracle.normal_f16((N, K), 3301 + N, 0.05)
    bias = oracle.normal_f16((N,), 3302, 0.5)
    res = oracle.normal_f16((M, N), 3303, 1.0)
    y = arena.alloc((M, N), gda.F16)
    tx, tw, tb, tr = (arena.from_numpy(a) for a in (x, w, bias, res))
    try:
        backend.set_tunable("linear_wide", 1)
        for tiles in (0, 1):
            backend.set_tunable("linear_tiles", tiles)
            backend.fill(y, 0x7e00)
            backend.fused_linear(tx, tw, None, None, None, y, True, 0, 0)
            _close(y.read(), oracle.linear_nt(x, w))
            backend.fused_linear(tx, tw, tb, None, None, y, True, 1, 0)
            _close(y.read(), oracle.linear(x, np.ascontiguousarray(w.T), bias))
            backend.fused_linear(tx, tw, tb, tr, None, y, True, 2, 0)
            inter = oracle.linear_nt(x, w, bias)
            _close(y.read(), oracle.add(res, inter), through=inter)
    finally:
        backend.set_tunable("linear_wide", -1)
        backend.set_tunable("linear_tiles", 0)


@pytest.mark.parametrize("M,N,gated", [(16, 5632, True), (33, 8200, False), (64, 4096, True), (5, 32768, False)])
def test_few_row_projection_weight_stream_through_lds(backend, arena, oracle, gda, M, N, gated):
    """rms_norm + projection with K = 2048 and 64 columns per workgroup stages its weight stream through LDS (whole
    128-byte lines per weight row and load) instead of loading MFMA fragments straight into registers.  Both paths
    multiply in the same order: the same bits, and both within the bar of the oracle (also where the last workgroup's
    columns run past N)."""
    K = 2048
    x = oracle.normal_f16((M, K), 3000 + M, 1.3)
    nw = (1.0 + 0.1 * oracle.normal_f16((K,), 3001).astype(np.float32)).astype(np.float16)
    rows = 2 * N if gated else N
    w = oracle.normal_f16((rows, K), 3002 + N, 0.05)
    bias = oracle.normal_f16((rows,), 3003, 0.5)
    y = arena.alloc((M, N), gda.F16)
    tx, tw, tb, tn = (arena.from_numpy(a) for a in (x, w, bias, nw))
    got = {}
    try:
        for off in (0, 1):
            backend.set_tunable("linear_no_lds_stream", off)
            backend.fill(y, 0x7e00)
            backend.fused_linear(tx, tw, tb, None, tn, y, True, 2, 2, 1e-5, epilogue=1 if gated else 0)
            got[off] = y.read()
    finally:
        backend.set_tunable("linear_no_lds_stream", 0)
    assert np.array_equal(got[0].view(np.uint16), got[1].view(np.uint16))
    u = oracle.linear_nt(oracle.rms_norm(x, nw, 1e-5), w, bias)
    if gated:
        through = (np.abs(u[:, :N].astype(np.float64)) + np.abs(bias[:N].astype(np.float64))) * \
                  (1.0 + np.abs(u[:, N:].astype(np.float64)) + np.abs(bias[N:].astype(np.float64)))
        _close(got[0], oracle.swiglu_split(u), through=through)
    else:
        _close(got[0], u)


# (5600 gated and 12352 plain columns leave a last tile with 12 and 4 columns in use)
@pytest.mark.parametrize("kind,N,M", [("swiglu", 5632, 16), ("swiglu", 5632, 32), ("plain", 12288, 16), ("plain", 12288, 32),
                                      ("swiglu", 5600, 16), ("plain", 12352, 32)])
def test_few_row_projection_narrow_tiles_fill_every_compute_unit(backend, arena, oracle, gda, kind, N, M):
    """Outputs with fewer full column tiles than compute units (5632 gated columns: 176 tiles of 32) are dealt out in
    narrower tiles, one per compute unit (22 columns each), whose unused columns repeat the last weight row and are not
    stored.  Same bits as the full-width tiles (tunable linear_tiles = 4) and as the stream kernel; nothing is written
    outside the output."""
    K = 2048
    rows = 2 * N if kind == "swiglu" else N
    x = oracle.normal_f16((M, K), 5300 + M, 1.2)
    nw = (1.0 + 0.1 * oracle.normal_f16((K,), 5301).astype(np.float32)).astype(np.float16)
    w = oracle.normal_f16((rows, K), 5302, 0.05)
    bias = oracle.normal_f16((rows,), 5303, 0.4)
    tx, tw, tb, tn = (arena.from_numpy(a) for a in (x, w, bias, nw))
    got = {}
    try:
        for name, wide, tiles in (("narrow", 1, 0), ("full", 1, 4), ("stream", 0, 0)):
            backend.set_tunable("linear_wide", wide)
            backend.set_tunable("linear_tiles", tiles)
            backend.set_tunable("linear_waves", 0 if wide else 8)
            y = arena.alloc((M, N), gda.F16)
            behind = arena.alloc((8192,), gda.F16)  # whatever is written past the output lands here
            backend.fill(y, 0x7e00)
            backend.fill(behind, 0x7e00)
            backend.fused_linear(tx, tw, tb, None, tn, y, True, 2, 2, 1e-5, epilogue=1 if kind == "swiglu" else 0)
            got[name] = y.read()
            assert backend.linear_last_kernel() == ("wide" if wide else "stream")
            assert np.all(_bits(behind.read()) == 0x7e00), name
    finally:
        backend.set_tunable("linear_wide", -1)
        backend.set_tunable("linear_tiles", 0)
        backend.set_tunable("linear_waves", 0)
    assert not np.isnan(got["narrow"].astype(np.float32)).any()
    assert np.array_equal(_bits(got["narrow"]), _bits(got["full"]))
    assert np.array_equal(_bits(got["narrow"]), _bits(got["stream"]))
    u = oracle.linear_nt(oracle.rms_norm(x, nw, 1e-5), w, bias)
    if kind == "plain":
        _close(got["narrow"], u)
    else:
        through = (np.abs(u[:, :N].astype(np.float64)) + np.abs(bias[:N].astype(np.float64))) * \
                  (1.0 + np.abs(u[:, N:].astype(np.float64)) + np.abs(bias[N:].astype(np.float64)))
        _close(got["narrow"], oracle.swiglu_split(u), through=through)


@pytest.mark.parametrize("M", [16, 32])
def test_few_row_qkv_rope_narrow_tiles_straddle_heads(backend, arena, oracle, gda, M):
    """The 3072 rotation pairs of a 16-head, 128-wide qkv projection are 192 full tiles of 16 pairs; on 256 compute units
    they are dealt out 12 pairs to a tile, which then straddle heads (pair -> weight row computed per lane).  Same
    bits as the full tiles (tunable linear_tiles = 4) and as the stream kernel, q and both caches."""
    K, H, D, Tmax = 2048, 16, 128, 6
    N = 3 * H * D
    x = oracle.normal_f16((M, K), 5400 + M, 1.2)
    nw = (1.0 + 0.1 * oracle.normal_f16((K,), 5401).astype(np.float32)).astype(np.float16)
    w = oracle.normal_f16((N, K), 5402, 0.05)
    bias = oracle.normal_f16((N,), 5403, 0.4)
    tx, tw, tb, tn = (arena.from_numpy(a) for a in (x, w, bias, nw))
    pos = oracle.uniform_i32(M, 5404, 0, 3000)
    cpos = oracle.uniform_i32(M, 5405, 0, Tmax - 1)
    cpos[1] = -1
    tp, tc = arena.from_numpy(pos), arena.from_numpy(cpos)
    k0, v0 = oracle.normal_f16((M, Tmax, H, D), 5406), oracle.normal_f16((M, Tmax, H, D), 5407)
    got = {}
    try:
        for name, wide, tiles in (("narrow", 1, 0), ("full", 1, 4), ("stream", 0, 0)):
            backend.set_tunable("linear_wide", wide)
            backend.set_tunable("linear_tiles", tiles)
            backend.set_tunable("linear_waves", 0 if wide else 8)
            q, kc, vc = arena.alloc((M, H, D), gda.F16), arena.from_numpy(k0), arena.from_numpy(v0)
            backend.fill(q, 0x7e00)
            backend.fused_qkv_rope_append(tx, tw, tb, tn, tp, tc, q, kc, vc, H, D, 2, 2, 1e-5)
            got[name] = (q.read(), kc.read(), vc.read())
            assert backend.linear_last_kernel() == ("wide" if wide else "stream")
    finally:
        backend.set_tunable("linear_wide", -1)
        backend.set_tunable("linear_tiles", 0)
        backend.set_tunable("linear_waves", 0)
    for other in ("full", "stream"):
        for a, b in zip(got["narrow"], got[other]):
            assert np.array_equal(_bits(a), _bits(b)), other
    u = oracle.linear_nt(oracle.rms_norm(x, nw, 1e-5), w, bias)
    qo, ko, vo = oracle.qkv_split_rope(u, pos, H, D)
    _close(got["narrow"][0], qo, atol=4e-3)
    for b in range(M):
        if 0 <= cpos[b] < Tmax:
            _close(got["narrow"][1][b, cpos[b]], ko[b], atol=4e-3)
            _close(got["narrow"][2][b, cpos[b]], vo[b])
        else:
            assert np.array_equal(_bits(got["narrow"][1][b]), _bits(k0[b]))


# (33 rows or more with the rotation take the stream kernel by design)
@pytest.mark.parametrize("kind,K,tiles,M", [(kind, K, tiles, M) for kind in ("plain", "swiglu", "rope")
                                            for (K, tiles) in ((1024, 0), (1536, 0), (2048, 1), (2048, 0))
                                            for M in (5, 32, 64) if not (kind == "rope" and M == 64)])
def test_few_row_projection_wide_kernel_forms(backend, arena, oracle, gda, M, K, tiles, kind):
    """Every form of the kernels built around the weight stream through LDS that sits behind an rms_norm: one, two and
    four row tiles of 16 in a workgroup (5, 32, 64 rows), K = 1024 and 1536 (one tile per workgroup), K = 2048 in the
    one-tile form (tunable linear_tiles = 1) and in the persistent form, with the plain, gated and rotate-and-append
    epilogues.  Against the oracle, and bit for bit against the kernel that loads its fragments straight from global
    memory with the same eight-way split of K (same products, same order of sums)."""
    H, D, Tmax = 4, 64, 12
    N = {"plain": 4096 if (K, M) == (2048, 64) else 320, "swiglu": 160, "rope": 3 * H * D}[kind]
    rows = 2 * N if kind == "swiglu" else N
    x = oracle.normal_f16((M, K), 5200 + M + K, 1.2)
    nw = (1.0 + 0.1 * oracle.normal_f16((K,), 5201).astype(np.float32)).astype(np.float16)
    w = oracle.normal_f16((rows, K), 5202 + K, 0.05)
    bias = oracle.normal_f16((rows,), 5203, 0.4)
    tx, tw, tb, tn = (arena.from_numpy(a) for a in (x, w, bias, nw))
    pos = oracle.uniform_i32(M, 5204, 0, 3000)
    cpos = oracle.uniform_i32(M, 5205, 0, Tmax - 1)
    cpos[0] = -1
    tp, tc = arena.from_numpy(pos), arena.from_numpy(cpos)
    k0, v0 = oracle.normal_f16((M, Tmax, H, D), 5206), oracle.normal_f16((M, Tmax, H, D), 5207)

    def run(wide):
        backend.set_tunable("linear_wide", wide)
        backend.set_tunable("linear_tiles", tiles if wide else 0)
        backend.set_tunable("linear_waves", 0 if wide else 8)
        try:
            if kind == "rope":
                q, kc, vc = arena.alloc((M, H, D), gda.F16), arena.from_numpy(k0), arena.from_numpy(v0)
                backend.fill(q, 0x7e00)
                backend.fused_qkv_rope_append(tx, tw, tb, tn, tp, tc, q, kc, vc, H, D, 2, 2, 1e-5)
                out = (q.read(), kc.read(), vc.read())
            else:
                y = arena.alloc((M, N), gda.F16)
                backend.fill(y, 0x7e00)
                backend.fused_linear(tx, tw, tb, None, tn, y, True, 2, 2, 1e-5, epilogue=1 if kind == "swiglu" else 0)
                out = (y.read(),)
            return out, backend.linear_last_kernel()
        finally:
            backend.set_tunable("linear_wide", -1)
            backend.set_tunable("linear_tiles", 0)
            backend.set_tunable("linear_waves", 0)

    wide, family = run(1)
    assert family == "wide", family
    stream, family = run(0)
    assert family == "stream", family
    for a, b in zip(wide, stream):
        assert np.array_equal(_bits(a), _bits(b))
    u = oracle.linear_nt(oracle.rms_norm(x, nw, 1e-5), w, bias)
    if kind == "plain":
        _close(wide[0], u)
    elif kind == "swiglu":
        through = (np.abs(u[:, :N].astype(np.float64)) + np.abs(bias[:N].astype(np.float64))) * \
                  (1.0 + np.abs(u[:, N:].astype(np.float64)) + np.abs(bias[N:].astype(np.float64)))
        _close(wide[0], oracle.swiglu_split(u), through=through)
    else:
        qo, ko, vo = oracle.qkv_split_rope(u, pos, H, D)
        _close(wide[0], qo, atol=4e-3)
        for b in range(M):
            if 0 <= cpos[b] < Tmax:
                _close(wide[1][b, cpos[b]], ko[b], atol=4e-3)
                _close(wide[2][b, cpos[b]], vo[b])
        assert np.array_equal(_bits(wide[1][0]), _bits(k0[0])) and np.array_equal(_bits(wide[2][0]), _bits(v0[0]))


@pytest.mark.parametrize("B,H,D,K", [(64, 8, 64, 512), (16, 16, 128, 2048), (5, 3, 32, 72), (33, 2, 96, 64)])
def test_fused_qkv_rope_append_equals_separate_ops(backend, arena, oracle, gda, B, H, D, K):
    """rms_norm -> qkv projection (+F16 bias) -> rope -> cache append in one launch against the fused projection
    followed by the rope + append operator.  The projection result is rounded to F16 at the same point, so v is
    bit-identical; the rotation runs in a different kernel, where the compiler may contract the trigonometric range
    reduction differently: q and k agree to one F16 unit in the last place in all but a few elements per thousand."""
    Tmax = 24
    x = oracle.normal_f16((B, K), 2700 + K, 1.2)
    nw = (1.0 + 0.1 * oracle.normal_f16((K,), 2701).astype(np.float32)).astype(np.float16)
    w = oracle.normal_f16((3 * H * D, K), 2702 + D, 0.05)
    bias = oracle.normal_f16((3 * H * D,), 2703, 0.3)
    pos = oracle.uniform_i32(B, 2704, 0, 4000)
    cpos = oracle.uniform_i32(B, 2705, 0, Tmax - 1)
    cpos[0] = -1
    if B > 2:
        cpos[2] = Tmax
    k0, v0 = oracle.normal_f16((B, Tmax, H, D), 2706), oracle.normal_f16((B, Tmax, H, D), 2707)
    tx, tw, tb, tn = (arena.from_numpy(a) for a in (x, w, bias, nw))
    tp, tc = arena.from_numpy(pos), arena.from_numpy(cpos)
    q1, k1, v1 = arena.alloc((B, H, D), 1), arena.from_numpy(k0), arena.from_numpy(v0)
    backend.fused_qkv_rope_append(tx, tw, tb, tn, tp, tc, q1, k1, v1, H, D, 2, 2, 1e-5)
    qkv = arena.alloc((B, 3 * H * D), 1)
    q2, k2, v2 = arena.alloc((B, H, D), 1), arena.from_numpy(k0), arena.from_numpy(v0)
    backend.fused_linear(tx, tw, tb, None, tn, qkv, True, 2, 2, 1e-5)
    backend.qkv_rope_append(qkv, tp, tc, q2, k2, v2, H, D)
    def one_ulp(a, b):
        a32, b32 = a.astype(np.float32), b.astype(np.float32)
        ulp = np.spacing(np.maximum(np.abs(a), np.abs(b)).astype(np.float16)).astype(np.float32)
        assert np.all(np.abs(a32 - b32) <= ulp)
        assert np.count_nonzero(_bits(a) != _bits(b)) <= max(2, a.size // 500)

    one_ulp(q1.read(), q2.read())
    one_ulp(k1.read(), k2.read())
    assert np.array_equal(_bits(v1.read()), _bits(v2.read()))
    # and against the oracle chain, to tolerance
    u = oracle.linear_nt(oracle.rms_norm(x, nw, 1e-5), w, bias)
    qo, ko, vo = oracle.qkv_split_rope(u, pos, H, D)
    _close(q1.read(), qo, atol=4e-3)
    got_k = k1.read()
    for b in range(B):
        if 0 <= cpos[b] < Tmax:
            _close(got_k[b, cpos[b]], ko[b], atol=4e-3)
    # without norm and bias
    backend.fused_qkv_rope_append(tx, tw, None, None, tp, tc, q1, k1, v1, H, D, 0, 0)
    backend.fused_linear(tx, tw, None, None, None, qkv, True, 0, 0)
    backend.qkv_rope_append(qkv, tp, tc, q2, k2, v2, H, D)
    one_ulp(q1.read(), q2.read())
    one_ulp(k1.read(), k2.read())


def test_fused_linear_rejects_bad_arguments(backend, arena, gda):
    x, w, y = arena.alloc((4, 16), gda.F16), arena.alloc((8, 16), gda.F16), arena.alloc((4, 8), gda.F16)
    b = arena.alloc((8,), gda.F16)
    a = gda.FusedLinearArgs(1, 0, 2, 1e-5)  # rms prologue without a norm weight
    assert backend.call("gd_backend_fused_linear", x.matrix(), w.matrix(), None, None, None, y.matrix(), C.byref(a)) == gda.INVALID_ARGUMENT
    a = gda.FusedLinearArgs(1, 1, 0, 0.0)  # bias mode without a bias
    assert backend.call("gd_backend_fused_linear", x.matrix(), w.matrix(), None, None, None, y.matrix(), C.byref(a)) == gda.INVALID_ARGUMENT
    a = gda.FusedLinearArgs(1, 0, 0, 0.0)  # bias without a bias mode
    assert backend.call("gd_backend_fused_linear", x.matrix(), w.matrix(), b.vector(), None, None, y.matrix(), C.byref(a)) == gda.INVALID_ARGUMENT


@pytest.mark.parametrize("B,H,D", [(64, 8, 64), (16, 16, 128), (3, 2, 32)])
def test_qkv_rope_append_equals_separate_ops(backend, arena, oracle, B, H, D):
    Tmax = 40
    qkv = oracle.normal_f16((B, 3 * H * D), 2200 + D)
    pos = oracle.uniform_i32(B, 2201, 0, Tmax - 1)
    cpos = pos.copy()
    cpos[0] = -1
    if B > 2:
        cpos[2] = Tmax
    k0, v0 = oracle.normal_f16((B, Tmax, H, D), 2202), oracle.normal_f16((B, Tmax, H, D), 2203)
    q = arena.alloc((B, H, D), 1)
    kc, vc = arena.from_numpy(k0), arena.from_numpy(v0)
    backend.qkv_rope_append(arena.from_numpy(qkv), arena.from_numpy(pos), arena.from_numpy(cpos), q, kc, vc, H, D)
    # same arithmetic as the separate device operators: bit-identical results
    q2, k2, v2 = (arena.alloc((B, H, D), 1) for _ in range(3))
    backend.qkv_split_rope_forward(arena.from_numpy(qkv), arena.from_numpy(pos), q2, k2, v2, H, D)
    kc2, vc2 = arena.from_numpy(k0), arena.from_numpy(v0)
    backend.kv_cache_append_positions(kc2, vc2, arena.from_numpy(cpos), k2.reshape(B, 1, H, D), v2.reshape(B, 1, H, D))
    assert np.array_equal(_bits(q.read()), _bits(q2.read()))
    assert np.array_equal(_bits(kc.read()), _bits(kc2.read())) and np.array_equal(_bits(vc.read()), _bits(vc2.read()))
    # and against the oracle
    wq, wk, wv = oracle.qkv_split_rope(qkv, pos, H, D)
    ok, ov = k0.copy(), v0.copy()
    oracle.kv_cache_append(ok, ov, wk.reshape(B, 1, H, D), wv.reshape(B, 1, H, D), cpos)
    _close(q.read(), wq)
    _close(kc.read(), ok)
    assert np.array_equal(_bits(vc.read()), _bits(ov))


@pytest.mark.parametrize("H,D,K,N", [(4, 128, 128, 11100), (8, 64, 192, 11010), (2, 128, 128, 300)])
def test_linear_qkv_rope_packed_equals_separate_ops(backend, arena, oracle, gda, H, D, K, N):
    """The packed prefill's qkv projection with rotation, split and cache append in its epilogue
    (gd_backend_rope_table_packed once, gd_backend_linear_qkv_rope_packed per layer) against the separate operators
    gd_backend_linear_nt -> gd_backend_qkv_split_rope_forward -> gd_backend_kv_cache_append_packed and against the
    oracle.  11,100 rows of 6 column tiles fill one round of 256 tiles (42 row tiles through the tile kernel's rotation
    epilogue, the rest through the plain projection and the table-driven rotation kernel); 300 rows take the second
    path only.  Values bit for bit; rotated elements within one F16 unit in the last place; the skip rules of the
    packed append: a sequence with a negative position, one whose rows do not fit, an empty one."""
    rng = np.random.default_rng(2900 + N)
    B, Tmax = 9, 2048
    cuts = np.sort(rng.choice(np.arange(1, N), B - 2, replace=False))
    cu = np.concatenate([[0], cuts[:3], [cuts[3]], cuts[3:], [N]]).astype(np.int32)  # sequence 4 is empty
    lens = np.diff(cu)
    cache_pos = np.zeros(B, np.int32)
    cache_pos[1], cache_pos[2] = -1, 5
    x = oracle.normal_f16((N, K), 2901, 1.0)
    w = oracle.normal_f16((3 * H * D, K), 2902, 1.0 / np.sqrt(K))
    bias = oracle.normal_f16((3 * H * D,), 2903, 0.1)
    pos = oracle.uniform_i32(N, 2904, 0, 4000)
    k0, v0 = oracle.normal_f16((B, Tmax, H, D), 2905), oracle.normal_f16((B, Tmax, H, D), 2906)
    tx, tw, tb = arena.from_numpy(x), arena.from_numpy(w), arena.from_numpy(bias)
    tpos, tcp, tcu = arena.from_numpy(pos), arena.from_numpy(cache_pos), arena.from_numpy(cu)
    # separate operators
    qkv = arena.alloc((N, 3 * H * D), gda.F16)
    backend.linear_nt(tx, tw, tb, qkv)
    q2, k2, v2 = (arena.from_numpy(np.full((N, H, D), 7.0, np.float16)) for _ in range(3))
    kc2, vc2 = arena.from_numpy(k0), arena.from_numpy(v0)
    backend.qkv_split_rope_forward(qkv, tpos, q2, k2, v2, H, D)
    backend.kv_cache_append_packed(kc2, vc2, tcp, tcu, k2, v2)
    # table + projection with the rotation epilogue
    Npad = (N + 31) // 32 * 32
    cos_rows, sin_rows = arena.alloc((Npad, D // 2), gda.F32), arena.alloc((Npad, D // 2), gda.F32)
    cache_rows = arena.alloc((N,), gda.I32)
    backend.rope_table_packed(tpos, tcp, tcu, cos_rows, sin_rows, cache_rows, D, Tmax)
    rows = cache_rows.read()
    want_rows = np.full(N, -1, np.int64)
    for b in range(B):
        if cache_pos[b] >= 0 and cache_pos[b] + lens[b] <= Tmax:
            want_rows[cu[b]:cu[b + 1]] = b * Tmax + cache_pos[b] + np.arange(lens[b])
    assert np.array_equal(rows, want_rows)
    ang = pos[:, None].astype(np.float64) * np.exp2(np.arange(D // 2) * (-2.0 * np.log2(10000.0) / D))[None, :]
    nn, pp = np.arange(N)[:, None], np.arange(D // 2)[None, :]   # where the tables keep element (n, p)
    at = (((nn // 32) * (D // 16) + pp // 8) * 2 + (pp // 4) % 2) * 128 + (nn % 32) * 4 + pp % 4
    assert np.allclose(cos_rows.read().reshape(-1)[at], np.cos(ang), atol=3e-3)
    assert np.allclose(sin_rows.read().reshape(-1)[at], np.sin(ang), atol=3e-3)
    q1 = arena.from_numpy(np.full((N, H, D), 7.0, np.float16))
    kc1, vc1 = arena.from_numpy(k0), arena.from_numpy(v0)
    work = arena.alloc((N, 3 * H * D), gda.F16)
    backend.linear_qkv_rope_packed(tx, tw, tb, cos_rows, sin_rows, cache_rows, q1, kc1, vc1, work, H, D, 2)
    assert np.array_equal(_bits(vc1.read()), _bits(vc2.read()))
    for a, b in ((q1, q2), (kc1, kc2)):
        a, b = a.read(), b.read()
        ulp = np.spacing(np.maximum(np.abs(a), np.abs(b)).astype(np.float16)).astype(np.float32)
        assert np.all(np.abs(a.astype(np.float32) - b.astype(np.float32)) <= ulp)
        assert np.count_nonzero(_bits(a) != _bits(b)) <= max(2, a.size // 300)
    skipped = [b for b in range(B) if not (cache_pos[b] >= 0 and cache_pos[b] + lens[b] <= Tmax)]
    assert 1 in skipped
    for b in skipped:
        assert np.array_equal(_bits(kc1.read()[b]), _bits(k0[b])) and np.array_equal(_bits(vc1.read()[b]), _bits(v0[b]))
    qo, ko, vo = oracle.qkv_split_rope(oracle.linear_nt(x, w, bias), pos, H, D)
    _close(q1.read(), qo, atol=8e-3)
    got_k, got_v = kc1.read(), vc1.read()
    for b in (b for b in range(B) if b not in skipped):
        _close(got_k[b, cache_pos[b]:cache_pos[b] + lens[b]], ko[cu[b]:cu[b + 1]], atol=8e-3)
        _close(got_v[b, cache_pos[b]:cache_pos[b] + lens[b]], vo[cu[b]:cu[b + 1]], atol=8e-3)
    # arguments that do not fit together are refused before anything is launched
    a = gda.RopeArgs(10000.0, D, 0)
    short = arena.alloc((N - 1,), gda.I32)
    assert backend.call("gd_backend_rope_table_packed", tpos.view(), tcp.view(), tcu.view(), cos_rows.view(), sin_rows.view(),
                        short.view(), D, Tmax, C.byref(a)) == gda.INVALID_ARGUMENT          # cache_rows one row short
    assert backend.call("gd_backend_rope_table_packed", tpos.view(), tcp.view(), tcu.view(), cos_rows.view(), sin_rows.view(),
                        cache_rows.view(), D, 0, C.byref(a)) == gda.INVALID_ARGUMENT         # caches without rows
    inter = gda.RopeArgs(10000.0, D, 1)
    assert backend.call("gd_backend_rope_table_packed", tpos.view(), tcp.view(), tcu.view(), cos_rows.view(), sin_rows.view(),
                        cache_rows.view(), D, Tmax, C.byref(inter)) == gda.UNSUPPORTED      # interleaved pairing
    assert backend.call("gd_backend_linear_qkv_rope_packed", tx.matrix(), tw.matrix(), tb.vector(), cos_rows.view(),
                        sin_rows.view(), short.view(), q1.view(), kc1.view(), vc1.view(), work.matrix(), H, D, 2) == gda.INVALID_ARGUMENT
    assert backend.call("gd_backend_linear_qkv_rope_packed", tx.matrix(), tw.matrix(), None, cos_rows.view(),
                        sin_rows.view(), cache_rows.view(), q1.view(), kc1.view(), vc1.view(), work.matrix(), H, D, 2) == gda.INVALID_ARGUMENT
    assert backend.call("gd_backend_linear_qkv_rope_packed", tx.matrix(), tw.matrix(), tb.vector(), cos_rows.view(),
                        sin_rows.view(), cache_rows.view(), q1.view(), kc1.view(), vc1.view(), work.matrix(), H + 1, D, 2) == gda.INVALID_ARGUMENT
    # refused, not mis-run: a head size the rotation epilogue does not cover
    q96 = arena.alloc((N, 4, 96), gda.F16)
    kc96 = arena.alloc((B, 16, 4, 96), gda.F16)
    c96 = arena.alloc((Npad, 48), gda.F32)
    w96 = arena.alloc((3 * 4 * 96, K), gda.F16)
    wk96 = arena.alloc((N, 3 * 4 * 96), gda.F16)
    b96 = arena.alloc((3 * 4 * 96,), gda.F16)
    assert backend.call("gd_backend_linear_qkv_rope_packed", tx.matrix(), w96.matrix(), b96.vector(), c96.view(), c96.view(),
                        cache_rows.view(), q96.view(), kc96.view(), kc96.view(), wk96.matrix(), 4, 96, 2) == gda.UNSUPPORTED


# ---- sampling front end -----------------------------------------------------------------------------------------

@pytest.mark.parametrize("H,D", [(8, 64), (16, 128), (3, 32)])
def test_qkv_rope_append_packed_equals_separate_ops(backend, arena, oracle, gda, H, D):
    """The packed-prefill form (rotation, split and append of all prompt rows in one launch) against
    gd_backend_qkv_split_rope_forward followed by gd_backend_kv_cache_append_packed: v and the value cache bit for
    bit, q, k and the key cache to one unit in the last place, with the append kernel's skip rules: a sequence with a negative position, one whose rows do not fit behind
    its position, an empty sequence; then a cu_seqlens that does not start at 0 (nothing is appended)."""
    lens = np.array([5, 0, 17, 9, 1, 30], np.int32)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    B, N, Tmax = len(lens), int(cu[-1]), 40
    cache_pos = np.array([0, 3, 20, -1, 39, 11], np.int32)   # 17 rows behind 20 fit exactly; 30 behind 11 do not
    qkv = oracle.normal_f16((N, 3 * H * D), 2800 + D, 1.0)
    pos = oracle.uniform_i32(N, 2801, 0, 4000)
    k0, v0 = oracle.normal_f16((B, Tmax, H, D), 2802), oracle.normal_f16((B, Tmax, H, D), 2803)
    tqkv, tpos, tcp = arena.from_numpy(qkv), arena.from_numpy(pos), arena.from_numpy(cache_pos)
    for cu_used in (cu, cu + 1):
        tcu = arena.from_numpy(cu_used.astype(np.int32))
        q1, k1, v1 = (arena.from_numpy(np.full((N, H, D), 7.0, np.float16)) for _ in range(3))
        kc1, vc1 = arena.from_numpy(k0), arena.from_numpy(v0)
        backend.qkv_rope_append_packed(tqkv, tpos, tcp, tcu, q1, k1, v1, kc1, vc1, H, D)
        # without the packed k / v outputs (a caller that reads the rows from the caches): q and the caches as before
        q3, kc3, vc3 = arena.from_numpy(np.full((N, H, D), 7.0, np.float16)), arena.from_numpy(k0), arena.from_numpy(v0)
        backend.qkv_rope_append_packed(tqkv, tpos, tcp, tcu, q3, None, None, kc3, vc3, H, D)
        for a, b in ((q3, q1), (kc3, kc1), (vc3, vc1)):
            assert np.array_equal(_bits(a.read()), _bits(b.read()))
        q2, k2, v2 = (arena.from_numpy(np.full((N, H, D), 7.0, np.float16)) for _ in range(3))
        kc2, vc2 = arena.from_numpy(k0), arena.from_numpy(v0)
        backend.qkv_split_rope_forward(tqkv, tpos, q2, k2, v2, H, D)
        backend.kv_cache_append_packed(kc2, vc2, tcp, tcu, k2, v2)
        # values are moved bit for bit; the rotation runs in another instantiation of the kernel, where the compiler may
        # contract the angle arithmetic differently: one F16 unit in the last place in a few elements per thousand
        for a, b in ((v1, v2), (vc1, vc2)):
            assert np.array_equal(_bits(a.read()), _bits(b.read()))
        for a, b in ((q1, q2), (k1, k2), (kc1, kc2)):
            a, b = a.read(), b.read()
            ulp = np.spacing(np.maximum(np.abs(a), np.abs(b)).astype(np.float16)).astype(np.float32)
            assert np.all(np.abs(a.astype(np.float32) - b.astype(np.float32)) <= ulp)
            assert np.count_nonzero(_bits(a) != _bits(b)) <= max(2, a.size // 300)
        if cu_used[0] == 0:
            got = kc1.read()
            assert np.array_equal(_bits(got[2, 20:37]), _bits(k1.read()[cu[2]:cu[3]]))       # appended: the rows of k
            assert np.array_equal(_bits(got[0, 0:5]), _bits(k1.read()[cu[0]:cu[1]]))
            assert np.array_equal(_bits(got[4, 39]), _bits(k1.read()[cu[4]]))
            assert np.array_equal(_bits(got[3]), _bits(k0[3])) and np.array_equal(_bits(got[5]), _bits(k0[5]))  # skipped
            assert np.array_equal(_bits(got[2, :20]), _bits(k0[2, :20])) and np.array_equal(_bits(got[2, 37:]), _bits(k0[2, 37:]))
        else:
            assert np.array_equal(_bits(kc1.read()), _bits(k0)) and np.array_equal(_bits(vc1.read()), _bits(v0))
    qo, ko, vo = oracle.qkv_split_rope(qkv, pos, H, D)
    _close(q1.read(), qo, atol=4e-3)
    _close(k1.read(), ko, atol=4e-3)
    assert np.array_equal(_bits(v1.read()), _bits(vo))


def _reference_sampling_step(oracle, logits, hist, hist_len, finished, rng, p, stop, H):
    """One pass of the reference's loop body over the rows (examples/gpt_lm/gpt_lm_shared.c:1606-1680 reordered as
    sample -> stop / full test -> append), with the oracle's restatement of its sampler.  Returns the new rng, the
    per-row record (appended token or -1), the next input ids and the margin of every draw."""
    B = logits.shape[0]
    rec, ids, margins = np.full(B, -1, np.int32), np.zeros(B, np.int32), np.full(B, np.inf)
    for b in range(B):
        if finished[b]:
            ids[b] = stop if stop >= 0 else 0
            continue
        row = oracle.logits_softcap(logits[b].astype(np.float32), p["softcap"])
        tok, rng, margins[b], after = oracle.sample_next_token(row, hist[b, :hist_len[b]], p["temperature"], p["min_p"],
                                                               p["penalty"], rng)
        if not np.isfinite(margins[b]):
            top = np.sort(after[np.isfinite(after)])[-2:]
            margins[b] = np.inf if top.size < 2 else float(top[1] - top[0])   # greedy: gap to the runner-up
        if stop >= 0 and tok == stop:
            finished[b] = 1
        elif hist_len[b] >= H:
            finished[b] = 1
        else:
            hist[b, hist_len[b]] = tok
            hist_len[b] += 1
            rec[b] = tok
        ids[b] = (stop if stop >= 0 else 0) if finished[b] else tok
    return rng, rec, ids, margins


@pytest.mark.parametrize("V", [64, 2048, 32003])
@pytest.mark.parametrize("params", [
    dict(temperature=0.8, min_p=0.05, penalty=1.3, softcap=20.0),
    dict(temperature=1.0, min_p=0.0, penalty=1.0, softcap=0.0),
    dict(temperature=0.0, min_p=0.0, penalty=1.5, softcap=0.0),
    dict(temperature=2.5, min_p=0.5, penalty=float("inf"), softcap=5.0),
])
def test_sample_advance_follows_the_reference_sampler(backend, arena, oracle, gda, V, params):
    B, H, steps, stop = 9, 24, 4, 5
    rng_np = np.random.default_rng(V)
    hist = np.full((B, H), -7, np.int32)
    hist_len = np.array([5, 0, 24, 23, 9, 3, 12, 1, 7], np.int32)   # row 2 is full, row 3 fills up after one token
    for b in range(B):
        hist[b, :hist_len[b]] = rng_np.integers(0, min(V, 40), hist_len[b])   # small range: repeats
    hist[4, 2] = V + 3                                                         # out of range: ignored
    finished = np.array([0, 0, 0, 0, 0, 1, 0, 0, 0], np.int32)
    state0 = 0x0123456789abcdef
    t = dict(history=arena.from_numpy(hist), hist_len=arena.from_numpy(hist_len), finished=arena.from_numpy(finished),
             state=arena.alloc((8 + 10 * B,), gda.I32), work=arena.alloc((backend.sample_work_count(B, V),), gda.F32),
             ids=arena.alloc((B,), gda.I32), positions=arena.from_numpy(np.arange(B, dtype=np.int32) * 3),
             step_counters=arena.from_numpy(np.zeros(B, np.int32)), out_ids=arena.alloc((steps * B,), gda.I32))
    words = np.zeros(8 + 10 * B, np.int32)
    words[:4] = np.array([state0, state0], np.uint64).view(np.int32)
    t["state"].write(words)
    table = oracle.normal_f16((V, 64), 77)
    t["table"], t["next_x"] = arena.from_numpy(table), arena.alloc((B, 64), gda.F16)
    rng = state0
    for s in range(steps):
        logits = oracle.normal_f16((B, V), 5000 + 10 * s + V % 7, 4.0)
        logits[1, 3] = np.nan
        logits[1, 9] = np.inf
        logits[6, :] = [np.nan, np.inf, -np.inf][s % 3]            # nothing finite: token 0, no draw
        logits[7, V // 2] = logits[7, V - 1] = np.float16(30.0)    # tied leaders
        if s == 1:
            logits[8, :] = -np.inf
            logits[8, stop] = 1.0                                  # row 8 must stop here
        backend.sample_advance(arena.from_numpy(logits), t, params["temperature"], params["min_p"], params["penalty"],
                               params["softcap"], stop_token=stop, pos_delta=1)
        rng, rec, ids, margins = _reference_sampling_step(oracle, logits, hist, hist_len, finished, rng, params, stop, H)
        got_rec = t["out_ids"].read().reshape(steps, B)[s]
        diff = np.nonzero(got_rec != rec)[0]
        for b in diff:
            assert margins[b] < 1e-5, f"step {s} row {b}: {got_rec[b]} vs {rec[b]}, margin {margins[b]}"
        if diff.size:
            return   # the histories legitimately part at a near-tie
        assert np.array_equal(t["ids"].read(), ids), s
        assert np.array_equal(t["history"].read(), hist) and np.array_equal(t["hist_len"].read(), hist_len), s
        assert np.array_equal(t["finished"].read(), finished), s
        assert np.array_equal(t["positions"].read(), np.arange(B) * 3 + s + 1)
        assert np.array_equal(t["step_counters"].read(), np.full(B, s + 1))
        assert np.array_equal(_bits(t["next_x"].read()), _bits(table[ids])), s
        got_state = t["state"].read()[:4].view(np.uint64)
        assert int(got_state[s % 2]) == rng, (s, hex(int(got_state[s % 2])), hex(rng))
    assert finished[2] == 1 and finished[3] == 1 and finished[8] == 1 and hist_len[3] == 24


def test_sample_advance_frequencies_and_draw_order(backend, arena, oracle, gda):
    """Every row draws from the same fixed distribution: row b's draw must be number b of the step (the reference
    serves the rows in order from one generator), and the tokens must follow the softmax."""
    B, V, steps = 64, 6, 300
    row = np.array([2.0, 1.0, 0.0, -1.0, 3.0, -4.0], np.float16)
    logits = arena.from_numpy(np.tile(row, (B, 1)))
    t = dict(history=arena.alloc((B, 4), gda.I32), hist_len=arena.from_numpy(np.zeros(B, np.int32)),
             finished=arena.from_numpy(np.zeros(B, np.int32)), state=arena.alloc((8 + 10 * B,), gda.I32),
             work=arena.alloc((backend.sample_work_count(B, V),), gda.F32), ids=arena.alloc((B,), gda.I32),
             positions=arena.from_numpy(np.zeros(B, np.int32)), step_counters=arena.from_numpy(np.zeros(B, np.int32)),
             out_ids=arena.alloc((steps * B,), gda.I32))
    words = np.zeros(8 + 10 * B, np.int32)
    words[:4] = np.array([42, 42], np.uint64).view(np.int32)
    t["state"].write(words)
    zeros = np.zeros(B, np.int32)
    for s in range(steps):
        t["hist_len"].write(zeros)          # keep the histories from filling up: every row keeps drawing
        backend.sample_advance(logits, t, 1.7, 0.0, 1.0, 0.0, stop_token=-1, pos_delta=0)
    got = t["ids"].read()
    out = t["out_ids"].read().reshape(steps, B)
    state, want = 42, np.empty((steps, B), np.int32)
    for s in range(steps):
        for b in range(B):
            want[s, b], state, margin, _ = oracle.sample_next_token(row.astype(np.float32), [], 1.7, 0.0, 1.0, state)
            assert margin > 1e-9
    assert np.array_equal(out, want) and np.array_equal(got, want[-1])
    p = np.exp(row.astype(np.float64) / 1.7)
    p /= p.sum()
    counts = np.bincount(out.ravel(), minlength=V)
    chi2 = float((((counts - out.size * p) ** 2) / (out.size * p)).sum())
    assert chi2 < 25.0, (chi2, counts / out.size, p)


def test_sample_advance_rejects_bad_arguments(backend, arena, gda):
    B, V = 2, 16
    ok = dict(history=arena.alloc((B, 4), gda.I32), hist_len=arena.alloc((B,), gda.I32), finished=arena.alloc((B,), gda.I32),
              state=arena.alloc((8 + 10 * B,), gda.I32), work=arena.alloc((backend.sample_work_count(B, V),), gda.F32), ids=arena.alloc((B,), gda.I32),
              positions=arena.alloc((B,), gda.I32), step_counters=arena.alloc((B,), gda.I32),
              out_ids=arena.alloc((3 * B,), gda.I32))
    logits = arena.alloc((B, V), gda.F16)
    for bad, status in ((dict(state=arena.alloc((8,), gda.I32)), gda.INVALID_ARGUMENT),
                        (dict(work=arena.alloc((B * V,), gda.F32)), gda.INVALID_ARGUMENT),
                        (dict(work=arena.alloc((B * V,), gda.F16)), gda.UNSUPPORTED),
                        (dict(ids=arena.alloc((B + 1,), gda.I32)), gda.INVALID_ARGUMENT),
                        (dict(history=arena.alloc((B + 1, 4), gda.I32)), gda.INVALID_ARGUMENT),
                        (dict(out_ids=arena.alloc((3 * B + 1,), gda.I32)), gda.INVALID_ARGUMENT),
                        (dict(table=arena.alloc((V, 8), gda.F16)), gda.INVALID_ARGUMENT)):
        with pytest.raises(gda.GdError) as err:
            backend.sample_advance(logits, dict(ok, **bad), 1.0)
        assert err.value.status == status, bad.keys()
    with pytest.raises(gda.GdError) as err:
        backend.sample_advance(logits, ok, 1.0, stop_token=V)
    assert err.value.status == gda.INVALID_ARGUMENT


def test_sample_advance_on_the_reference_samplers_golden_cases(backend, arena, oracle, gda):
    """The inputs of tests/golden/sampler_cases.npz through the device kernels: the tokens the reference's own host
    sampler returned (margins from the oracle: a differing token must lie within 1e-5 of a boundary), its generator
    after the last row, and the capped + penalised rows it left behind (work buffer; tanhf may differ by an ulp)."""
    z = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "sampler_cases.npz"))
    for c in sorted({k.split("_")[0] for k in z.files}):
        temperature, min_p, penalty, softcap = (float(v) for v in z[f"{c}_params"])
        logits, hist_len, history = z[f"{c}_logits"], z[f"{c}_hist_len"], z[f"{c}_history"]
        B, V = logits.shape
        H = history.shape[1] + 1                                   # one free place: no row ends by a full history
        hist = np.zeros((B, H), np.int32)
        hist[:, :H - 1] = history
        t = dict(history=arena.from_numpy(hist), hist_len=arena.from_numpy(hist_len),
                 finished=arena.from_numpy(np.zeros(B, np.int32)), state=arena.alloc((8 + 10 * B,), gda.I32),
                 work=arena.alloc((backend.sample_work_count(B, V),), gda.F32), ids=arena.alloc((B,), gda.I32),
                 positions=arena.from_numpy(np.zeros(B, np.int32)), step_counters=arena.from_numpy(np.zeros(B, np.int32)),
                 out_ids=arena.alloc((B,), gda.I32))
        words = np.zeros(8 + 10 * B, np.int32)
        words[:2] = words[2:4] = z[f"{c}_rng"].view(np.int32)
        t["state"].write(words)
        backend.sample_advance(arena.from_numpy(logits.astype(np.float16)), t, temperature, min_p, penalty, softcap,
                               stop_token=-1, pos_delta=0)
        got = t["ids"].read()
        state = int(z[f"{c}_rng"].view(np.uint64)[0])
        for r in range(B):
            tok, state, margin, left = oracle.sample_next_token(oracle.logits_softcap(logits[r], softcap),
                                                                history[r, :hist_len[r]], temperature, min_p, penalty, state)
            assert tok == z[f"{c}_tokens"][r]
            if got[r] != tok:
                if not np.isfinite(margin):
                    top = np.sort(left[np.isfinite(left)])[-2:]
                    margin = float(top[1] - top[0])
                assert margin < 1e-5, (c, r, got[r], tok, margin)
        assert int(t["state"].read()[:4].view(np.uint64)[0]) == int(z[f"{c}_rng_after"].view(np.uint64)[-1]), c
        work = t["work"].read()[:B * V].reshape(B, V)
        want = z[f"{c}_logits_after"]
        same = (work == want) | (np.isnan(work) & np.isnan(want))
        with np.errstate(invalid="ignore"):  # inf - inf on entries `same` already covers
            close = np.abs(work - want) <= 2e-6 * np.abs(want)
        assert np.all(same | close), c
        assert np.array_equal(t["hist_len"].read(), hist_len + 1)


# ---- MiniMax-M3 block-sparse attention --------------------------------------------------------------------------

def _minimax_golden():
    z = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "minimax_cases.npz"))
    for c in sorted({k.split("_")[0] for k in z.files}, key=lambda s: int(s[1:])):
        B, Hq, Hkv, Dh, block, topk, init, local, given = (int(x) for x in z[f"{c}_head"])
        N = int(z[f"{c}_cu"][-1])
        yield dict(name=c, Hq=Hq, Hkv=Hkv, Dh=Dh, block=block, topk=topk, init=init, local=local, given=bool(given),
                   scale=float(z[f"{c}_scale"][0]), cu=z[f"{c}_cu"], q=z[f"{c}_q"].view(np.float16).reshape(N, Hq, Dh),
                   k=z[f"{c}_k"].view(np.float16).reshape(N, Hkv, Dh), v=z[f"{c}_v"].view(np.float16).reshape(N, Hkv, Dh),
                   topk_ref=z[f"{c}_topk"], out_ref=z[f"{c}_out"])


def _assert_same_blocks(oracle, got, want, q, k, cu, block, init, local, where):
    """Identical lists, or the rows that differ hold blocks whose scores tie within 1e-3 (the device sums the
    products in F32, the models in F64)."""
    bad = np.argwhere((got != want).any(axis=2))
    for h, n in bad:
        b = int(np.searchsorted(cu, n, side="right") - 1)
        i = int(n - cu[b])
        qs = q[n, h].astype(np.float64)

        def score(blk):
            j0, j1 = cu[b] + blk * block, cu[b] + min(min((blk + 1) * block, cu[b + 1] - cu[b]), i + 1)
            return float((k[j0:j1, h].astype(np.float64) @ qs).max())
        diff = [(int(x), int(y)) for x, y in zip(got[h, n], want[h, n]) if x != y]
        for x, y in diff:
            assert x >= 0 and y >= 0 and abs(score(x) - score(y)) < 1e-3, f"{where}: head {h} row {n}: {got[h, n]} vs {want[h, n]}"


def test_minimax_m3_reference_models_golden_cases(backend, arena, oracle, gda):
    """The reference's in-test models (tests/golden/minimax_cases.npz; its own two forward cases and six seeded
    shapes): block ids identical, attention within the reference test's 2.5e-3."""
    for c in _minimax_golden():
        N = c["q"].shape[0]
        tq, tk, tv, tcu = (arena.from_numpy(c[n]) for n in ("q", "k", "v", "cu"))
        idx = arena.from_numpy(np.full((c["Hkv"], N, c["topk"]), -9, np.int32))
        if not c["given"]:
            backend.minimax_m3_index_topk(tq, tk, tcu, idx, c["block"], c["init"], c["local"])
            _assert_same_blocks(oracle, idx.read(), c["topk_ref"], c["q"], c["k"], c["cu"], c["block"], c["init"], c["local"],
                                c["name"])
        idx.write(c["topk_ref"])
        out = arena.from_numpy(np.full((N, c["Hq"], c["Dh"]), 7.0, np.float16))
        backend.minimax_m3_sparse_attention(tq, tk, tv, tcu, idx, out, c["block"], c["scale"])
        assert np.abs(out.read().astype(np.float32) - c["out_ref"]).max() < 2.5e-3, c["name"]


@pytest.mark.parametrize("lens,H,Hkv,Dh,block,topk,init,local", [
    ([300, 17, 129, 1], 4, 4, 64, 128, 4, 1, 1),
    ([700], 8, 2, 64, 64, 16, 1, 2),
    ([257, 256, 255], 2, 2, 32, 32, 5, 0, 0),
    ([1000, 40], 2, 1, 16, 8, 8, 3, 1),
])
def test_minimax_m3_matches_oracle(backend, arena, oracle, gda, lens, H, Hkv, Dh, block, topk, init, local):
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    N = int(cu[-1])
    q = oracle.normal_f16((N, H, Dh), 7100 + Dh)
    kq = oracle.normal_f16((N, Hkv, Dh), 7101)            # index q has the kv heads' count
    k = oracle.normal_f16((N, Hkv, Dh), 7102)
    v = oracle.normal_f16((N, Hkv, Dh), 7103)
    tcu, tk = arena.from_numpy(cu), arena.from_numpy(k)
    idx = arena.alloc((Hkv, N, topk), gda.I32)
    backend.minimax_m3_index_topk(arena.from_numpy(kq), tk, tcu, idx, block, init, local, max_seqlen=max(lens))
    want_idx = oracle.minimax_m3_index_topk(kq, k, cu, block, topk, init, local)
    _assert_same_blocks(oracle, idx.read(), want_idx, kq, k, cu, block, init, local, "picker")
    idx.write(want_idx)
    out = arena.from_numpy(np.full((N, H, Dh), 7.0, np.float16))
    scale = float(1.0 / np.sqrt(Dh))
    backend.minimax_m3_sparse_attention(arena.from_numpy(q), tk, arena.from_numpy(v), tcu, idx, out, block, scale,
                                        max_seqlen=max(lens))
    _close(out.read(), oracle.minimax_m3_sparse_attention(q, k, v, cu, want_idx, block, scale))


@pytest.mark.parametrize("Dh,shift", [(24, 0), (7, 0), (1, 0), (63, 0), (48, 0), (16, 3), (64, 1)])
def test_minimax_m3_any_head_size_and_alignment(backend, arena, oracle, gda, Dh, shift):
    """Head sizes without a kernel of their own (the reference takes every size up to 64) and views that start off
    a 16-byte boundary take the half-by-half path; the padding it adds is exact zeros, so the bar is the same."""
    lens, H, Hkv, block, topk = [37, 70], 4, 2, 8, 3
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    N = int(cu[-1])
    q, v = oracle.normal_f16((N, H, Dh), 7300 + Dh), oracle.normal_f16((N, Hkv, Dh), 7400 + Dh)
    k, iq = oracle.normal_f16((N, Hkv, Dh), 7500 + Dh), oracle.normal_f16((N, Hkv, Dh), 7600 + Dh)

    def put(a):  # the view starts `shift` halfs into its allocation
        if shift == 0:
            return arena.from_numpy(a)
        whole = arena.alloc((a.size + shift,), gda.F16)
        whole.write(np.concatenate([np.zeros(shift, np.float16), a.ravel()]))
        return gda.Tensor(whole.buffer, whole.offset + 2 * shift, a.shape, gda.F16)

    tq, tk, tv, tiq = put(q), put(k), put(v), put(iq)
    tcu = arena.from_numpy(cu)
    idx = arena.alloc((Hkv, N, topk), gda.I32)
    backend.minimax_m3_index_topk(tiq, tk, tcu, idx, block, 1, 1)
    want_idx = oracle.minimax_m3_index_topk(iq, k, cu, block, topk, 1, 1)
    _assert_same_blocks(oracle, idx.read(), want_idx, iq, k, cu, block, 1, 1, "picker")
    idx.write(want_idx)
    out = put(np.full((N, H, Dh), 7.0, np.float16))
    scale = float(1.0 / np.sqrt(Dh))
    backend.minimax_m3_sparse_attention(tq, tk, tv, tcu, idx, out, block, scale)
    _close(out.read(), oracle.minimax_m3_sparse_attention(q, k, v, cu, want_idx, block, scale))


@pytest.mark.parametrize("lens,H,Hkv,block,topk,init,local", [
    ([300, 17, 129, 1, 640], 4, 4, 128, 4, 1, 1),
    ([1500], 4, 2, 64, 16, 1, 2),
    ([257, 256, 255, 64, 65], 2, 2, 64, 5, 0, 0),
    ([2100, 40], 2, 1, 128, 3, 2, 0),
])
def test_minimax_m3_matrix_core_kernels(backend, arena, oracle, gda, lens, H, Hkv, block, topk, init, local):
    """Head size 64 with block sizes 64 / 128 (the reference's M3 configuration) takes the matrix-core kernels: both
    against the oracle, and the attention also against the per-row kernel on lists that repeat a block, name blocks
    out of range or past the row, and leave slots empty (lists the picker never produces, the operator must take)."""
    Dh = 64
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    N = int(cu[-1])
    q = oracle.normal_f16((N, H, Dh), 7300 + block)
    kq = oracle.normal_f16((N, Hkv, Dh), 7301)
    k = oracle.normal_f16((N, Hkv, Dh), 7302)
    v = oracle.normal_f16((N, Hkv, Dh), 7303)
    tcu, tk, tq, tv = arena.from_numpy(cu), arena.from_numpy(k), arena.from_numpy(q), arena.from_numpy(v)
    idx = arena.from_numpy(np.full((Hkv, N, topk), -9, np.int32))
    backend.minimax_m3_index_topk(arena.from_numpy(kq), tk, tcu, idx, block, init, local, max_seqlen=max(lens))
    want_idx = oracle.minimax_m3_index_topk(kq, k, cu, block, topk, init, local)
    _assert_same_blocks(oracle, idx.read(), want_idx, kq, k, cu, block, init, local, "matrix-core picker")
    scale = 0.125
    idx.write(want_idx)
    out = arena.from_numpy(np.full((N, H, Dh), 7.0, np.float16))
    backend.minimax_m3_sparse_attention(tq, tk, tv, tcu, idx, out, block, scale, max_seqlen=max(lens))
    _close(out.read(), oracle.minimax_m3_sparse_attention(q, k, v, cu, want_idx, block, scale))
    # hand-made lists
    rng = np.random.default_rng(block + topk)
    odd = rng.integers(-1, max(lens) // block + 3, (Hkv, N, topk)).astype(np.int32)
    odd[:, ::7, 0] = odd[:, ::7, topk - 1]                 # repeated blocks
    idx.write(odd)
    out2 = arena.from_numpy(np.full((N, H, Dh), 7.0, np.float16))
    backend.minimax_m3_sparse_attention(tq, tk, tv, tcu, idx, out2, block, scale, max_seqlen=max(lens))
    want = oracle.minimax_m3_sparse_attention(q, k, v, cu, odd, block, scale)
    _close(out2.read(), want)
    backend.set_tunable("m3_simple", 1)
    try:
        out3 = arena.from_numpy(np.full((N, H, Dh), 7.0, np.float16))
        backend.minimax_m3_sparse_attention(tq, tk, tv, tcu, idx, out3, block, scale, max_seqlen=max(lens))
        idx2 = arena.from_numpy(np.full((Hkv, N, topk), -9, np.int32))
        backend.minimax_m3_index_topk(arena.from_numpy(kq), tk, tcu, idx2, block, init, local, max_seqlen=max(lens))
    finally:
        backend.set_tunable("m3_simple", 0)
    _close(out3.read(), want)
    _assert_same_blocks(oracle, idx2.read(), want_idx, kq, k, cu, block, init, local, "per-row picker")


def test_minimax_m3_full_size_prefill(backend, arena, oracle, gda):
    """The reference's M3 settings (head size 64, blocks of 128, 3 picked, first and last block always) at two full
    4096-token sequences: every list and every output row against the oracle; and rows whose whole context fits
    the picked blocks (the first 3 x 128) equal dense causal attention."""
    lens, H, Hkv, Dh, block, topk = [4096, 4096], 4, 2, 64, 128, 3
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    N = int(cu[-1])
    q, iq, k, v = (oracle.normal_f16((N, h, Dh), s) for h, s in ((H, 7800), (Hkv, 7801), (Hkv, 7802), (Hkv, 7803)))
    tq, tiq, tk, tv, tcu = (arena.from_numpy(a) for a in (q, iq, k, v, cu))
    idx = arena.alloc((Hkv, N, topk), gda.I32)
    backend.minimax_m3_index_topk(tiq, tk, tcu, idx, block, 1, 1, max_seqlen=4096)
    want_idx = oracle.minimax_m3_index_topk(iq, k, cu, block, topk, 1, 1)
    _assert_same_blocks(oracle, idx.read(), want_idx, iq, k, cu, block, 1, 1, "full-size picker")
    idx.write(want_idx)
    out = arena.alloc((N, H, Dh), gda.F16)
    backend.minimax_m3_sparse_attention(tq, tk, tv, tcu, idx, out, block, 0.125, max_seqlen=4096)
    got = out.read()
    _close(got, oracle.minimax_m3_sparse_attention(q, k, v, cu, want_idx, block, 0.125))
    head = slice(4096, 4096 + topk * block)  # second sequence, rows that see at most 3 blocks
    dense = oracle.sdpa_varlen(q[head], k[head], v[head], np.array([0, topk * block], np.int32), 0.125)
    _close(got[head], dense)


@pytest.mark.parametrize("Dh,block", [(64, 64), (32, 16)])
def test_minimax_m3_max_seqlen_cuts_rows_exactly(backend, arena, oracle, gda, Dh, block):
    """Rows at or beyond max_seqlen inside their sequence keep what the outputs held; the rows in front of it are
    what they are without the limit (matrix-core and per-row kernels, a limit inside a row tile)."""
    lens, H, Hkv, topk, limit = [300, 90, 200], 4, 2, 4, 150
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    N = int(cu[-1])
    q, iq, k, v = (oracle.normal_f16((N, h, Dh), s) for h, s in ((H, 7700), (Hkv, 7701), (Hkv, 7702), (Hkv, 7703)))
    tq, tiq, tk, tv, tcu = (arena.from_numpy(a) for a in (q, iq, k, v, cu))
    inside = np.concatenate([np.arange(n) < limit for n in lens])
    full_idx = arena.alloc((Hkv, N, topk), gda.I32)
    backend.minimax_m3_index_topk(tiq, tk, tcu, full_idx, block, 1, 1)
    idx = arena.from_numpy(np.full((Hkv, N, topk), -7, np.int32))
    backend.minimax_m3_index_topk(tiq, tk, tcu, idx, block, 1, 1, max_seqlen=limit)
    got, want = idx.read(), full_idx.read()
    assert np.array_equal(got[:, inside], want[:, inside]) and (got[:, ~inside] == -7).all()
    scale = float(1.0 / np.sqrt(Dh))
    full_out = arena.alloc((N, H, Dh), gda.F16)
    backend.minimax_m3_sparse_attention(tq, tk, tv, tcu, full_idx, full_out, block, scale)
    out = arena.from_numpy(np.full((N, H, Dh), 7.0, np.float16))
    backend.minimax_m3_sparse_attention(tq, tk, tv, tcu, full_idx, out, block, scale, max_seqlen=limit)
    got, want = out.read(), full_out.read()
    assert np.array_equal(got[inside], want[inside]) and (got[~inside] == 7.0).all()


def test_minimax_m3_all_blocks_is_dense_causal_attention(backend, arena, oracle, gda):
    lens = [100, 33]
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    N, H, Dh, block = int(cu[-1]), 4, 64, 8
    q, k, v = (oracle.normal_f16((N, H, Dh), s) for s in (7200, 7201, 7202))
    tq, tk, tv, tcu = (arena.from_numpy(a) for a in (q, k, v, cu))
    idx = arena.alloc((H, N, 13), gda.I32)                 # 13 slots >= 13 blocks of the longest sequence
    backend.minimax_m3_index_topk(tq, tk, tcu, idx, block, 0, 0)
    out = arena.alloc((N, H, Dh), gda.F16)
    backend.minimax_m3_sparse_attention(tq, tk, tv, tcu, idx, out, block, 0.125)
    _close(out.read(), oracle.sdpa_varlen(q, k, v, cu, 0.125))


def test_minimax_m3_rejects_bad_arguments(backend, arena, gda):
    N, H, Dh = 16, 2, 16
    q, k = arena.alloc((N, H, Dh), gda.F16), arena.alloc((N, H, Dh), gda.F16)
    cu, idx = arena.from_numpy(np.array([0, N], np.int32)), arena.alloc((H, N, 4), gda.I32)
    for bad in (dict(k=arena.alloc((N, 1, Dh), gda.F16)), dict(idx=arena.alloc((H, N + 1, 4), gda.I32)),
                dict(idx=arena.alloc((H, N, 17), gda.I32)), dict(block=129), dict(block=0),
                dict(q=arena.alloc((N, H, Dh), gda.F32))):
        a = dict(q=q, k=k, cu=cu, idx=idx, block=8)
        a.update(bad)
        with pytest.raises(gda.GdError) as err:
            backend.minimax_m3_index_topk(a["q"], a["k"], a["cu"], a["idx"], a["block"])
        assert err.value.status == gda.INVALID_ARGUMENT, bad
    with pytest.raises(gda.GdError) as err:  # the reference's limit on the head size
        backend.minimax_m3_index_topk(arena.alloc((N, H, 65), gda.F16), arena.alloc((N, H, 65), gda.F16), cu, idx, 8)
    assert err.value.status == gda.INVALID_ARGUMENT
    out = arena.alloc((N, H, Dh), gda.F16)
    with pytest.raises(gda.GdError) as err:
        backend.minimax_m3_sparse_attention(q, k, arena.alloc((N, H, 8), gda.F16), cu, idx, out, 8, 0.25)
    assert err.value.status == gda.INVALID_ARGUMENT
    with pytest.raises(gda.GdError) as err:
        backend.minimax_m3_sparse_attention(q, k, k, cu, idx, out, 8, 0.0)
    assert err.value.status == gda.INVALID_ARGUMENT
