"""Pins every function of oracle/gd_oracle.c without the HIP backend.

Each oracle function is checked against something it did not come from: the
literal vectors of the reference's own tests (tests/golden/*.json), a library
routine (numpy float16 conversion, numpy float64 matmul, torch's CPU
scaled_dot_product_attention), a closed form, an invariant, or a brute-force
model written as plain Python loops.
"""
import json
import math
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _golden(name):
    with open(os.path.join(GOLDEN, name)) as f:
        return json.load(f)


# ---- F16 conversion -------------------------------------------------------------

def test_f16_to_f32_all_bit_patterns(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    got = oracle.f16_bits_to_f32(bits)
    want = bits.view(np.float16).astype(np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_f32_to_f16_matches_ieee_rne(oracle):
    rng = np.random.default_rng(7)
    exact_halves = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
    x = np.concatenate([
        (rng.standard_normal(200000) * 10.0 ** rng.integers(-9, 6, 200000)).astype(np.float32),
        exact_halves,
        np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 1e9, -1e9, np.inf, -np.inf,
                  2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0000001, 2.0 ** -14, 5.9604645e-08],
                 np.float32),
    ])
    # ties: halfway points between consecutive halves
    h = np.arange(0, 0x7bff, dtype=np.uint16).view(np.float16).astype(np.float64)
    mid = ((h[:-1] + h[1:]) / 2).astype(np.float32)
    x = np.concatenate([x, mid, -mid])
    x = x.astype(np.float32)
    x = x[~np.isnan(x)]
    got = oracle.f32_to_f16_bits(x)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(got, want)


def test_f32_to_f16_nan_collapses(oracle):
    # reference src/core/dtype_internal.h:22-24: any NaN -> sign | 0x7e00
    assert int(oracle.f32_to_f16_bits(np.array([np.nan], np.float32))[0]) & 0x7fff == 0x7e00


# ---- generators -------------------------------------------------------------------

def test_splitmix64_known_answers(oracle):
    # First outputs of Vigna's splitmix64 for state 1234567 (published test vector).
    want = [6457827717110365317, 3203168211198807973, 9817491932198370423,
            4593380528125082431, 16408922859458223821]
    state = 1234567
    got = []
    for _ in want:
        got.append(oracle.splitmix64(state))  # splitmix64(x) = mix(x + golden), one stream step
        state = (state + 0x9E3779B97F4A7C15) & 0xFFFFFFFFFFFFFFFF
    assert got == want


def test_fill_normal_statistics_and_stream(oracle):
    v = oracle.fill_normal(200001, 99, 0.02).astype(np.float64)
    assert abs(v.mean()) < 3e-4
    assert abs(v.std() - 0.02) < 2e-4
    # Box-Muller pairs share one radius: (v0^2+v1^2)/stddev^2 = -2 ln u1 with u1 from the stream.
    u1 = ((oracle.splitmix64(99) >> 11) + 1.0) / 9007199254740992.0
    r2 = (v[0] ** 2 + v[1] ** 2) / 0.02 ** 2
    assert abs(r2 - (-2.0 * math.log(u1))) < 1e-5 * max(1.0, r2)
    # odd count ends on a cosine draw, prefix property
    assert np.array_equal(oracle.fill_normal(7, 5, 1.0), oracle.fill_normal(8, 5, 1.0)[:7])
    h = oracle.normal_f16((9,), 5, 1.0)
    assert np.array_equal(h, oracle.fill_normal(9, 5, 1.0).astype(np.float16))


def test_rand_uniform_is_the_24_bit_draw_of_the_published_stream(oracle):
    # u_i = top 24 bits of splitmix64(seed + i): with seed 1234567 element 0 uses Vigna's published
    # first output 6457827717110365317, whose top 24 bits are 6457827717110365317 >> 40.
    v = oracle.rand_uniform_f32(4, 1234567, 0.0, 1.0)
    assert v[0] == np.float32((6457827717110365317 >> 40) / 16777216.0)
    # affine map: exact for a power-of-two span, and the endpoints bound every draw
    w = oracle.rand_uniform_f32(4, 1234567, -1.0, 1.0)
    assert np.array_equal(w, (-1.0 + 2.0 * v.astype(np.float64)).astype(np.float32))
    big = oracle.rand_uniform_f32(200000, 7, -1.0, 1.0).astype(np.float64)
    assert big.min() >= -1.0 and big.max() < 1.0
    assert abs(big.mean()) < 6e-3 and abs(big.var() - 1.0 / 3.0) < 3e-3
    # element i of seed s is element 0 of seed s + i (counter-based, no carried state)
    assert oracle.rand_uniform_f32(6, 11, 0.0, 1.0)[5] == oracle.rand_uniform_f32(1, 16, 0.0, 1.0)[0]


def test_uniform_i32_range(oracle):
    v = oracle.uniform_i32(50000, 3, 1, 4096)
    assert v.min() >= 1 and v.max() <= 4096 and v.min() < 20 and v.max() > 4080


def test_fill_tokens_and_values_formulas(oracle):
    i = np.arange(40, dtype=np.uint32)
    want = (np.float32(0.25) + np.float32(0.03125) * ((i * 17 + 3) % 19).astype(np.float32)
            - np.float32(0.015625) * (i % 5).astype(np.float32)).astype(np.float16)
    assert np.array_equal(oracle.fill_tokens(40, 0.25), want)
    j = np.arange(50)
    want = 0.1 + 0.05 * ((j * 17 + 5) % 31) - 0.5 * 0.05 * (j % 7)
    assert np.allclose(oracle.fill_values(50, 0.05, 0.1), want, atol=1e-6)


# ---- A1 append ----------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_append_reference_golden_vectors(oracle, dtype):
    g = _golden("kv_cache_append_vectors.json")
    c = g["at"]
    k, v = np.zeros(c["cache_shape"], dtype), np.zeros(c["cache_shape"], dtype)
    oracle.kv_cache_append(k, v, np.array(c["k_new"], dtype).reshape(c["new_shape"]),
                           np.array(c["v_new"], dtype).reshape(c["new_shape"]), c["cache_pos"])
    assert np.array_equal(k.ravel(), np.array(c["expect_k"], dtype))
    assert np.array_equal(v.ravel(), np.array(c["expect_v"], dtype))
    c = g["positions"]
    k, v = np.zeros(c["cache_shape"], dtype), np.zeros(c["cache_shape"], dtype)
    oracle.kv_cache_append(k, v, np.array(c["k_new"], dtype).reshape(c["new_shape"]),
                           np.array(c["v_new"], dtype).reshape(c["new_shape"]),
                           np.array(c["cache_pos"], np.int32))
    assert np.array_equal(k.ravel(), np.array(c["expect_k"], dtype))
    assert np.array_equal(v.ravel(), np.array(c["expect_v"], dtype))
    c = g["packed"]
    k, v = np.zeros(c["cache_shape"], dtype), np.zeros(c["cache_shape"], dtype)
    oracle.kv_cache_append_packed(k, v, np.array(c["k_new"], dtype).reshape(c["new_shape"]),
                                  np.array(c["v_new"], dtype).reshape(c["new_shape"]),
                                  c["cache_pos"], c["cu_seqlens"])
    assert np.array_equal(k.ravel(), np.array(c["expect_k"], dtype))
    assert np.array_equal(v.ravel(), np.array(c["expect_v"], dtype))


def test_append_skip_rules_brute_force(oracle):
    rng = np.random.default_rng(0)
    B, Tmax, H, D, Tnew = 5, 7, 2, 4, 2
    k0 = rng.standard_normal((B, Tmax, H, D)).astype(np.float16)
    v0 = rng.standard_normal((B, Tmax, H, D)).astype(np.float16)
    kn = rng.standard_normal((B, Tnew, H, D)).astype(np.float16)
    vn = rng.standard_normal((B, Tnew, H, D)).astype(np.float16)
    pos = np.array([0, 5, 6, -1, 3], np.int32)  # 6+2 > 7 and -1 are skipped
    k, v = k0.copy(), v0.copy()
    oracle.kv_cache_append(k, v, kn, vn, pos)
    wk, wv = k0.copy(), v0.copy()
    for b in range(B):
        if pos[b] < 0 or pos[b] + Tnew > Tmax:
            continue
        for t in range(Tnew):
            wk[b, pos[b] + t] = kn[b, t]
            wv[b, pos[b] + t] = vn[b, t]
    assert np.array_equal(k.view(np.uint16), wk.view(np.uint16))
    assert np.array_equal(v.view(np.uint16), wv.view(np.uint16))


def test_append_packed_skip_rules_brute_force(oracle):
    rng = np.random.default_rng(1)
    B, Tmax, H, D = 4, 6, 1, 8
    cu = np.array([0, 3, 3, 8, 10], np.int32)  # empty segment 1; segment 2 (len 5) overflows at pos 2
    pos = np.array([1, 0, 2, -1], np.int32)     # segment 3 has a negative position
    N = 12                                       # two trailing rows beyond cu[B]
    kn = rng.standard_normal((N, H, D)).astype(np.float16)
    vn = rng.standard_normal((N, H, D)).astype(np.float16)
    k0 = rng.standard_normal((B, Tmax, H, D)).astype(np.float16)
    v0 = rng.standard_normal((B, Tmax, H, D)).astype(np.float16)
    k, v = k0.copy(), v0.copy()
    oracle.kv_cache_append_packed(k, v, kn, vn, pos, cu)
    wk, wv = k0.copy(), v0.copy()
    for b in range(B):
        n = cu[b + 1] - cu[b]
        if pos[b] < 0 or pos[b] + n > Tmax:
            continue
        for t in range(n):
            wk[b, pos[b] + t] = kn[cu[b] + t]
            wv[b, pos[b] + t] = vn[cu[b] + t]
    assert np.array_equal(k.view(np.uint16), wk.view(np.uint16))
    assert np.array_equal(v.view(np.uint16), wv.view(np.uint16))
    # cu[0] != 0 -> nothing written (reference metal_kv_cache_append.metal:102-104)
    k, v = k0.copy(), v0.copy()
    oracle.kv_cache_append_packed(k, v, kn, vn, np.zeros(B, np.int32), np.array([1, 2, 3, 4, 5], np.int32))
    assert np.array_equal(k.view(np.uint16), k0.view(np.uint16))


# ---- attention mask -------------------------------------------------------------------

def _visible_set(i, T, causal, window, prefix):
    """Independent statement of the mask as a set (not the branch structure):
    causal: keys up to i; with a prefix, queries inside the prefix see the whole prefix.
    window: drop keys more than window-1 behind the query, except that prefix keys are
    never dropped and prefix queries drop nothing."""
    vis = set(range(T))
    if causal:
        if prefix > 0 and i < prefix:
            vis &= set(range(prefix))
        else:
            vis &= set(range(i + 1))
    if window > 0:
        if prefix > 0:
            if i >= prefix:
                vis -= {j for j in range(prefix, T) if i - j >= window}
        else:
            vis -= {j for j in range(T) if i - j >= window}
    return vis


def test_mask_truth_table(oracle):
    T = 9
    for causal in (0, 1):
        for window in (0, 1, 3, 20):
            for prefix in ((0, 2, 5) if causal else (0,)):
                for i in range(T):
                    got = {j for j in range(T) if oracle.attn_allowed(i, j, causal, window, prefix)}
                    assert got == _visible_set(i, T, causal, window, prefix), (causal, window, prefix, i)


# ---- A2 sdpa_decode ----------------------------------------------------------------------

def _np_decode(q, k, v, pos, scale, window=0, prefix=0):
    """float64 numpy model: explicit softmax over the visible set."""
    B, Tq, Hq, D = q.shape
    Tmax, Hkv = k.shape[1], k.shape[2]
    q, k, v = (a.astype(np.float64) for a in (q, k, v))
    out = np.zeros(q.shape)
    for b in range(B):
        live = min(pos[b] + Tq, Tmax)
        for i in range(Tq):
            vis = sorted(j for j in _visible_set(pos[b] + i, Tmax, 1, window, prefix) if j < live)
            if not vis:
                continue
            for h in range(Hq):
                s = scale * (k[b, vis, h // (Hq // Hkv)] @ q[b, i, h])
                p = np.exp(s - s.max())
                out[b, i, h] = (p / p.sum()) @ v[b, vis, h // (Hq // Hkv)]
    return out


def test_decode_reference_test_case(oracle):
    c = _golden("reference_test_cases.json")["sdpa_decode_test_decode"]
    B, Tq, Tmax, Hq, Hkv, D = (c[x] for x in ("B", "Tq", "Tmax", "Hq", "Hkv", "Dh"))
    q = oracle.fill_tokens(B * Tq * Hq * D, c["q_base"]).reshape(B, Tq, Hq, D)
    k = oracle.fill_tokens(B * Tmax * Hkv * D, c["k_base"]).reshape(B, Tmax, Hkv, D)
    v = oracle.fill_tokens(B * Tmax * Hkv * D, c["v_base"]).reshape(B, Tmax, Hkv, D)
    got = oracle.sdpa_decode(q, k, v, [c["cache_pos"]], c["scale"])
    want = _np_decode(q, k, v, [c["cache_pos"]], c["scale"])
    assert np.abs(got - want).max() < 1e-6


@pytest.mark.parametrize("window,prefix", [(0, 0), (3, 0), (4, 2), (0, 3), (64, 0)])
def test_decode_vs_numpy_and_gqa(oracle, window, prefix):
    rng = np.random.default_rng(3)
    B, Tq, Tmax, Hq, Hkv, D = 3, 2, 11, 4, 2, 8
    q = rng.standard_normal((B, Tq, Hq, D)).astype(np.float16)
    k = rng.standard_normal((B, Tmax, Hkv, D)).astype(np.float16)
    v = rng.standard_normal((B, Tmax, Hkv, D)).astype(np.float16)
    pos = np.array([0, 4, 9], np.int32)
    got = oracle.sdpa_decode(q, k, v, pos, 0.3, window, prefix)
    assert np.abs(got - _np_decode(q, k, v, pos, 0.3, window, prefix)).max() < 1e-6
    got32 = oracle.sdpa_decode(q.astype(np.float32), k.astype(np.float32), v.astype(np.float32),
                               pos, 0.3, window, prefix)
    assert np.abs(got32 - got).max() < 1e-6


def test_decode_vs_torch_sdpa(oracle):
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(4)
    B, Tmax, H, D = 2, 37, 3, 16
    q = rng.standard_normal((B, 1, H, D)).astype(np.float16)
    k = rng.standard_normal((B, Tmax, H, D)).astype(np.float16)
    v = rng.standard_normal((B, Tmax, H, D)).astype(np.float16)
    pos = np.array([36, 12], np.int32)
    got = oracle.sdpa_decode(q, k, v, pos, 0.25)
    mask = torch.zeros(B, 1, 1, Tmax, dtype=torch.bool)
    for b in range(B):
        mask[b, 0, 0, : pos[b] + 1] = True
    tq, tk, tv = (torch.from_numpy(a.astype(np.float64)).permute(0, 2, 1, 3) for a in (q, k, v))
    want = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, attn_mask=mask, scale=0.25)
    assert np.abs(got - want.permute(0, 2, 1, 3).numpy()).max() < 1e-6


def test_decode_closed_forms(oracle):
    rng = np.random.default_rng(5)
    B, Tmax, H, D = 2, 9, 2, 4
    q = rng.standard_normal((B, 1, H, D)).astype(np.float16)
    v = rng.standard_normal((B, Tmax, H, D)).astype(np.float16)
    # equal keys -> uniform weights -> mean of the visible values
    k = np.broadcast_to(rng.standard_normal((1, 1, H, D)).astype(np.float16), (B, Tmax, H, D)).copy()
    pos = np.array([8, 3], np.int32)
    got = oracle.sdpa_decode(q, k, v, pos, 1.0)
    for b in range(B):
        assert np.abs(got[b, 0] - v[b, : pos[b] + 1].astype(np.float64).mean(0)).max() < 1e-6
    # one visible key -> that value
    got = oracle.sdpa_decode(q, k, v, np.zeros(B, np.int32), 1.0)
    assert np.array_equal(got[:, 0], v[:, 0].astype(np.float32))
    # negative position -> output left as it was; window 1 -> the newest key's value
    init = np.full(q.shape, 7.0, np.float32)
    got = oracle.sdpa_decode(q, k, v, np.array([-1, 5], np.int32), 1.0, window=1, out_init=init)
    assert np.all(got[0] == 7.0) and np.array_equal(got[1, 0], v[1, 5].astype(np.float32))
    # pos beyond the cache: live length clamps to Tmax
    k2 = rng.standard_normal((B, Tmax, H, D)).astype(np.float16)
    a = oracle.sdpa_decode(q, k2, v, np.array([20, 20], np.int32), 0.5)
    assert np.abs(a - _np_decode(q, k2, v, [20, 20], 0.5)).max() < 1e-6


# ---- A11 sdpa_varlen -------------------------------------------------------------------------

def test_varlen_rows_equal_decode(oracle):
    """Row i of a length-T causal segment equals a decode at position i."""
    rng = np.random.default_rng(6)
    H, Hkv, D = 4, 2, 8
    cu = np.array([0, 5, 5, 12], np.int32)
    N = 12
    q = rng.standard_normal((N, H, D)).astype(np.float16)
    k = rng.standard_normal((N, Hkv, D)).astype(np.float16)
    v = rng.standard_normal((N, Hkv, D)).astype(np.float16)
    for window, prefix in [(0, 0), (3, 0), (2, 3)]:
        got = oracle.sdpa_varlen(q, k, v, cu, 0.4, True, window, prefix)
        for b in range(len(cu) - 1):
            s, e = cu[b], cu[b + 1]
            T = e - s
            for i in range(T):
                # float64 numpy model over the visible set
                vis = sorted(_visible_set(i, T, 1, window, prefix))
                for h in range(H):
                    sc = 0.4 * (k[s:e][vis, h // 2].astype(np.float64) @ q[s + i, h].astype(np.float64))
                    p = np.exp(sc - sc.max())
                    want = (p / p.sum()) @ v[s:e][vis, h // 2].astype(np.float64)
                    assert np.abs(got[s + i, h] - want).max() < 1e-6
                if i < prefix - 1:
                    continue  # a decode at position i cannot see prefix keys that are not live yet
                want = oracle.sdpa_decode(q[s + i][None, None], k[s:e][None], v[s:e][None], [i],
                                          0.4, window, prefix)[0, 0]
                assert np.abs(got[s + i] - want).max() < 1e-6
    # non-causal: every row sees the whole segment
    got = oracle.sdpa_varlen(q, k, v, cu, 0.4, False)
    s = 0.4 * np.einsum("hd,jhd->hj", q[2].astype(np.float64), np.repeat(k[:5], 2, 1).astype(np.float64))
    p = np.exp(s - s.max(1, keepdims=True))
    want = np.einsum("hj,jhd->hd", p / p.sum(1, keepdims=True), np.repeat(v[:5], 2, 1).astype(np.float64))
    assert np.abs(got[2] - want).max() < 1e-6
    # max_seqlen truncates the queries of a longer segment
    got = oracle.sdpa_varlen(q, k, v, cu, 0.4, True, max_seqlen=6)
    assert np.all(got[11] == 0) and np.any(got[10] != 0)


# ---- A3 rms_norm ---------------------------------------------------------------------------------

def test_rms_norm_reference_case_and_invariants(oracle):
    c = _golden("reference_test_cases.json")["rms_norm_f32_2x4"]
    x = np.array(c["x"], np.float32).reshape(2, 4)
    w = np.array(c["w"], np.float32)
    x64 = x.astype(np.float64)
    want = x64 * w / np.sqrt((x64 ** 2).mean(1, keepdims=True) + c["eps"])
    assert np.abs(oracle.rms_norm(x, w, c["eps"]) - want).max() < c["tol_abs"]
    rng = np.random.default_rng(8)
    xh = rng.standard_normal((5, 512)).astype(np.float16)
    wh = (1 + 0.1 * rng.standard_normal(512)).astype(np.float16)
    y = oracle.rms_norm(xh, wh, 1e-5).astype(np.float64)
    x64 = xh.astype(np.float64)
    want = x64 * wh.astype(np.float64) / np.sqrt((x64 ** 2).mean(1, keepdims=True) + 1e-5)
    assert np.abs(y - want).max() <= np.abs(want).max() * 2 ** -10
    # unit weight -> unit RMS; scale invariance
    y1 = oracle.rms_norm(xh, np.ones(512, np.float16), 1e-5).astype(np.float64)
    assert np.abs(np.sqrt((y1 ** 2).mean(1)) - 1).max() < 1e-3
    y2 = oracle.rms_norm((xh * np.float16(4)).astype(np.float16), np.ones(512, np.float16), 1e-5)
    assert np.abs(y2.astype(np.float64) - y1).max() < 2e-3


# ---- A4 qkv_split_rope -----------------------------------------------------------------------------

def test_rope_split_map_and_rotation(oracle):
    rng = np.random.default_rng(9)
    N, H, D = 6, 3, 8
    qkv = rng.standard_normal((N, 3 * H * D)).astype(np.float16)
    pos = np.array([0, 1, 2, 17, 511, 4095], np.int32)
    q, k, v = oracle.qkv_split_rope(qkv, pos, H, D)
    src = qkv.reshape(N, 3, H, D)
    assert np.array_equal(v.view(np.uint16), src[:, 2].view(np.uint16))      # v: bit copy
    assert np.array_equal(q[0].view(np.uint16), src[0, 0].view(np.uint16))   # pos 0: identity
    assert np.array_equal(k[0].view(np.uint16), src[0, 1].view(np.uint16))
    # rope_ref of the reference's tests/test_rope.c:67-104 (powf frequency), in float64
    half = D // 2
    for n in range(N):
        for p in range(half):
            ang = float(np.float32(pos[n]) * np.float32(np.float32(10000.0) ** np.float32(-2.0 * p / D)))
            c, s = math.cos(ang), math.sin(ang)
            for which, got in ((0, q), (1, k)):
                x0 = src[n, which, :, p].astype(np.float64)
                x1 = src[n, which, :, p + half].astype(np.float64)
                tol = 2e-3 + 2e-3 * max(np.abs(x0).max(), np.abs(x1).max())
                assert np.abs(got[n, :, p].astype(np.float64) - (x0 * c - x1 * s)).max() < tol
                assert np.abs(got[n, :, p + half].astype(np.float64) - (x0 * s + x1 * c)).max() < tol
    # rotation preserves each pair's norm
    n_in = src[:, 0].astype(np.float64) ** 2
    n_out = q.astype(np.float64) ** 2
    assert np.abs((n_in[..., :half] + n_in[..., half:]) - (n_out[..., :half] + n_out[..., half:])).max() < 2e-2
    # known angle: pos 1, pair 0 -> 1 radian applied to (1, 0)
    one = np.zeros((1, 3 * H * D), np.float16)
    one[0, 0] = 1.0
    q1, _, _ = oracle.qkv_split_rope(one, [1], H, D)
    assert abs(float(q1[0, 0, 0]) - math.cos(1.0)) < 1e-3 and abs(float(q1[0, 0, half]) - math.sin(1.0)) < 1e-3
    # interleaved pairing (2p, 2p+1)
    qi, _, _ = oracle.qkv_split_rope(one, [1], H, D, interleaved=True)
    assert abs(float(qi[0, 0, 1]) - math.sin(1.0)) < 1e-3 and float(qi[0, 0, half]) == 0.0


# ---- A5/A6 projections -------------------------------------------------------------------------------

def test_linear_vs_numpy_float64(oracle):
    c = _golden("reference_test_cases.json")["linear_f16"]
    M, K, N = 5, 48, 24
    x = oracle.fill_values(M * K, 0.01, -0.1).astype(np.float16).reshape(M, K)
    w_kn = oracle.fill_values(K * N, 0.02, -0.3).astype(np.float16).reshape(K, N)
    bias = oracle.fill_values(N, 0.05, -0.5).astype(np.float16)
    x64, w64, b64 = (a.astype(np.float64) for a in (x, w_kn, bias))
    y = oracle.linear(x, w_kn, bias).astype(np.float64)
    want = x64 @ w64 + b64
    assert np.abs(y - want).max() < c["tol_abs"] * max(1.0, np.abs(want).max())
    assert np.array_equal(oracle.linear(x, w_kn, bias), want.astype(np.float32).astype(np.float16))
    w_nk = np.ascontiguousarray(w_kn.T)
    y_nt = oracle.linear_nt(x, w_nk)
    assert np.array_equal(y_nt, (x64 @ w64).astype(np.float32).astype(np.float16))
    # NT with bias rounds twice
    y_ntb = oracle.linear_nt(x, w_nk, bias)
    assert np.array_equal(y_ntb, (y_nt.astype(np.float32) + bias.astype(np.float32)).astype(np.float16))
    # identity weight returns the input; one-hot input selects a weight row
    eye = np.eye(K, dtype=np.float16)
    assert np.array_equal(oracle.linear(x, eye), x) and np.array_equal(oracle.linear_nt(x, eye), x)
    onehot = np.zeros((1, K), np.float16)
    onehot[0, 7] = 1
    assert np.array_equal(oracle.linear(onehot, w_kn)[0], w_kn[7])
    assert np.array_equal(oracle.linear_nt(onehot, w_nk)[0], w_nk[:, 7])


# ---- A7 swiglu, A8 add, A9 embedding, A10 argmax ---------------------------------------------------------

def test_swiglu_reference_cases(oracle):
    g = _golden("reference_test_cases.json")
    c = g["swiglu_split"]
    i = np.arange(c["rows"] * 2 * c["H"])
    x12 = (((i % 17) - 8) * 0.375).astype(np.float16).reshape(c["rows"], 2 * c["H"])
    x64 = x12.astype(np.float64)
    z = x64[:, c["H"]:]
    want = x64[:, :c["H"]] * z / (1 + np.exp(-z))
    got = oracle.swiglu_split(x12)
    assert np.abs(got.astype(np.float64) - want).max() < c["tol_abs"]
    assert np.array_equal(got, want.astype(np.float32).astype(np.float16))
    # silu(0) = 0, silu(large) -> z, silu(-large) -> 0
    t = np.array([[2.0, 3.0, 5.0, 0.0, 30.0, -30.0]], np.float16)
    assert np.array_equal(oracle.swiglu_split(t)[0], np.array([0.0, 90.0, -0.0], np.float16))
    c = g["swiglu_split_linear"]
    i = np.arange(c["rows"] * 2 * c["H"])
    x12 = (((i % 13) - 6) * 0.25).astype(np.float16).reshape(c["rows"], 2 * c["H"])
    j = np.arange(c["H"] * c["O"])
    w = (((j % 7) - 3) * 0.125).astype(np.float16).reshape(c["H"], c["O"])
    x64 = x12.astype(np.float64)
    act = x64[:, :c["H"]] * x64[:, c["H"]:] / (1 + np.exp(-x64[:, c["H"]:]))
    want = act @ w.astype(np.float64)
    assert np.abs(oracle.swiglu_split_linear(x12, w).astype(np.float64) - want).max() < c["tol_abs"]


def test_add_is_ieee_half_add(oracle):
    rng = np.random.default_rng(10)
    a = (rng.standard_normal((7, 33)) * 100).astype(np.float16)
    b = (rng.standard_normal((7, 33)) * 0.1).astype(np.float16)
    assert np.array_equal(oracle.add(a, b).view(np.uint16), (a + b).view(np.uint16))
    bias = rng.standard_normal(33).astype(np.float16)
    assert np.array_equal(oracle.add(a, bias).view(np.uint16), (a + bias).view(np.uint16))
    big = np.array([65504.0], np.float16)
    assert np.isinf(oracle.add(big, big)[0])


def test_embedding_gather_and_invalid_id(oracle):
    rng = np.random.default_rng(11)
    table = rng.standard_normal((10, 6)).astype(np.float16)
    ids = np.array([3, 0, 9, -1, 10, 3], np.int32)
    out = oracle.embedding(table, ids)
    for i, t in enumerate(ids):
        if 0 <= t < 10:
            assert np.array_equal(out[i].view(np.uint16), table[t].view(np.uint16))
        else:
            assert np.all(out[i].view(np.uint16) == 0x7e00)


def test_argmax_brute_force(oracle):
    rng = np.random.default_rng(12)
    logits = rng.standard_normal((6, 50)).astype(np.float16)
    logits[1, 10] = logits[1, 30] = np.float16(9.0)   # tie: first wins
    logits[2, :] = np.nan                             # nothing finite -> 0
    logits[3, 5] = np.inf                             # +inf is skipped (non-finite)
    logits[3, 7] = np.float16(8.0)
    logits[4, :] = -np.inf
    logits[4, 20] = np.float16(-3.0)                  # single finite value
    logits[5, 0] = np.nan
    ids, gap = oracle.argmax_rows(logits)
    for r in range(6):
        best, bv, second = 0, None, None
        for i in range(50):
            val = float(logits[r, i])
            if not math.isfinite(val):
                continue
            if bv is None or val > bv:
                second = bv if bv is not None else second
                bv, best = val, i
            elif second is None or val > second:
                second = val
        assert ids[r] == best
        if bv is not None and second is not None:
            assert gap[r] == np.float32(bv - second)
        else:
            assert np.isinf(gap[r])
    assert ids[1] == 10 and gap[1] == 0.0 and ids[2] == 0 and ids[3] == 7 and ids[4] == 20


# ---- A13 decoder ----------------------------------------------------------------------------------------------

def _small_decoder(oracle, batch, window=0, seed=1000):
    return oracle.Decoder(vocab=96, d_model=32, n_layers=2, n_heads=4, head_dim=8, mlp_hidden=48,
                          max_seq=16, batch=batch, window=window, seed=seed)


def test_decoder_weight_init_follows_reference_seeds(oracle):
    d = _small_decoder(oracle, 1)
    emb = oracle.fill_normal(96 * 32, oracle.splitmix64(1000 ^ 0xabc001), 0.02).astype(np.float16)
    assert np.array_equal(d.tensor("embed").ravel(), emb)
    bs = 1000 ^ (1 << 8)
    resid = np.float32(0.02) / np.sqrt(np.float32(4.0))
    w = oracle.fill_normal(48 * 32, oracle.splitmix64(bs ^ 4), float(resid)).astype(np.float16)
    assert np.array_equal(d.tensor("w_down", 1).ravel(), w)
    assert np.all(d.tensor("attn_norm", 0) == 1) and np.all(d.tensor("b_qkv", 1) == 0)


@pytest.mark.parametrize("window", [0, 4])
def test_decoder_decode_matches_full_forward(oracle, window):
    """The invariant of the reference's probes/gpt_lm_debug/compare_decode.c:14-18:
    prefill(n) + one cached decode step == row n of a packed forward over n+1 tokens."""
    ids = oracle.uniform_i32(9, 42, 0, 95)
    a = _small_decoder(oracle, 1, window)
    a.prefill(ids[:8], [0, 8])
    logits_step, nxt_step, _ = a.step(ids[8:9])
    b = _small_decoder(oracle, 1, window)
    logits_full, nxt_full, _ = b.prefill(ids, [0, 9])
    assert np.array_equal(a.positions, [9]) and np.array_equal(b.positions, [9])
    assert np.abs(logits_step.astype(np.float32) - logits_full.astype(np.float32)).max() < 2e-3
    assert np.array_equal(a.tensor("k_cache", 1)[0, :9].view(np.uint16),
                          b.tensor("k_cache", 1)[0, :9].view(np.uint16))


def test_decoder_batch_rows_independent(oracle):
    ids = oracle.uniform_i32(12, 43, 0, 95)
    d2 = _small_decoder(oracle, 2)
    cu = np.array([0, 5, 12], np.int32)
    lg2, nx2, _ = d2.prefill(ids, cu)
    d1 = _small_decoder(oracle, 1)
    lg1, nx1, _ = d1.prefill(ids[5:], [0, 7])
    assert np.array_equal(lg2[1].view(np.uint16), lg1[0].view(np.uint16))
    s2, n2, _ = d2.step(nx2)
    s1, n1, _ = d1.step(nx1)
    assert np.array_equal(s2[1].view(np.uint16), s1[0].view(np.uint16)) and n2[1] == n1[0]


# ---- sampling front end (reference examples/gpt_lm/gpt_lm_shared.c:1322-1442) --------------------------------

def test_softcap_against_numpy_and_identity_cases(oracle):
    rng = np.random.default_rng(3)
    x = np.concatenate([rng.normal(0, 30, 4000), [0.0, -0.0, 1e-8, 200.0, -200.0, np.inf, -np.inf]]).astype(np.float32)
    got = oracle.logits_softcap(x, 20.0)
    want = 20.0 * np.tanh(x.astype(np.float64) / 20.0)
    assert np.allclose(got, want, rtol=3e-7, atol=1e-12)
    assert got[-2] == 20.0 and got[-1] == -20.0 and np.all(np.abs(got) <= 20.0)
    for cap in (0.0, -1.0, float("nan")):
        assert np.array_equal(oracle.logits_softcap(x, cap), x)


def test_repetition_penalty_brute_force(oracle):
    rng = np.random.default_rng(4)
    logits = rng.normal(0, 3, 50).astype(np.float32)
    logits[7] = 0.0
    history = np.array([3, 7, 3, 49, -1, 50, 12, 12, 12, 0, 3], np.int32)
    got = oracle.repetition_penalty(logits, history, 1.3)
    want = logits.copy()
    for t in set(int(t) for t in history if 0 <= t < 50):   # once per distinct token, however often it occurs
        want[t] = want[t] / np.float32(1.3) if want[t] > 0 else want[t] * np.float32(1.3)
    assert np.array_equal(got, want)
    assert got[3] != logits[3] and got[7] == 0.0 and got[5] == logits[5]
    for off in (1.0, 0.5, float("nan"), float("inf")):
        assert np.array_equal(oracle.repetition_penalty(logits, history, off), logits)
    assert np.array_equal(oracle.repetition_penalty(logits, history[:0], 1.3), logits)


def test_sampling_greedy_cases_leave_the_generator_alone(oracle):
    logits = np.array([1.0, 5.0, np.nan, 5.0, np.inf, -np.inf, 2.0], np.float32)
    for temperature in (0.0, -1.0, float("nan"), float("inf")):
        tok, state, margin, _ = oracle.sample_next_token(logits, [], temperature, 0.0, 1.0, 99)
        assert (tok, state) == (1, 99) and margin == np.inf     # first of the tied finite maxima, no draw
    bad = np.array([np.nan, np.inf, -np.inf], np.float32)
    assert oracle.sample_next_token(bad, [], 1.0, 0.0, 1.0, 5)[:2] == (0, 5)
    # the penalty acts before the pick: the repeated leader loses
    assert oracle.sample_next_token(np.array([4.0, 3.9], np.float32), [0], 0.0, 0.0, 1.5, 1)[0] == 1


def test_sampling_draw_is_the_inverse_cdf_of_the_softmax(oracle):
    # equal logits: token = floor(u * V) with u the 53-bit fraction of the advanced state
    state = 0x1234
    for _ in range(200):
        tok, new_state, margin, _ = oracle.sample_next_token(np.zeros(8, np.float32), [], 1.0, 0.0, 1.0, state)
        assert new_state == oracle.splitmix64(state)
        u = (new_state >> 11) / 2.0 ** 53
        assert tok == int(np.floor(u * 8)), (tok, u)
        assert abs(margin - min(u * 8 - tok, tok + 1 - u * 8) / 8) < 1e-12
        state = new_state
    # general logits, temperature and min_p against numpy's float64 softmax / cumsum / searchsorted
    rng = np.random.default_rng(8)
    for case in range(300):
        V = int(rng.integers(2, 300))
        logits = rng.normal(0, 4, V).astype(np.float32)
        if case % 3 == 0:
            logits[rng.integers(0, V, 3)] = [np.nan, np.inf, -np.inf]
        temperature = float(rng.choice([0.3, 0.8, 1.0, 2.5]))
        min_p = float(rng.choice([0.0, 0.05, 0.3, 1.0]))
        tok, new_state, margin, _ = oracle.sample_next_token(logits, [], temperature, min_p, 1.0, 1000 + case)
        finite = np.isfinite(logits)
        if not finite.any():
            assert (tok, new_state) == (0, 1000 + case)
            continue
        z = np.where(finite, logits.astype(np.float64), -np.inf)
        p = np.exp((z - z.max()) / temperature)                 # relative to the leader: p.max() == 1
        keep = finite & (p >= min_p * (1 - 1e-12)) if min_p > 0 else finite
        mass = np.where(keep, p, 0.0)
        u = (oracle.splitmix64(1000 + case) >> 11) / 2.0 ** 53
        want = int(np.searchsorted(np.cumsum(mass), u * mass.sum(), side="left"))
        if margin > 1e-9:
            assert tok == want, (case, tok, want, margin)
        assert keep[tok]


def test_sampling_frequencies_follow_the_distribution(oracle):
    logits = np.array([2.0, 1.0, 0.0, -1.0, 3.0, -4.0], np.float32)
    temperature, n = 1.7, 40000
    counts = np.zeros(6)
    state = 777
    for _ in range(n):
        tok, state, _, _ = oracle.sample_next_token(logits, [], temperature, 0.0, 1.0, state)
        counts[tok] += 1
    p = np.exp(logits.astype(np.float64) / temperature)
    p /= p.sum()
    chi2 = float((((counts - n * p) ** 2) / (n * p)).sum())
    assert chi2 < 25.0, (chi2, counts / n, p)                   # 5 degrees of freedom: P(chi2 > 25) ~ 1e-4
    # with min_p the tail is cut and the rest renormalised
    counts[:] = 0
    for _ in range(n):
        tok, state, _, _ = oracle.sample_next_token(logits, [], temperature, 0.2, 1.0, state)
        counts[tok] += 1
    keep = p >= 0.2 * p.max()
    assert counts[~keep].sum() == 0 and 1 < keep.sum() < 6
    q = np.where(keep, p, 0) / p[keep].sum()
    chi2 = float((((counts[keep] - n * q[keep]) ** 2) / (n * q[keep])).sum())
    assert chi2 < 25.0


def test_sampler_equals_the_reference_sampler_on_golden_cases(oracle):
    """tests/golden/sampler_cases.npz holds what the reference's own gpt_apply_logits_softcap +
    gpt_sample_next_token returned (tests/golden/make_sampler_fixture.py ran them through oracle/_ref/ref_sampler):
    tokens, the generator after every row and the rows as the sampler left them must be identical."""
    import os
    z = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "sampler_cases.npz"))
    cases = sorted({k.split("_")[0] for k in z.files})
    assert len(cases) == 7
    for c in cases:
        temperature, min_p, penalty, softcap = (float(v) for v in z[f"{c}_params"])
        state = int(z[f"{c}_rng"].view(np.uint64)[0])
        after = z[f"{c}_rng_after"].view(np.uint64)
        drew = 0
        for r, row in enumerate(z[f"{c}_logits"]):
            capped = oracle.logits_softcap(row, softcap)
            hist = z[f"{c}_history"][r, :z[f"{c}_hist_len"][r]]
            tok, new_state, _, left = oracle.sample_next_token(capped, hist, temperature, min_p, penalty, state)
            assert tok == z[f"{c}_tokens"][r], (c, r)
            assert new_state == int(after[r]), (c, r)
            assert np.array_equal(left.view(np.uint32), z[f"{c}_logits_after"][r].view(np.uint32)), (c, r)
            drew += new_state != state
            state = new_state
        assert (drew > 0) == (np.isfinite(temperature) and temperature > 0), c


# ---- MiniMax-M3 block-sparse attention (reference tests/test_minimax_m3_sparse_attention.c) -------------------

def _minimax_cases():
    import os
    z = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "minimax_cases.npz"))
    for c in sorted({k.split("_")[0] for k in z.files}, key=lambda s: int(s[1:])):
        B, Hq, Hkv, Dh, block, topk, init, local, given = (int(x) for x in z[f"{c}_head"])
        N = int(z[f"{c}_cu"][-1])
        yield dict(name=c, B=B, Hq=Hq, Hkv=Hkv, Dh=Dh, block=block, topk=topk, init=init, local=local, given=bool(given),
                   scale=float(z[f"{c}_scale"][0]), cu=z[f"{c}_cu"], q=z[f"{c}_q"].view(np.float16).reshape(N, Hq, Dh),
                   k=z[f"{c}_k"].view(np.float16).reshape(N, Hkv, Dh), v=z[f"{c}_v"].view(np.float16).reshape(N, Hkv, Dh),
                   topk_ref=z[f"{c}_topk"], out_ref=z[f"{c}_out"])


def test_minimax_block_picker_and_attention_equal_the_reference_models(oracle):
    """tests/golden/minimax_cases.npz: the reference's own ref_topk / ref_sparse_fwd / ref_sparse_fwd_gqa (its test
    program's functions, run by oracle/_ref/ref_minimax) on its two forward test cases and six seeded shapes.  Block
    ids must be identical; outputs within the reference test's own bound (2.5e-3 absolute, :677, 762)."""
    n = 0
    for c in _minimax_cases():
        if not c["given"]:
            got = oracle.minimax_m3_index_topk(c["q"], c["k"], c["cu"], c["block"], c["topk"], c["init"], c["local"])
            assert np.array_equal(got, c["topk_ref"]), c["name"]
        out = oracle.minimax_m3_sparse_attention(c["q"], c["k"], c["v"], c["cu"], c["topk_ref"], c["block"], c["scale"])
        assert np.abs(out.astype(np.float32) - c["out_ref"]).max() < 2.5e-3, c["name"]
        assert np.abs(out.astype(np.float32) - c["out_ref"]).max() < 1e-3 * max(1.0, np.abs(c["out_ref"]).max())
        n += 1
    assert n == 8


def test_minimax_all_blocks_selected_is_dense_causal_attention(oracle):
    """With at least as many slots as blocks every visible block is listed: the operator pair must then equal plain
    causal attention over the packed sequences (sdpa_varlen of this oracle, pinned elsewhere against numpy / torch)."""
    rng = np.random.default_rng(5)
    lens = [19, 1, 40]
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    N, Hq, Hkv, Dh, block = int(cu[-1]), 4, 2, 16, 8
    q = rng.normal(0, 1, (N, Hq, Dh)).astype(np.float16)
    k = rng.normal(0, 1, (N, Hkv, Dh)).astype(np.float16)
    v = rng.normal(0, 1, (N, Hkv, Dh)).astype(np.float16)
    idx = oracle.minimax_m3_index_topk(k, k, cu, block, 5, 0, 0)          # 5 slots, at most 5 blocks per row
    for b in range(3):
        for i in range(lens[b]):
            row = idx[0, cu[b] + i]
            assert sorted(x for x in row if x >= 0) == list(range(i // block + 1))
    sparse = oracle.minimax_m3_sparse_attention(q, k, v, cu, idx, block, 0.25)
    dense = oracle.sdpa_varlen(q, k, v, cu, 0.25)
    assert np.abs(sparse.astype(np.float32) - dense.astype(np.float32)).max() < 2e-3


def test_minimax_block_picker_priorities_and_ties(oracle):
    # one sequence of 40 rows, block 4 -> 10 blocks; scores made explicit: q = e0, k_j = s_j * e0
    block, T = 4, 40
    scores = np.array([0.5, 3.0, 3.0, -1.0, 2.0, 9.0, 0.0, 1.0, 9.0, 4.0], np.float32)   # per block
    q = np.zeros((T, 1, 4), np.float16)
    q[:, 0, 0] = 1.0
    k = np.zeros((T, 1, 4), np.float16)
    k[:, 0, 0] = np.repeat(scores, block)
    cu = [0, T]
    last = oracle.minimax_m3_index_topk(q, k, cu, block, 4, 0, 0)[0, T - 1].tolist()
    assert last == [5, 8, 9, 1]                       # 9.0 twice: the earlier block first; 3.0 twice: block 1 wins
    assert oracle.minimax_m3_index_topk(q, k, cu, block, 4, 2, 0)[0, T - 1].tolist() == [0, 1, 5, 8]   # forced first blocks
    assert oracle.minimax_m3_index_topk(q, k, cu, block, 4, 2, 1)[0, T - 1].tolist() == [0, 1, 9, 5]   # then the local one
    assert oracle.minimax_m3_index_topk(q, k, cu, block, 4, 0, 2)[0, T - 1].tolist() == [8, 9, 5, 1]
    row5 = oracle.minimax_m3_index_topk(q, k, cu, block, 4, 0, 0)[0, 5].tolist()
    assert row5 == [1, 0, -1, -1]                     # row 5 sees blocks 0 and 1 only
    # a block that is both first and local ranks as local (1e29 after 1e30): visible in the order of rows in block 0
    assert oracle.minimax_m3_index_topk(q, k, cu, block, 2, 1, 1)[0, 2].tolist() == [0, -1]
    assert oracle.minimax_m3_index_topk(q, k, cu, block, 2, 1, 1)[0, 9].tolist() == [0, 2]
    k[:, 0, 0] = np.nan                               # NaN scores: nothing is picked unless forced
    assert oracle.minimax_m3_index_topk(q, k, cu, block, 3, 0, 0)[0, T - 1].tolist() == [-1, -1, -1]
    assert oracle.minimax_m3_index_topk(q, k, cu, block, 3, 1, 1)[0, T - 1].tolist() == [0, 9, -1]
