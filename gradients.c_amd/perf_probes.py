"""Operator-local performance probes (the counterpart of the reference's per-operator perf programs, e.g.
src/ops/sdpa_varlen/perf_test.c and docs/guides/register_op.md:218-247): one operator at the shapes of the
BASELINE.json configurations, timed with stream events around graph replays, one JSON line per probe.

    python bench.py --probe sdpa_decode        split-KV decode attention, caches rotating through HBM
    python bench.py --probe few_row_linear     decode-time projections of the scaled decoder, weights rotating through HBM
    python bench.py --probe tile_gemm          prefill projections on the matrix cores (also the program of the --pmc runs)
    python bench.py --probe prefill_attention  packed causal attention of the prefill (gd_backend_sdpa_varlen) at the
                                               prompt mixes of configs[3] and [4] and at equal lengths
    python bench.py --probe tile_timeline      the same projections in a profiling build of the library
                                               (make -C gradients.c_amd/csrc TILE_TIMELINE=1): K loop and epilogue
                                               time per tile and the clock the chip ran at

Every probe reads more distinct bytes between two reads of the same byte than the 256 MB memory-side cache holds, so
what it times comes from HBM.
"""
import json

import numpy as np

HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0


def _timed(pkg, be, fns, replays=4, repeats=3):
    """Every fn once per graph; median microseconds per fn call over `repeats` timings of `replays` graph launches."""
    timer = pkg.Timer(be)
    be.scope_begin()
    for f in fns:
        f()
    be.graph_begin_capture()
    for f in fns:
        f()
    graph = be.graph_end_capture()
    be.graph_launch(graph)
    res = []
    for _ in range(repeats):
        timer.start()
        for _ in range(replays):
            be.graph_launch(graph)
        timer.stop()
        res.append(timer.elapsed_ms() * 1e3 / (replays * len(fns)))
    be.fence_wait(be.record_fence())
    be.graph_destroy(graph)
    timer.close()
    return sorted(res)[len(res) // 2]


def sdpa_decode(pkg):
    """gd_backend_sdpa_decode_positions at the shapes of configs[2], [1], [3], [4] and at equal rows of the same total
    size (what raggedness costs); with cacheable and streaming K/V loads, and with the rows of a ragged batch cut into
    pieces that the last piece to arrive merges (the dispatch's choice where it applies) or left whole, one workgroup
    per (row, kv head)."""
    be = pkg.Backend()
    shapes = [("configs[2]: B64 H8 D64, 512 keys", 64, 8, 64, 512, None),
              ("configs[1]: B32 H8 D64, 1..4096 keys", 32, 8, 64, 4352, (1, 4097)),
              ("configs[1] total, equal rows: 2048 keys", 32, 8, 64, 4352, (2048, 2049)),
              ("configs[3]: B16 H16 D128, 1024..4095 keys", 16, 16, 128, 4096, (1024, 4096)),
              ("configs[3] total, equal rows: 2560 keys", 16, 16, 128, 4096, (2559, 2560)),
              ("configs[3] caches full: 4096 keys", 16, 16, 128, 4096, (4095, 4096)),
              ("configs[4] decode: B32 H16 D128, 64..2200 keys", 32, 16, 128, 4096, (64, 2200))]
    rows = []
    for (label, B, H, Dh, T, lr) in shapes:
        cache_bytes = B * T * H * Dh * 2
        nsets = max(2, int(600e6 // (2 * cache_bytes)) + 1)
        buf = be.buffer(nsets * 2 * cache_bytes + (8 << 20))
        rng = np.random.default_rng(1003)
        lens = np.full(B, T - 1, np.int32) if lr is None else rng.integers(lr[0], lr[1], B).astype(np.int32)
        sets = []
        for i in range(nsets):
            k, v = buf.alloc((B, T, H, Dh), pkg.F16), buf.alloc((B, T, H, Dh), pkg.F16)
            be.rand_uniform(k, 2 * i, -1.0, 1.0)
            be.rand_uniform(v, 2 * i + 1, -1.0, 1.0)
            sets.append((k, v))
        q = buf.from_numpy(rng.standard_normal((B, 1, H, Dh)).astype(np.float16))
        out = buf.alloc((B, 1, H, Dh), pkg.F16)
        pos = buf.from_numpy(lens)
        algo = int(np.sum(lens.astype(np.int64) + 1)) * H * Dh * 4 + 2 * B * H * Dh * 2 + 4 * B
        for pieces in (1, 0):
            for nt in ((-1, 0, 1) if pieces else (1,)):
                be.set_tunable("sdpa_merge", pieces)
                be.set_tunable("sdpa_nontemporal", nt)
                fns = [(lambda kv=kv: be.sdpa_decode_positions(q, kv[0], kv[1], pos, out, 1.0 / np.sqrt(Dh)))
                       for _ in range(3) for kv in sets]   # consecutive launches read different caches
                us = _timed(pkg, be, fns)
                rows.append({"shape": label, "streaming_loads": {-1: "auto", 0: "off", 1: "on"}[nt],
                             "ragged_rows_in_pieces": "dispatch's choice" if pieces else "off",
                             "kernel": be.sdpa_decode_last_kernel(), "us_per_launch": round(us, 2),
                             "gbs": round(algo / us / 1e3, 1), "frac_of_hbm_peak": round(algo / us / 1e3 / HBM_PEAK_GBS, 4),
                             "algorithmic_bytes": algo, "distinct_cache_sets": nsets})
        be.set_tunable("sdpa_nontemporal", -1)
        be.set_tunable("sdpa_merge", 1)
        be.free(buf)
    be.close()
    print(json.dumps({"probe": "sdpa_decode", "unit": "us per launch, stream events around graph replays",
                      "peak_gbs": HBM_PEAK_GBS, "results": rows}))


def few_row_linear(pkg, rows_list=(16, 32, 64)):
    """The five projections of a decode step of the scaled decoder (d_model 2048, hidden 5632, vocabulary 32768) with
    16 / 32 / 64 rows, through gd_backend_fused_linear / gd_backend_fused_qkv_rope_append with the step's prologues and
    epilogues; copies of the weight matrix are rotated.  Both kernel families ("linear_wide" off / automatic)."""
    be = pkg.Backend()
    buf = be.buffer(3 << 30)
    rng = np.random.default_rng(0)
    results = []

    def weights(rows, K):
        copies = max(2, int(400e6 // (rows * K * 2)) + 1)
        w0 = (rng.standard_normal((rows, K)) * 0.05).astype(np.float16)
        return [buf.from_numpy(w0) for _ in range(copies)], w0.nbytes

    for M in rows_list:
        for label, K, N, pro, epi, res_on in (("qkv + rope + append", 2048, 6144, 2, 2, False),
                                              ("attention projection + residual", 2048, 2048, 0, 0, True),
                                              ("up/gate + swiglu", 2048, 5632, 2, 1, False),
                                              ("down projection + residual", 5632, 2048, 0, 0, True),
                                              ("LM head", 2048, 32768, 2, 0, False)):
            buf.reset()
            wrows = N * (2 if epi == 1 else 1)
            ws, wbytes = weights(wrows, K)
            x = buf.from_numpy((rng.standard_normal((M, K)) * 1.2).astype(np.float16))
            b = buf.from_numpy((rng.standard_normal(wrows) * 0.3).astype(np.float16))
            nw = buf.from_numpy((1 + 0.1 * rng.standard_normal(K)).astype(np.float16))
            r = buf.from_numpy(rng.standard_normal((M, N)).astype(np.float16))
            y = buf.alloc((M, N), pkg.F16)
            if epi == 2:
                H, D, Tmax = 16, 128, 8
                pos = buf.from_numpy(rng.integers(0, 4000, M).astype(np.int32))
                cpos = buf.from_numpy(rng.integers(0, Tmax, M).astype(np.int32))
                qo = buf.alloc((M, H, D), pkg.F16)
                kc, vc = buf.alloc((M, Tmax, H, D), pkg.F16), buf.alloc((M, Tmax, H, D), pkg.F16)
            # third variant: every launch reads the same copy, which then stays in the 256 MB memory-side cache: what a
            # projection would gain if its weights had been brought there ahead of time
            for wide, resident in ((0, False), (-1, False), (-1, True)):
                be.set_tunable("linear_wide", wide)
                wl = [ws[0]] * len(ws) if resident else ws
                if epi == 2:
                    fns = [(lambda w=w: be.fused_qkv_rope_append(x, w, b, nw, pos, cpos, qo, kc, vc, H, D, 2, 2, 1e-5)) for w in wl]
                else:
                    fns = [(lambda w=w: be.fused_linear(x, w, b, r if res_on else None, nw if pro == 2 else None, y, True, 2,
                                                        pro, 1e-5, epi)) for w in wl]
                us = _timed(pkg, be, fns)
                results.append({"projection": label, "rows": M, "K": K, "N": N, "kernel_family": "stream" if wide == 0 else "wide",
                                "weights_from": "memory-side cache (one copy re-read)" if resident else "HBM (copies rotated)",
                                "us_per_launch": round(us, 2), "weight_gbs": round(wbytes / us / 1e3, 1),
                                "frac_of_hbm_peak": round(wbytes / us / 1e3 / HBM_PEAK_GBS, 4), "weight_bytes": wbytes,
                                "weight_copies_rotated": 1 if resident else len(ws)})
            be.set_tunable("linear_wide", -1)
    be.free(buf)
    be.close()
    print(json.dumps({"probe": "few_row_linear", "unit": "us per launch, stream events around graph replays",
                      "peak_gbs": HBM_PEAK_GBS, "results": results}))


def tile_gemm(pkg, launches=6):
    """gd_backend_fused_linear with 128 rows or more (the matrix-core kernel) at the prefill shapes of configs[4]
    (30,229 rows, d_model 2048, hidden 5632: qkv, attention projection + residual, up/gate + swiglu, down + residual)
    and at 8192^3.  With few launches this is also the program of the counter runs (rocprofv3 --pmc)."""
    be = pkg.Backend()
    buf = be.buffer(3 << 30)
    rng = np.random.default_rng(0)
    results = []
    timer = pkg.Timer(be)
    for label, M, K, N, epi, res_on in (("qkv", 30229, 2048, 6144, 0, False),
                                        ("attention projection + residual", 30229, 2048, 2048, 0, True),
                                        ("up/gate + swiglu", 30229, 2048, 5632, 1, False),
                                        ("down projection + residual", 30229, 5632, 2048, 0, True),
                                        ("square", 8192, 8192, 8192, 0, False)):
        buf.reset()
        wrows = N * (2 if epi == 1 else 1)
        x = buf.alloc((M, K), pkg.F16)
        w = buf.alloc((wrows, K), pkg.F16)
        be.rand_uniform(x, 1, -1.0, 1.0)
        be.rand_uniform(w, 2, -0.05, 0.05)
        b = buf.from_numpy((rng.standard_normal(wrows) * 0.3).astype(np.float16))
        r = buf.alloc((M, N), pkg.F16)
        be.rand_uniform(r, 3, -1.0, 1.0)
        y = buf.alloc((M, N), pkg.F16)
        be.scope_begin()
        call = lambda: be.fused_linear(x, w, b, r if res_on else None, None, y, True, 2, 0, 0.0, epi)
        # the first matrix work of a process runs at a lower clock than what follows (about 15 % on the first shape):
        # the chip is given some ten milliseconds of it before anything is timed
        for _ in range(12 if not results else 1):
            call()
        timer.start()
        for _ in range(launches):
            call()
        timer.stop()
        us = timer.elapsed_ms() * 1e3 / launches
        be.fence_wait(be.record_fence())
        flops = 2.0 * M * K * wrows
        results.append({"projection": label, "M": M, "K": K, "N": wrows, "us_per_launch": round(us, 1),
                        "tflops": round(flops / us / 1e6, 1), "frac_of_mfma_peak": round(flops / us / 1e6 / MFMA_F16_PEAK_TFLOPS, 4)})
    timer.close()
    be.free(buf)
    be.close()
    print(json.dumps({"probe": "tile_gemm", "unit": "us per launch (stream events)", "peak_tflops_f16_mfma": MFMA_F16_PEAK_TFLOPS,
                      "launches_per_shape": launches + 1, "results": results}))


def prefill_attention(pkg, launches=5):
    """gd_backend_sdpa_varlen (packed causal attention, 16 heads of 128, F16) over the prompt mixes of configs[3]
    (16 prompts of 1024..4095 tokens) and configs[4] (32 prompts of 64..2048 tokens), at equal lengths, and with 8
    heads of 64 (64 prompts of 511 tokens: the prefill of configs[2]).  Flops are counted on the visible
    (query, key) pairs only: 4 * D per pair and head."""
    be = pkg.Backend()
    buf = be.buffer(3 << 30)
    timer = pkg.Timer(be)
    results = []
    rng = np.random.default_rng(1004)
    for label, H, D, lens in (("configs[3] prompts: 16 x 1024..4095", 16, 128, rng.integers(1024, 4096, 16)),
                              ("configs[4] prompts: 32 x 64..2048", 16, 128, rng.integers(64, 2049, 32)),
                              ("16 x 2560 (equal lengths)", 16, 128, np.full(16, 2560)),
                              ("4 x 8192 (equal lengths)", 16, 128, np.full(4, 8192)),
                              ("configs[2] prompts: 64 x 511, 8 heads of 64", 8, 64, np.full(64, 511))):
        buf.reset()
        n = int(lens.sum())
        cu = np.zeros(len(lens) + 1, np.int32)
        cu[1:] = np.cumsum(lens)
        q, k, v, out = (buf.alloc((n, H, D), pkg.F16) for _ in range(4))
        for t, seed in ((q, 11), (k, 12), (v, 13)):
            be.rand_uniform(t, seed, -1.0, 1.0)
        tcu = buf.from_numpy(cu)
        be.scope_begin()
        call = lambda: be.sdpa_varlen(q, k, v, tcu, out, 1.0 / np.sqrt(D))
        call()
        timer.start()
        for _ in range(launches):
            call()
        timer.stop()
        us = timer.elapsed_ms() * 1e3 / launches
        be.fence_wait(be.record_fence())
        pairs = int(sum(int(t) * (int(t) + 1) // 2 for t in lens))
        flops = 4.0 * D * H * pairs
        results.append({"prompts": label, "tokens": n, "heads": H, "head_dim": D, "us_per_launch": round(us, 1),
                        "tflops_on_visible_pairs": round(flops / us / 1e6, 1),
                        "frac_of_mfma_peak": round(flops / us / 1e6 / MFMA_F16_PEAK_TFLOPS, 4)})
    timer.close()
    be.free(buf)
    be.close()
    print(json.dumps({"probe": "prefill_attention", "unit": "us per launch (stream events)",
                      "peak_tflops_f16_mfma": MFMA_F16_PEAK_TFLOPS, "results": results}))


def tile_timeline(pkg):
    """Per-tile time stamps of the prefill projection kernel (library built with TILE_TIMELINE=1): for each shape of
    tile_gemm and the up/gate + swiglu projection, microseconds in the K loop and in the epilogue per tile (mean over
    the workgroups, first full rounds of tiles) and the shader clock during the K loop (s_memtime ticks per
    nanosecond of the 100 MHz real-time counter)."""
    import ctypes
    lib = pkg.lib()
    if not hasattr(lib, "gd_hip_linear_tile_timeline"):
        raise SystemExit("this probe needs the profiling build: make -C gradients.c_amd/csrc TILE_TIMELINE=1")
    be = pkg.Backend()
    buf = be.buffer(3 << 30)
    rng = np.random.default_rng(0)
    timer = pkg.Timer(be)
    results = []
    for label, M, K, N, epi, res_on in (("qkv", 30229, 2048, 6144, 0, False),
                                        ("attention projection + residual", 30229, 2048, 2048, 0, True),
                                        ("up/gate + swiglu", 30229, 2048, 5632, 1, False),
                                        ("down projection + residual", 30229, 5632, 2048, 0, True),
                                        ("square", 8192, 8192, 8192, 0, False)):
        buf.reset()
        wrows = N * (2 if epi == 1 else 1)
        x, w = buf.alloc((M, K), pkg.F16), buf.alloc((wrows, K), pkg.F16)
        be.rand_uniform(x, 1, -1.0, 1.0)
        be.rand_uniform(w, 2, -0.05, 0.05)
        b = buf.from_numpy((rng.standard_normal(wrows) * 0.3).astype(np.float16))
        r = buf.alloc((M, N), pkg.F16)
        be.rand_uniform(r, 3, -1.0, 1.0)
        y = buf.alloc((M, N), pkg.F16)
        be.scope_begin()
        call = lambda: be.fused_linear(x, w, b, r if res_on else None, None, y, True, 2, 0, 0.0, epi)
        for _ in range(3):
            call()
        timer.start()
        call()
        timer.stop()
        us = timer.elapsed_ms() * 1e3
        be.fence_wait(be.record_fence())
        notes = np.zeros(256 * 32 * 4, np.uint64)
        rc = lib.gd_hip_linear_tile_timeline(notes.ctypes.data_as(ctypes.c_void_p))
        if rc != 0:
            raise SystemExit(f"gd_hip_linear_tile_timeline: {rc}")
        notes = notes.reshape(256, 32, 4).astype(np.int64)
        tiles = (M + 255) // 256 * ((wrows + 255) // 256)
        rounds = min(32, tiles // 256)
        k_loop = (notes[:, :rounds, 1] - notes[:, :rounds, 0]) / 100.0
        epilogue = (notes[:, :rounds, 2] - notes[:, :rounds, 1]) / 100.0
        clock = notes[:, :rounds, 3] / (k_loop * 1e3)
        k_tiles = K // 64
        results.append({"projection": label, "M": M, "K": K, "N": wrows, "launch_us": round(us, 1), "tiles": tiles,
                        "full_rounds": rounds, "k_loop_us_per_tile": round(float(k_loop.mean()), 2),
                        "epilogue_us_per_tile": round(float(epilogue.mean()), 2),
                        "shader_clock_ghz_in_k_loop": round(float(clock.mean()), 3),
                        "clocks_per_64_wide_k_tile": round(float((notes[:, :rounds, 3] / k_tiles).mean()), 0),
                        "matrix_instruction_clocks_per_k_tile": 2048})
    timer.close()
    be.free(buf)
    be.close()
    print(json.dumps({"probe": "tile_timeline", "results": results}))


PROBES = {"tile_timeline": tile_timeline, "prefill_attention": prefill_attention, "sdpa_decode": sdpa_decode, "few_row_linear": few_row_linear, "tile_gemm": tile_gemm}
