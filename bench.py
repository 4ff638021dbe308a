#!/usr/bin/env python3
"""Benchmark of the decode hot path on one MI355X.

Workload (BASELINE.json configs[2]): gpt_lm default architecture (vocab 2048, d_model 512,
3 layers, 8 heads x 64, SwiGLU hidden 1536, untied LM head), random-init F16 weights, batch 64,
every sequence's K/V cache pre-filled to 511 tokens by a real packed prefill of uniform random
token ids.  One step = the full layer stack for 64 new tokens at cache position 511 (512 keys per
sequence): embedding, rms_norm, qkv projection, qkv_split_rope, K/V append, sdpa_decode, output
projection, swiglu_split_linear, LM head, greedy argmax; the token of one step feeds the next on
the device.  The cache position is held at 511 so that every timed step has exactly this shape.
After the warm-up the K steps are timed BATCHES times (each batch bracketed by a stream
synchronisation and a host clock); the line reports the median batch.

Prints ONE JSON line: whole-job tokens/s, plus
  roofline      sdpa_decode (the dominant HBM consumer) timed alone with stream events at the same
                shape, rotating over more distinct K/V caches than the 256 MB memory-side cache holds:
                algorithmic bytes / mean launch time vs 8 TB/s;
  cpu_baseline  the CPU oracle's decoder running the same step shape on the host cores;
  others        the remaining BASELINE.json configs: configs[0] (batch 1, 32-token prompt, 64 greedy
                tokens; in a child process under the runtime's default graph replay when this process
                replays node by node), and in the same process configs[1] (isolated append + sdpa_decode, ragged),
                configs[3] (scaled decoder, B=16, long ragged caches), configs[4] (packed prefill of 32
                prompts + 128 greedy steps), each with its own roofline fraction.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth
MFMA_F16_PEAK_TFLOPS = 2500.0  # published dense F16 matrix rate
# HBM bytes per sdpa_decode launch at this shape from the FETCH_SIZE / WRITE_SIZE counter runs summarised in
# profiles/sdpa_decode_config2_pmc.md (fetch scaled by the factor a 64 MiB device copy shows in the same run); the
# kernel with cacheable loads (the one the step uses) and the one with streaming loads
SDPA_TRAFFIC_BYTES = 67333269
SDPA_TRAFFIC_BYTES_STREAMING = 67315867


# A hardware queue's ring holds 16384 dispatch packets.  rocprofv3's queue interception has ended the profiled process
# with a segmentation fault inside hipGraphLaunch whenever a graph launch wrapped around the end of that ring, so a
# profiled run must stay below it.  Unprofiled runs are not affected.
QUEUE_RING_PACKETS = 16384


def profiler_attached(env=None):
    """True when a rocprofiler tool library rides in this process (rocprofv3 sets these for the program it starts)."""
    env = os.environ if env is None else env
    if any(k.startswith(("ROCPROF_", "ROCPROFILER_", "ROCP_TOOL")) for k in env):
        return True
    return "rocprofiler" in env.get("LD_PRELOAD", "") or "rocprofiler" in env.get("HSA_TOOLS_LIB", "")


def planned_dispatches(a):
    """Upper estimate of the dispatch packets the chosen flags put on the backend's queue, as (total, parts): pure
    arithmetic on the flags.  A fused decode step is 5 launches per layer + 2; weight initialisation and a packed
    prefill are priced at 12 launches per layer + 8 each (more than either issues); a step through the public
    operators (step 0 of a resident session) at 14 per layer + 6."""
    def init(layers):
        return 12 * layers + 8

    def step(layers):
        return 5 * layers + 2

    def eager_step(layers):
        return 14 * layers + 6

    def long_context(which, steps, warmup, batches):
        if a.prefill_only:
            return init(24) + 2 * init(24)
        if which == 4:
            steps, warmup, batches = a.decode_steps, 0, 1
        return init(24) + 2 * init(24) + eager_step(24) + (warmup + steps * batches) * step(24)

    parts = {}
    if a.kernel_only:
        parts["kernel_only"] = 40
    elif a.probe:
        # graphs of at most a few dozen launches, replayed 13 times per timing (perf_probes._timed)
        parts["probe"] = {"sdpa_decode": 7 * 3 * (2 + 13) * 30, "few_row_linear": 3 * 10 * (2 + 13) * 24}.get(a.probe, 400)
    elif a.minimax_kernels:
        parts["minimax_kernels"] = 2 * (8 + 4 * (1 + 10 + 20))
    elif a.workload != 2:
        parts[f"configs[{a.workload}]"] = long_context(a.workload, a.steps, a.warmup, (a.batches or 3) if a.workload == 3 else 1)
    elif a.sampled:
        parts["sampled"] = 2 * init(3) + eager_step(3) + (a.warmup + a.steps) * (step(3) + 2)
    else:
        batches = a.batches or 5
        parts["configs[2]"] = 2 * init(3) + eager_step(3) + (a.warmup + batches * a.steps) * step(3)
        parts["roofline"] = 12 + 2 * (1 + 24 * (4 + max(1, 200 // 24)))
        if not a.headline_only:
            parts["configs[0]"] = init(3) + 6 * init(3) + 5 * (eager_step(3) + 63 * (step(3) + 1))
            parts["configs[1]"] = 8 + 2 * (2 + 24 * (2 + 120 // 12))
            parts["configs[3]"] = long_context(3, 20, 3, 3)
            parts["configs[4]"] = long_context(4, 0, 0, 1)
    return sum(parts.values()), parts


def refuse_if_profiled_run_would_wrap_the_queue(a, env=None):
    """Exits non-zero, before anything touches the GPU, when a profiler is attached and the flags would queue more
    dispatch packets than the ring holds."""
    if not profiler_attached(env):
        return
    total, parts = planned_dispatches(a)
    if total >= QUEUE_RING_PACKETS:
        sys.exit(f"bench.py: refusing to run under the profiler: these flags queue about {total} dispatch packets "
                 f"({parts}), the hardware queue's ring holds {QUEUE_RING_PACKETS}, and rocprofv3's queue interception "
                 "has crashed the profiled process (segmentation fault inside hipGraphLaunch) whenever a graph launch "
                 "wrapped around the ring's end.  Profile one workload per process with fewer steps, e.g. "
                 "--headline-only --no-cpu-baseline --batches 1, --workload 3 --steps 40 --warmup 5 --batches 1, "
                 "--workload 4 --decode-steps 80.")


def _package():
    import __graft_entry__ as entry
    return entry._package(), entry._oracle()


def sdpa_roofline(dec, D, pkg, iters=200):
    """Mean duration of one sdpa_decode launch at the step's shape, with events on the backend stream.  Consecutive
    launches read different caches (the decoder's own three layers plus five more K/V pairs of the same shape filled
    with uniform random halfs: 8 x 67 MB = 537 MB of distinct rows), so no launch can find its rows in the 256 MB
    memory-side cache or in an L2: every timed byte comes from HBM."""
    import ctypes as C
    cfg = dec.cfg
    be = dec.ctx.backend()
    B, H, Dh, T = cfg.batch, cfg.n_heads, cfg.head_dim, cfg.max_seq
    cache_bytes = B * T * H * Dh * 2
    extra = 5
    buf = be.buffer(2 * extra * cache_bytes + (8 << 20))
    rng = np.random.default_rng(1)
    q = buf.from_numpy((rng.standard_normal((B, 1, H, Dh))).astype(np.float16))
    out = buf.alloc((B, 1, H, Dh), pkg.F16)
    pos = buf.from_numpy(np.full(B, T - 1, np.int32))
    sets = [(D.view_of(dec.tensor("k_cache", l)), D.view_of(dec.tensor("v_cache", l))) for l in range(cfg.n_layers)]
    for e in range(extra):
        k, v = buf.alloc((B, T, H, Dh), pkg.F16), buf.alloc((B, T, H, Dh), pkg.F16)
        be.rand_uniform(k, 900 + 2 * e, -1.0, 1.0)
        be.rand_uniform(v, 901 + 2 * e, -1.0, 1.0)
        sets.append((k.view(), v.view()))
    args = pkg.SdpaDecodeArgs(1.0 / np.sqrt(Dh), cfg.sdpa_window, 0, 0)

    def launch(i):
        kv, vv = sets[i % len(sets)]
        st = be.call("gd_backend_sdpa_decode_positions", q.view(), kv, vv, pos.view(), out.view(), C.byref(args))
        assert st == 0, st

    # launches are captured into a graph and replayed so that the host's per-call cost (python + ctypes,
    # ~15 us) does not sit between kernels; events are recorded on the backend's own stream
    per_graph = 3 * len(sets)
    timer = pkg.Timer(be)

    def measure():
        be.scope_begin()
        launch(0)
        name = be.sdpa_decode_last_kernel()
        be.graph_begin_capture()
        for i in range(per_graph):
            launch(i)
        graph = be.graph_end_capture()
        for _ in range(3):
            be.graph_launch(graph)
        replays = max(1, iters // per_graph)
        timer.start()
        for _ in range(replays):
            be.graph_launch(graph)
        timer.stop()
        ms = timer.elapsed_ms()
        be.fence_wait(be.record_fence())
        be.graph_destroy(graph)
        return name, ms / 1e3 / (replays * per_graph), replays * per_graph

    kernel, sec, iters = measure()
    # the same launches with the K/V loads marked streaming (what the dispatch chooses by itself for caches too large
    # to survive in the memory-side cache between steps): reported next to the figure of the kernel the step uses
    be.set_tunable("sdpa_nontemporal", 1)
    try:
        kernel_nt, sec_nt, _ = measure()
    finally:
        be.set_tunable("sdpa_nontemporal", -1)
    timer.close()
    be.free(buf)
    keys = min(T, cfg.sdpa_window) if cfg.sdpa_window > 0 else T
    algo_bytes = B * keys * H * Dh * 2 * 2 + 2 * B * H * Dh * 2 + 4 * B
    gbs = algo_bytes / sec / 1e9
    return {"bound": "hbm", "kernel": kernel, "achieved": round(gbs, 1),
            "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
            "traffic": SDPA_TRAFFIC_BYTES, "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of the same "
            "launch (profiles/sdpa_decode_config2_pmc.md), not re-measured in this run",
            "algorithmic_bytes_per_launch": algo_bytes, "us_per_launch": round(sec * 1e6, 3), "launches": iters,
            "distinct_cache_bytes_rotated": len(sets) * 2 * cache_bytes,
            "with_streaming_loads": {"kernel": kernel_nt, "us_per_launch": round(sec_nt * 1e6, 3),
                                     "achieved": round(algo_bytes / sec_nt / 1e9, 1),
                                     "frac": round(algo_bytes / sec_nt / 1e9 / HBM_PEAK_GBS, 4),
                                     "traffic": SDPA_TRAFFIC_BYTES_STREAMING,
                                     "traffic_source": "counter runs of this kernel in the same profile"}}


def kernel_only(pkg, launches=20, copy_mib=64):
    """For counter collection (rocprofv3 --pmc): the sdpa_decode launch of the benchmark shape on
    pattern-filled caches, followed by device copies of a known size whose counters calibrate the
    units of FETCH_SIZE / WRITE_SIZE."""
    import ctypes as C
    be = pkg.Backend()
    B, H, Dh, T = 64, 8, 64, 512
    buf = be.buffer(256 << 20)
    k, v = buf.alloc((B, T, H, Dh), pkg.F16), buf.alloc((B, T, H, Dh), pkg.F16)
    be.fill(k, 0x3400)
    be.fill(v, 0x3800)
    rng = np.random.default_rng(1)
    q = buf.from_numpy(rng.standard_normal((B, 1, H, Dh)).astype(np.float16))
    out = buf.alloc((B, 1, H, Dh), pkg.F16)
    pos = buf.from_numpy(np.full(B, T - 1, np.int32))
    args = pkg.SdpaDecodeArgs(0.125, 0, 0, 0)
    src, dst = buf.alloc((copy_mib << 20,), pkg.U8), buf.alloc((copy_mib << 20,), pkg.U8)
    be.fill(src, 0x11)
    be.scope_begin()
    for _ in range(launches):
        assert be.call("gd_backend_sdpa_decode_positions", q.view(), k.view(), v.view(), pos.view(), out.view(),
                       C.byref(args)) == 0
    for _ in range(5):
        assert pkg.lib().gd_backend_copy(be.handle, dst.buffer.handle, dst.offset, src.buffer.handle, src.offset,
                                         src.nbytes) == 0
    be.fence_wait(be.record_fence())
    print(json.dumps({"kernel_only": "gd_sdpa_decode_split_kernel", "launches": launches,
                      "algorithmic_bytes_per_launch": B * T * H * Dh * 4 + 2 * B * H * Dh * 2 + 4 * B,
                      "calibration_copy_bytes": copy_mib << 20, "calibration_copies": 5}))
    be.close()


def cpu_baseline(oracle, cfg_tuple, budget_s=12.0, max_steps=64):
    """The CPU oracle's decoder on the same step shape: caches filled to 511 rows with random F16 rows
    (a CPU prefill of 32k tokens would take minutes), then whole decode steps until the budget is used."""
    vocab, d_model, layers, heads, head_dim, hidden, max_seq, batch = cfg_tuple
    ref = oracle.Decoder(vocab, d_model, layers, heads, head_dim, hidden, max_seq, batch, 0, 1002, False)
    for l in range(layers):
        ref.tensor("k_cache", l)[:] = oracle.normal_f16((batch, max_seq, heads, head_dim), 7000 + l, 0.5)
        ref.tensor("v_cache", l)[:] = oracle.normal_f16((batch, max_seq, heads, head_dim), 7100 + l, 0.5)
    ids = oracle.uniform_i32(batch, 7200, 0, vocab - 1)
    steps, t0 = 0, time.perf_counter()
    while steps < max_steps and (steps == 0 or time.perf_counter() - t0 < budget_s):
        ref.positions[:] = max_seq - 1
        _, ids, _ = ref.step(ids)
        steps += 1
    dt = time.perf_counter() - t0
    ref.close()
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    return {"value": round(batch * steps / dt, 2), "unit": "tokens/s", "cores": threads, "kind": "port",
            "sample": f"{steps} whole decode steps of the same shape (B={batch}, 511-row caches filled with random "
                      f"F16 rows instead of a CPU prefill), {dt:.1f} s, oracle/gd_oracle.c with OpenMP"}


C3_ARCH = (32768, 2048, 24, 16, 128, 5632)  # vocab, d_model, layers, heads, head_dim, mlp_hidden (configs[3], [4])


def _event_ms(pkg, be, fn):
    """Stream-event time of fn() (which only enqueues) on the backend stream."""
    timer = pkg.Timer(be)
    timer.start()
    fn()
    timer.stop()
    ms = timer.elapsed_ms()
    timer.close()
    return ms


def _median(values):
    v = sorted(values)
    return v[len(v) // 2]


def config0_batch1(oracle, D, new_tokens=64, prompt_len=32):
    """configs[0] on the device: batch 1, 32-token prompt, 64 greedy tokens with the K/V cache.  A batch-1 step
    reads every weight once for one row (the projections are matrix-vector products): it is priced on weight
    bytes per step against the HBM peak.  The reference's generator reports prompts x generated / elapsed with the
    clock started before the prefill (gpt_lm_shared.c:1696-1707): that figure is end_to_end_tokens_per_s."""
    V, Dm, L, H, Dh, Hm = 2048, 512, 3, 8, 64, 1536
    dec = D.GptDecoder(D.gpt_config(V, Dm, L, H, Dh, Hm, 128, 1, window=0, tie_lm_head=False, seed=1000),
                       max_prefill_tokens=prompt_len)
    prompt = oracle.uniform_i32(prompt_len, 1000, 0, V - 1)
    dec.prefill(prompt, [0, prompt_len], want_logits=False)  # first call: code objects load here, not in the clock
    dec.positions[:] = 0
    runs = []
    for _ in range(5):
        dec.positions[:] = 0
        t0 = time.perf_counter()
        _, first, _ = dec.prefill(prompt, [0, prompt_len], want_logits=False)
        dec.resident_begin(first, new_tokens)       # step 0 eagerly + capture of the step graph
        t1 = time.perf_counter()
        dec.resident_run(new_tokens - 1)
        dec.resident_sync()
        t2 = time.perf_counter()
        ids, _ = dec.resident_end()
        assert ids.shape == (new_tokens, 1) and ids.min() >= 0 and ids.max() < V
        runs.append((t2 - t0, (t2 - t1) / (new_tokens - 1)))
    dec.close()
    total_s, step_s = _median([r[0] for r in runs]), _median([r[1] for r in runs])
    weight_bytes = 2 * (L * (Dm * 3 * Dm + Dm * Dm + Dm * 2 * Hm + Hm * Dm) + V * Dm + Dm)  # + one embedding row
    gbs = weight_bytes / step_s / 1e9
    return {"workload": "configs[0]: gpt_lm default decoder, batch 1, 32-token prompt of uniform random ids, 64 greedy "
                        "tokens with the K/V cache (device-resident loop)",
            "tokens_per_s": round(1.0 / step_s, 1), "us_per_step": round(step_s * 1e6, 2),
            "end_to_end_tokens_per_s": round(new_tokens / total_s, 1),
            "end_to_end_note": "prefill + first step + graph capture + 63 replays inside the clock",
            "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(gbs / HBM_PEAK_GBS, 4), "algorithmic_bytes_per_step": weight_bytes,
                         "note": "weight bytes per step / step time; 18 dependent launches on 22.6 MB: launch-latency "
                                 "bound, the weights stay in the memory-side cache"}}


def config1_append_decode(pkg, iters=120):
    """configs[1]: isolated K/V append + sdpa_decode, B=32, H=8, DH=64, F16, cache lengths uniform in [1,4096]; one
    token is appended per sequence at its length, then the decode attends over length + 1 keys.  Three cache sets
    are rotated (3 x 134 MB of live rows), times from stream events around graph replays."""
    import ctypes as C
    be = pkg.Backend()
    B, H, Dh, T = 32, 8, 64, 4352
    rng = np.random.default_rng(1001)
    lens = rng.integers(1, 4097, B).astype(np.int32)
    nsets = 3
    buf = be.buffer(nsets * 2 * B * T * H * Dh * 2 + (16 << 20))
    sets = []
    for i in range(nsets):
        k, v = buf.alloc((B, T, H, Dh), pkg.F16), buf.alloc((B, T, H, Dh), pkg.F16)
        be.rand_uniform(k, 700 + 2 * i, -1.0, 1.0)
        be.rand_uniform(v, 701 + 2 * i, -1.0, 1.0)
        sets.append((k, v))
    q = buf.from_numpy(rng.standard_normal((B, 1, H, Dh)).astype(np.float16))
    kn = buf.from_numpy(rng.standard_normal((B, 1, H, Dh)).astype(np.float16))
    vn = buf.from_numpy(rng.standard_normal((B, 1, H, Dh)).astype(np.float16))
    out = buf.alloc((B, 1, H, Dh), pkg.F16)
    pos = buf.from_numpy(lens)
    scale = 1.0 / np.sqrt(Dh)
    timer = pkg.Timer(be)

    def timed(fn, per_graph):
        be.scope_begin()    # recording the fence below closes the scope again
        fn(0)
        be.graph_begin_capture()
        for i in range(per_graph):
            fn(i)
        graph = be.graph_end_capture()
        be.graph_launch(graph)
        replays = max(1, iters // per_graph)
        timer.start()
        for _ in range(replays):
            be.graph_launch(graph)
        timer.stop()
        ms = timer.elapsed_ms()
        be.fence_wait(be.record_fence())
        be.graph_destroy(graph)
        return ms * 1e3 / (replays * per_graph)

    def pair(i):
        k, v = sets[i % nsets]
        be.kv_cache_append_positions(k, v, pos, kn, vn)
        be.sdpa_decode_positions(q, k, v, pos, out, scale)

    def decode_only(i):
        k, v = sets[i % nsets]
        be.sdpa_decode_positions(q, k, v, pos, out, scale)

    pair_us = timed(pair, 4 * nsets)
    decode_us = timed(decode_only, 4 * nsets)
    kernel = be.sdpa_decode_last_kernel()
    timer.close()
    be.free(buf)
    be.close()
    row = H * Dh * 2
    decode_bytes = int(np.sum(lens.astype(np.int64) + 1)) * row * 2 + 2 * B * row + 4 * B
    append_bytes = 4 * B * row + 4 * B
    gbs_pair = (decode_bytes + append_bytes) / pair_us / 1e3
    gbs_dec = decode_bytes / decode_us / 1e3
    return {"workload": "configs[1]: isolated K/V append + sdpa_decode, B=32, H=8, DH=64, F16, cache lengths uniform "
                        "in [1,4096], one token appended per sequence",
            "us_per_append_plus_decode": round(pair_us, 2), "us_per_decode": round(decode_us, 2),
            "cached_tokens": int(lens.sum()), "kernel": kernel,
            "roofline": {"bound": "hbm", "achieved": round(gbs_pair, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(gbs_pair / HBM_PEAK_GBS, 4), "algorithmic_bytes": decode_bytes + append_bytes,
                         "decode_alone_gbs": round(gbs_dec, 1), "decode_alone_frac": round(gbs_dec / HBM_PEAK_GBS, 4)}}


def long_context_workload(a, oracle, D, which, steps=None, warmup=None, batches=1):
    """configs[3]: B=16 sequences with 1024..4095 cached tokens (built by a real packed prefill), decode steps
    with the positions held; configs[4]: 32 prompts of 64..2048 tokens, packed prefill, then 128 greedy steps with
    growing caches (the reference generator's tok/s = prompts x generated / elapsed, clock started before prefill).
    Returns the JSON object of the workload (None after --prefill-only, which prints its own line)."""
    vocab, d_model, layers, heads, head_dim, hidden = C3_ARCH
    B, T = (16, 4096) if which == 3 else (32, 4096)
    rng = np.random.default_rng(1003 if which == 3 else 1004)
    lens = rng.integers(1024, 4096, B) if which == 3 else rng.integers(64, 2049, B)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    n_tokens = int(cu[-1])
    cfg = D.gpt_config(vocab, d_model, layers, heads, head_dim, hidden, T, B, window=0, tie_lm_head=False,
                       seed=1000 + which)
    t0 = time.perf_counter()
    dec = D.GptDecoder(cfg, max_prefill_tokens=n_tokens)
    init_s = time.perf_counter() - t0
    prompt = oracle.uniform_i32(n_tokens, 1000 + which, 0, vocab - 1)
    # one untimed pass first: the first tens of milliseconds of matrix work in a process run at a lower clock
    # (about 15 % on the first projections); the pass fills the same cache rows with the same values
    dec.prefill(prompt, cu, want_logits=False)
    t0 = time.perf_counter()
    _, first, _ = dec.prefill(prompt, cu, want_logits=False)
    prefill_s = time.perf_counter() - t0
    dense_flops = 2.0 * n_tokens * layers * (d_model * 3 * d_model + d_model * d_model + d_model * 2 * hidden + hidden * d_model)
    attn_flops = 4.0 * head_dim * heads * layers * float(np.sum(lens.astype(np.float64) * (lens + 1) / 2))
    prefill_tflops = (dense_flops + attn_flops) / prefill_s / 1e12
    if a.prefill_only:
        dec.close()
        print(json.dumps({"prefill_only": f"configs[{which}]", "prompt_tokens": n_tokens, "prefill_seconds": round(prefill_s, 4),
                          "prefill_tokens_per_s": round(n_tokens / prefill_s, 1),
                          "prefill_tflops": round(prefill_tflops, 1)}))
        return None
    steps = (a.steps if steps is None else steps) if which == 3 else a.decode_steps
    warmup = (a.warmup if warmup is None else warmup) if which == 3 else 0
    batches = batches if which == 3 else 1
    total = warmup + steps * batches
    t0 = time.perf_counter()
    dec.resident_begin(first, total + 1, hold_positions=(which == 3))
    times = []
    if which == 3:
        dec.resident_run(warmup)
        dec.resident_sync()
    for _ in range(batches):
        if which == 3:
            t0 = time.perf_counter()    # configs[4] keeps the session set-up inside its one clock
        # configs[4]: the session's first step ran inside resident_begin, so steps - 1 replays complete its `steps` steps
        dec.resident_run(steps if which == 3 else steps - 1)
        dec.resident_sync()
        times.append(time.perf_counter() - t0)
    elapsed = _median(times)
    ids, _ = dec.resident_end()
    assert ids.min() >= 0 and ids.max() < vocab
    dec.close()
    weight_bytes = 2.0 * (layers * (d_model * 3 * d_model + d_model * d_model + d_model * 2 * hidden + hidden * d_model) + vocab * d_model)
    if which == 3:
        kv_bytes = float(np.sum(np.minimum(lens + 1, T))) * heads * head_dim * 2 * 2 * layers
    else:  # caches grow by one row per step: mean over the 128 steps
        kv_bytes = float(np.sum(lens + 1 + (steps - 1) / 2.0)) * heads * head_dim * 2 * 2 * layers
    floor_ms = (kv_bytes + weight_bytes) / 8e12 * 1e3
    ms_per_step = elapsed * 1e3 / steps
    out = {
        "workload": f"configs[{which}]: scaled decoder (V32768 Dm2048 L24 H16 Dh128 Hm5632, untied head), "
                    + ("B=16, caches of 1024..4095 tokens built by packed prefill, positions held"
                       if which == 3 else
                       f"32 prompts of 64..2048 tokens, packed prefill then {steps} greedy steps with growing caches"),
        "decode_tokens_per_s": round(B * steps / elapsed, 1), "ms_per_step": round(ms_per_step, 5),
        "steps": steps, "warmup": warmup, "batches": batches, "batch": B, "prompt_tokens": n_tokens,
        "prefill_seconds": round(prefill_s, 4), "prefill_tokens_per_s": round(n_tokens / prefill_s, 1),
        "prefill_tflops": round(prefill_tflops, 1), "prefill_warmup_passes": 1, "weight_init_seconds": round(init_s, 1),
        "step_hbm_floor_ms": round(floor_ms, 4),
        "roofline": {"bound": "hbm", "achieved": round((kv_bytes + weight_bytes) / (ms_per_step / 1e3) / 1e9, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(floor_ms / ms_per_step, 4),
                     "algorithmic_bytes_per_step": int(kv_bytes + weight_bytes),
                     "note": "whole decode step: every weight and every live cache row once per step"},
    }
    if which == 4:
        out["end_to_end_tokens_per_s"] = round(B * steps / (elapsed + prefill_s), 1)
        out["decode_note"] = f"first step, graph capture and {steps - 1} replays inside the decode clock"
        out["prefill_roofline"] = {"bound": "mfma", "achieved": round(prefill_tflops, 1), "peak": MFMA_F16_PEAK_TFLOPS,
                                   "unit": "TFLOP/s", "frac": round(prefill_tflops / MFMA_F16_PEAK_TFLOPS, 4),
                                   "note": "projection + visible-pair attention flops over the whole prefill call "
                                           "(host clock, uploads and elementwise kernels included)"}
    return out


def long_context_line(a, obj, which):
    """The stand-alone line of --workload 3|4."""
    return {"metric": f"decode tokens/sec at B={obj['batch']}", "value": obj["decode_tokens_per_s"], "unit": "tokens/s",
            "n_gpus": 1, "steps": obj["steps"], "warmup": obj["warmup"], "ms_per_step": obj["ms_per_step"],
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
            "config": {k: v for k, v in obj.items() if k not in ("roofline", "prefill_roofline")},
            "roofline": obj["roofline"], "cpu_baseline": None}


def minimax_kernels(pkg, reps=10):
    """gd_backend_minimax_m3_index_topk and gd_backend_minimax_m3_sparse_attention at the reference's M3 settings
    (block 128, head size 64, first and last block forced) on packed sequences of uniform random values: the lists
    the picker makes from such data differ from row to row (the worst case for the attention, which walks the union
    of the lists of 128 rows), so the attention is also timed on lists that neighbouring rows share (first block, own
    block and the blocks before it).  Dense causal attention over the same tensors for comparison.  Times per launch
    from stream events around graph replays."""
    be = pkg.Backend()
    arena = be.buffer(1 << 30)
    be.scope_begin()
    tm = pkg.Timer(be)
    results = []
    for (B, T, H, topk) in ((8, 4096, 8, 4), (2, 16384, 8, 4)):
        Dh, block = 64, 128
        arena._top = 0
        N = B * T
        cu = arena.from_numpy((np.arange(B + 1) * T).astype(np.int32))
        q, k, v, out = (arena.alloc((N, H, Dh), pkg.F16) for _ in range(4))
        for n, t in enumerate((q, k, v)):
            be.rand_uniform(t, 10 + n, -1.0, 1.0)
        idx = arena.alloc((H, N, topk), pkg.I32)

        def timed(fn):
            fn()
            be.graph_begin_capture()
            for _ in range(reps):
                fn()
            graph = be.graph_end_capture()
            ms = 0.0
            for _ in range(2):
                tm.start()
                be.graph_launch(graph)
                tm.stop()
                ms = tm.elapsed_ms()
            return ms * 1e3 / reps

        pick = timed(lambda: be.minimax_m3_index_topk(q, k, cu, idx, block, 1, 1, max_seqlen=T))
        attn = timed(lambda: be.minimax_m3_sparse_attention(q, k, v, cu, idx, out, block, 0.125, max_seqlen=T))
        own = np.arange(T) // block
        shared = np.stack([np.zeros(T, np.int64), own, own - 1, own - 2], 1)[:, :topk]
        shared[:, 1:][shared[:, 1:] <= 0] = -1          # block 0 is listed once; nothing in front of the sequence
        idx.write(np.tile(shared[None, None], (H, B, 1, 1)).reshape(H, N, topk).astype(np.int32))
        attn_shared = timed(lambda: be.minimax_m3_sparse_attention(q, k, v, cu, idx, out, block, 0.125, max_seqlen=T))
        dense = timed(lambda: be.sdpa_varlen(q, k, v, cu, out, 0.125, True, 0, 0, T))
        pairs = B * H * (T * (T + 1) // 2)
        results.append({"sequences": B, "tokens_each": T, "heads": H, "head_dim": Dh, "block": block, "topk": topk,
                        "picker_us": round(pick, 1), "picker_tflops": round(2 * Dh * pairs / pick / 1e6, 1),
                        "sparse_attention_random_lists_us": round(attn, 1),
                        "sparse_attention_shared_lists_us": round(attn_shared, 1),
                        "dense_causal_attention_us": round(dense, 1),
                        "dense_tflops": round(4 * Dh * pairs / dense / 1e6, 1)})
    be.close()
    print(json.dumps({"metric": "MiniMax-M3 prefill attention kernels, time per launch", "unit": "us", "dtype": "f16",
                      "data": "synthetic", "peak_tflops_f16_mfma": 2500.0, "results": results}))


def sampled_workload(a, oracle, D):
    """The headline step (B=64, 511 cached tokens, positions held) with gd_backend_sample_advance after the LM head.
    Cache rows are allocated for 1024 tokens so that the rows' histories (prompt + sampled tokens, which the
    repetition penalty scans) can grow for the length of the run; attention still covers 512 keys per step."""
    B, T, cap = 64, 512, 1024
    total = a.warmup + a.steps
    if T - 1 + total + 2 > cap:
        sys.exit("--sampled: warmup + steps must stay below 510")
    dec = D.GptDecoder(D.gpt_config(2048, 512, 3, 8, 64, 1536, cap, B, window=0, tie_lm_head=False, seed=1002),
                       max_prefill_tokens=B * (T - 1))
    prompt = oracle.uniform_i32(B * (T - 1), 1002, 0, 2047)
    cu = (np.arange(B + 1) * (T - 1)).astype(np.int32)
    dec.prefill(prompt, cu, want_logits=False)
    dec.resident_begin_sampled(prompt, cu, total + 2, temperature=0.8, min_p=0.05, repetition_penalty=1.3,
                               logits_softcap=20.0, stop_token=-1, rng_state=1002, hold_positions=True)
    dec.resident_run(a.warmup)
    dec.resident_sync()
    t0 = time.perf_counter()
    dec.resident_run(a.steps)
    dec.resident_sync()
    elapsed = time.perf_counter() - t0
    ids, _ = dec.resident_end()
    assert ids.shape == (total + 2, B) and ids.min() >= 0 and ids.max() < 2048
    distinct = len(np.unique(ids))
    dec.close()
    print(json.dumps({
        "metric": "decode tokens/sec at B=64", "value": round(B * a.steps / elapsed, 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(elapsed * 1e3 / a.steps, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "configs[2] with the sampling front end: gpt_lm default decoder (V2048 Dm512 L3 H8 Dh64 "
                               "Hm1536, untied head), B=64, 511 cached tokens, soft cap 20 + repetition penalty 1.3 + "
                               "temperature 0.8 + min-p 0.05 drawn on the device, device-resident token feedback",
                   "batch": B, "cache_tokens": T, "sdpa_window": 0, "distinct_tokens_drawn": distinct},
        "roofline": None, "cpu_baseline": None,
    }))


def config0_in_a_process_of_its_own():
    """configs[0] under the HIP runtime's default graph replay.  How graphs are replayed is decided once per process, when
    the runtime starts; node by node (what the rest of this run uses) the host spends 4.4 us per kernel, more than a
    batch-1 step of the small decoder gives it.  A batch-1 server would leave the runtime's default, so that is what its
    figure is measured under: a child process, started before this one has touched the GPU."""
    import subprocess
    env = {k: v for k, v in os.environ.items() if k not in ("GD_HIP_GRAPH_NODE_REPLAY", "DEBUG_CLR_GRAPH_PACKET_CAPTURE")}
    r = subprocess.run([sys.executable, os.path.abspath(__file__), "--config0-only", "--graph-replay", "runtime"],
                       capture_output=True, text=True, timeout=600, env=env)
    if r.returncode != 0:
        raise RuntimeError(f"child process ended with {r.returncode}: {r.stderr[-300:]}")
    obj = json.loads(r.stdout.strip().splitlines()[-1])
    obj["graph_replay"] = "runtime default, in a process of its own"
    return obj


def build_parser():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--graph-replay", choices=("nodes", "runtime"), default="nodes",
                    help="how the HIP runtime replays the captured decode step: node by node through its usual launch "
                         "path (GD_HIP_GRAPH_NODE_REPLAY=1, default here) or its own default (recorded dispatch packets)")
    ap.add_argument("--batches", type=int, default=0,
                    help="how many times the K steps are timed (the median batch is reported); default 5 for the headline "
                         "line, 3 for --workload 3.  Kernel traces use --batches 1: a profiled run that would "
                         "queue more dispatch packets than a hardware queue's ring holds is refused (QUEUE_RING_PACKETS)")
    ap.add_argument("--decode-steps", type=int, default=128,
                    help="--workload 4: greedy steps after the prefill (BASELINE: 128; fewer for kernel traces, see --batches)")
    ap.add_argument("--config0-only", action="store_true",
                    help="measure configs[0] (batch 1) alone and print its object; the default run starts this in a "
                         "process of its own under the runtime's default graph replay, which suits a batch-1 step")
    ap.add_argument("--headline-only", action="store_true",
                    help="skip the other BASELINE.json configs (the 'others' object of the line)")
    ap.add_argument("--workload", type=int, default=2, choices=(2, 3, 4),
                    help="BASELINE.json configs index: 2 = the headline line (default, which also carries configs 0, 1, 3 "
                         "and 4 in its 'others' object); 3, 4 = only the scaled-decoder workload, as a line of its own")
    ap.add_argument("--prefill-only", action="store_true",
                    help="with --workload 3 or 4: stop after the packed prefill (for kernel traces of the prefill kernels)")
    ap.add_argument("--sampled", action="store_true",
                    help="the headline step with the sampling front end (soft cap 20, repetition penalty 1.3, "
                         "temperature 0.8, min-p 0.05) in place of the greedy pick; reported without roofline / "
                         "cpu_baseline objects")
    ap.add_argument("--minimax-kernels", action="store_true",
                    help="time the MiniMax-M3 block picker and block-sparse attention next to dense causal attention on "
                         "packed sequences (auxiliary: prints its own JSON line, not the headline metric)")
    ap.add_argument("--probe", choices=("sdpa_decode", "few_row_linear", "tile_gemm", "tile_timeline", "prefill_attention"),
                    help="operator-local performance probe (gradients.c_amd/perf_probes.py): one operator at the shapes of "
                         "the BASELINE.json configurations, operands rotating through HBM; prints its own JSON line")
    ap.add_argument("--kernel-only", action="store_true",
                    help="only launch sdpa_decode at the benchmark shape plus calibration copies (for --pmc runs)")
    return ap


def main():
    a = build_parser().parse_args()
    if a.gpus != 1:
        sys.exit("bench.py measures one GPU: the decode path holds every sequence, its K/V cache and a full "
                 "weight replica on a single device (sequences are independent, so more GPUs would only add "
                 "replicas); run with --gpus 1")
    refuse_if_profiled_run_would_wrap_the_queue(a)
    # graphs replayed node by node (the library's GD_HIP_GRAPH_NODE_REPLAY=1: it sets the HIP runtime's
    # DEBUG_CLR_GRAPH_PACKET_CAPTURE=0 in front of the first HIP call): +3.3 % on the 17-kernel step of the headline,
    # nothing at the 24-layer decoders, -11 % on the batch-1 step.  --graph-replay runtime keeps the runtime's default.
    config0 = None
    if (a.graph_replay == "nodes" and a.workload == 2 and not profiler_attached() and
            not (a.headline_only or a.config0_only or a.kernel_only or a.probe or a.minimax_kernels or a.sampled)):
        try:
            config0 = config0_in_a_process_of_its_own()
        except Exception as e:  # measured in this process instead, below
            print(f"bench.py: configs[0] in a process of its own failed ({type(e).__name__}: {e})", file=sys.stderr)
    if a.graph_replay == "nodes":
        os.environ.setdefault("GD_HIP_GRAPH_NODE_REPLAY", "1")
    pkg, oracle = _package()
    pkg.lib()
    if a.kernel_only:
        kernel_only(pkg)
        return
    if a.probe:
        from gradients_c_amd import perf_probes
        if a.probe == "tile_gemm":
            perf_probes.tile_gemm(pkg, launches=max(1, min(a.steps, 6)))
        else:
            perf_probes.PROBES[a.probe](pkg)
        return
    if a.minimax_kernels:
        minimax_kernels(pkg)
        return
    from gradients_c_amd import decoder as D
    if a.config0_only:
        print(json.dumps(config0_batch1(oracle, D)))
        return
    if a.workload != 2:
        obj = long_context_workload(a, oracle, D, a.workload, batches=(a.batches or 3) if a.workload == 3 else 1)
        if obj is not None:
            print(json.dumps(long_context_line(a, obj, a.workload)))
        return

    if a.sampled:
        sampled_workload(a, oracle, D)
        return

    B, T = 64, 512
    batches = a.batches or 5
    shape = (2048, 512, 3, 8, 64, 1536, T, B)
    cfg = D.gpt_config(*shape, window=0, tie_lm_head=False, seed=1002)
    dec = D.GptDecoder(cfg, max_prefill_tokens=B * (T - 1))
    prompt = oracle.uniform_i32(B * (T - 1), 1002, 0, 2047)
    cu = (np.arange(B + 1) * (T - 1)).astype(np.int32)
    t0 = time.perf_counter()
    _, first, _ = dec.prefill(prompt, cu, want_logits=False)
    prefill_s = time.perf_counter() - t0

    total = a.warmup + batches * a.steps
    dec.resident_begin(first, total + 1, hold_positions=True)  # step 0 runs eagerly inside begin
    dec.resident_run(a.warmup)
    dec.resident_sync()
    times = []
    for _ in range(batches):
        t0 = time.perf_counter()
        dec.resident_run(a.steps)
        dec.resident_sync()
        times.append(time.perf_counter() - t0)
    elapsed = _median(times)
    ids, gaps = dec.resident_end()
    assert ids.shape == (total + 1, B) and ids.min() >= 0 and ids.max() < 2048

    roof = sdpa_roofline(dec, D, pkg)
    dec.close()

    others = None
    if not a.headline_only:
        others = {}
        for name, fn in (("configs[0]", lambda: config0 if config0 is not None else config0_batch1(oracle, D)),
                         ("configs[1]", lambda: config1_append_decode(pkg)),
                         ("configs[3]", lambda: long_context_workload(a, oracle, D, 3, steps=20, warmup=3, batches=3)),
                         ("configs[4]", lambda: long_context_workload(a, oracle, D, 4))):
            try:
                others[name] = fn()
            except Exception as e:  # the headline line must survive a failing secondary workload; the error is reported
                others[name] = {"error": f"{type(e).__name__}: {e}"}
                print(f"bench.py: {name} failed: {type(e).__name__}: {e}", file=sys.stderr)
    cpu = None if a.no_cpu_baseline else cpu_baseline(oracle, shape)

    ms_per_step = elapsed * 1e3 / a.steps
    line = {
        "metric": "decode tokens/sec at B=64", "value": round(B * a.steps / elapsed, 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "configs[2]: gpt_lm default decoder (V2048 Dm512 L3 H8 Dh64 Hm1536, untied head), "
                               "batched decode step B=64, caches pre-filled to 511 tokens by packed prefill of "
                               "uniform random ids, full stack incl. greedy argmax, device-resident token feedback",
                   "batch": B, "cache_tokens": T, "sdpa_window": 0, "prefill_seconds": round(prefill_s, 3),
                   "timed_batches": batches, "reported": "median batch",
                   "graph_replay": "node by node (GD_HIP_GRAPH_NODE_REPLAY=1)" if os.environ.get("GD_HIP_GRAPH_NODE_REPLAY") == "1"
                                   else "runtime default",
                   "ms_per_step_of_each_batch": [round(t * 1e3 / a.steps, 5) for t in times]},
        "roofline": roof, "cpu_baseline": cpu, "others": others,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
    # The line is out: leave without the interpreter's and the HIP runtime's teardown, whose order at process exit is
    # not ours to control (one small program of this repository once ended with SIGSEGV after its work was done).  Not
    # under a profiler, which writes its traces at exit.
    sys.stdout.flush()
    sys.stderr.flush()
    if not profiler_attached():
        os._exit(0)
