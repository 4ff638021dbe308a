"""End-to-end parity of the C decoder (public gd_* operators over the HIP backend) against the CPU
oracle decoder on identical seeded weights and inputs.

Bars: greedy token ids identical over 64 steps except reported near-ties (top-2 logit gap < 1e-3,
BASELINE.json north_star); logits within rtol 2e-3 / atol 1e-3 scaled by the accumulated depth; caches
compared row by row.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _pair(gda, oracle, batch, window=0, tie=True, max_seq=128, layers=3, hidden=1536, seed=1000):
    from gradients_c_amd import decoder as D
    cfg = D.gpt_config(2048, 512, layers, 8, 64, hidden, max_seq, batch, window, tie, seed)
    dev = D.GptDecoder(cfg, max_prefill_tokens=batch * max_seq)
    ref = oracle.Decoder(2048, 512, layers, 8, 64, hidden, max_seq, batch, window, seed, tie)
    return dev, ref


def _assert_ids(dev_ids, ref_ids, dev_gap, ref_gap, where):
    """ids equal, or the row is a near-tie in either implementation"""
    bad = [(int(i), float(dev_gap[i]), float(ref_gap[i])) for i in np.nonzero(dev_ids != ref_ids)[0]
           if min(dev_gap[i], ref_gap[i]) >= 1e-3]
    assert not bad, f"{where}: token mismatch that is not a near-tie: {bad}"
    return int(np.count_nonzero(dev_ids != ref_ids))


def test_weights_match_oracle_bit_for_bit(gda, oracle):
    dev, ref = _pair(gda, oracle, 1)
    try:
        for name in ("embed", "final_norm", "lm_bias"):
            assert np.array_equal(dev.read_tensor(name).view(np.uint16), ref.tensor(name).view(np.uint16)), name
        for layer in (0, 2):
            for name in ("attn_norm", "w_qkv", "b_qkv", "w_attn", "w_upgate", "w_down", "b_down"):
                assert np.array_equal(dev.read_tensor(name, layer).view(np.uint16),
                                      ref.tensor(name, layer).view(np.uint16)), (name, layer)
    finally:
        dev.close()


def test_config0_prompt_then_64_greedy_steps(gda, oracle):
    """BASELINE config 0: batch 1, 32-token prompt of uniform ids, 64 greedy tokens with KV cache."""
    dev, ref = _pair(gda, oracle, 1)
    try:
        prompt = oracle.uniform_i32(32, 1000, 0, 2047)
        lg_d, nx_d, gp_d = dev.prefill(prompt, [0, 32])
        lg_r, nx_r, gp_r = ref.prefill(prompt, [0, 32])
        assert np.abs(lg_d.astype(np.float32) - lg_r.astype(np.float32)).max() < 4e-3
        ties = _assert_ids(nx_d, nx_r, gp_d, gp_r, "prefill")
        for l in range(3):
            kd, kr = dev.read_tensor("k_cache", l)[0, :32], ref.tensor("k_cache", l)[0, :32]
            assert np.abs(kd.astype(np.float32) - kr.astype(np.float32)).max() < 4e-3
        tok = nx_r.copy()
        for step in range(64):
            lg_d, nx_d, gp_d = dev.step(tok)
            lg_r, nx_r, gp_r = ref.step(tok)
            assert np.abs(lg_d.astype(np.float32) - lg_r.astype(np.float32)).max() < 4e-3, step
            ties += _assert_ids(nx_d, nx_r, gp_d, gp_r, f"step {step}")
            tok = nx_r.copy()  # both follow the oracle's token so one near-tie cannot fork the rest
        assert np.array_equal(dev.positions, [96]) and np.array_equal(ref.positions, [96])
        print("near-ties:", ties)
    finally:
        dev.close()


@pytest.mark.parametrize("window,tie", [(0, False), (16, True)])
def test_batched_ragged_prefill_and_steps(gda, oracle, window, tie):
    B = 4
    dev, ref = _pair(gda, oracle, B, window, tie, max_seq=64, layers=2, hidden=1024, seed=77)
    try:
        assert np.array_equal(dev.read_tensor("lm_head").view(np.uint16), ref.tensor("lm_head").view(np.uint16))
        assert tie == np.array_equal(ref.tensor("lm_head"), ref.tensor("embed"))
        lens = np.array([9, 1, 30, 17], np.int32)
        cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        prompt = oracle.uniform_i32(int(cu[-1]), 78, 0, 2047)
        lg_d, nx_d, gp_d = dev.prefill(prompt, cu)
        lg_r, nx_r, gp_r = ref.prefill(prompt, cu)
        assert np.abs(lg_d.astype(np.float32) - lg_r.astype(np.float32)).max() < 4e-3
        _assert_ids(nx_d, nx_r, gp_d, gp_r, "prefill")
        tok = nx_r.copy()
        for step in range(12):
            lg_d, nx_d, gp_d = dev.step(tok)
            lg_r, nx_r, gp_r = ref.step(tok)
            assert np.abs(lg_d.astype(np.float32) - lg_r.astype(np.float32)).max() < 4e-3, step
            _assert_ids(nx_d, nx_r, gp_d, gp_r, f"step {step}")
            tok = nx_r.copy()
        for l in range(2):
            for b in range(B):
                n = lens[b] + 12
                kd, kr = dev.read_tensor("k_cache", l)[b, :n], ref.tensor("k_cache", l)[b, :n]
                vd, vr = dev.read_tensor("v_cache", l)[b, :n], ref.tensor("v_cache", l)[b, :n]
                assert np.abs(kd.astype(np.float32) - kr.astype(np.float32)).max() < 6e-3
                assert np.abs(vd.astype(np.float32) - vr.astype(np.float32)).max() < 6e-3
        assert np.array_equal(dev.positions, lens + 12)
    finally:
        dev.close()


def test_scaled_architecture_prefill_and_steps(gda, oracle):
    """The layer shapes of BASELINE configs 3 and 4 (d_model 2048, 16 heads of 128, SwiGLU hidden 5632) at two layers
    and a 4096-token vocabulary: a ragged packed prefill long enough for the many-row kernels (336 rows: one full and
    one ragged 256-row tile, attention over several 64-key blocks), then cached steps through the public-operator
    loop and through the fused resident loop, all against the CPU oracle decoder."""
    from gradients_c_amd import decoder as D
    V, Dm, L, H, Dh, Hm, T, B = 4096, 2048, 2, 16, 128, 5632, 256, 4
    cfg = D.gpt_config(V, Dm, L, H, Dh, Hm, T, B, 0, False, 4242)
    dev = D.GptDecoder(cfg, max_prefill_tokens=512)
    ref = oracle.Decoder(V, Dm, L, H, Dh, Hm, T, B, 0, 4242, False)
    try:
        lens = np.array([150, 40, 129, 17], np.int32)
        cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        prompt = oracle.uniform_i32(int(cu[-1]), 4243, 0, V - 1)
        lg_d, nx_d, gp_d = dev.prefill(prompt, cu)
        lg_r, nx_r, gp_r = ref.prefill(prompt, cu)
        worst = np.abs(lg_d.astype(np.float32) - lg_r.astype(np.float32)).max()
        print("prefill logits: worst difference", worst, "largest logit", np.abs(lg_r.astype(np.float32)).max())
        assert worst < 8e-3
        _assert_ids(nx_d, nx_r, gp_d, gp_r, "prefill")
        for l in range(L):
            for b in range(B):
                kd, kr = dev.read_tensor("k_cache", l)[b, :lens[b]], ref.tensor("k_cache", l)[b, :lens[b]]
                vd, vr = dev.read_tensor("v_cache", l)[b, :lens[b]], ref.tensor("v_cache", l)[b, :lens[b]]
                assert np.abs(kd.astype(np.float32) - kr.astype(np.float32)).max() < 8e-3, (l, b)
                assert np.abs(vd.astype(np.float32) - vr.astype(np.float32)).max() < 8e-3, (l, b)
        tok = nx_r.copy()
        for step in range(4):
            lg_d, nx_d, gp_d = dev.step(tok)
            lg_r, nx_r, gp_r = ref.step(tok)
            assert np.abs(lg_d.astype(np.float32) - lg_r.astype(np.float32)).max() < 8e-3, step
            _assert_ids(nx_d, nx_r, gp_d, gp_r, f"step {step}")
            tok = nx_r.copy()
        # fused resident loop from the same state: every step against the oracle following the device's tokens
        ids, gaps, _ = dev.run_resident(tok, 6)
        for s in range(6):
            _, nx_r, gp_r = ref.step(tok)
            bad = [i for i in np.nonzero(ids[s] != nx_r)[0] if min(gaps[s][i], gp_r[i]) >= 1e-3]
            assert not bad, (s, bad)
            tok = ids[s].copy()
        assert np.array_equal(dev.positions, lens + 10) and np.array_equal(ref.positions, lens + 10)
    finally:
        dev.close()


def _resident_pair(D, oracle, seed):
    cfg = D.gpt_config(2048, 512, 3, 8, 64, 1536, 96, 8, 0, True, seed)
    a, b = D.GptDecoder(cfg, max_prefill_tokens=8 * 32), D.GptDecoder(cfg, max_prefill_tokens=8 * 32)
    lens = np.array([5, 9, 1, 20, 7, 7, 13, 2], np.int32)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    prompt = oracle.uniform_i32(int(cu[-1]), seed + 1, 0, 2047)
    _, first_a, _ = a.prefill(prompt, cu)
    _, first_b, _ = b.prefill(prompt, cu)
    assert np.array_equal(first_a, first_b)
    return a, b, first_a


def test_resident_unfused_graph_replay_equals_stepwise_bit_for_bit(gda, oracle):
    """Device-resident graph replay of the public-operator step: same tokens, gaps and caches as the
    per-step loop with host uploads/downloads."""
    from gradients_c_amd import decoder as D
    a, b, first = _resident_pair(D, oracle, 5)
    try:
        a.resident_begin(first, 24, unfused=True)
        a.resident_run(23)
        ids, gaps = a.resident_end()
        tok = first.copy()
        for s in range(24):
            _, nxt, gp = b.step(tok)
            assert np.array_equal(ids[s], nxt), s
            assert np.array_equal(gaps[s], gp), s
            tok = nxt
        assert np.array_equal(a.positions, b.positions)
        for l in range(3):
            assert np.array_equal(a.read_tensor("k_cache", l).view(np.uint16), b.read_tensor("k_cache", l).view(np.uint16))
    finally:
        a.close()
        b.close()


def test_resident_fused_matches_stepwise_and_oracle(gda, oracle):
    """The fused step keeps the rounding points of the separate operators; only the order of the F32
    sum inside the rms_norm prologue differs, so tokens agree except reported near-ties."""
    from gradients_c_amd import decoder as D
    a, b, first = _resident_pair(D, oracle, 6)
    try:
        ids, gaps, ms = a.run_resident(first, 24)
        assert ms > 0
        tok, ties = first.copy(), 0
        for s in range(24):
            lg, nxt, gp = b.step(tok)
            bad = [i for i in np.nonzero(ids[s] != nxt)[0] if min(gaps[s][i], gp[i]) >= 1e-3]
            assert not bad, (s, bad)
            ties += int(np.count_nonzero(ids[s] != nxt))
            assert np.abs(gaps[s] - gp).max() < 5e-2
            tok = ids[s].copy()  # follow the resident run
        assert np.array_equal(a.positions, b.positions)
        for l in range(3):
            ka, kb = a.read_tensor("k_cache", l), b.read_tensor("k_cache", l)
            assert np.abs(ka.astype(np.float32) - kb.astype(np.float32)).max() < 6e-3
    finally:
        a.close()
        b.close()


def test_resident_hold_positions_repeats_one_shape(gda, oracle):
    from gradients_c_amd import decoder as D
    a, b, first = _resident_pair(D, oracle, 7)
    try:
        before = a.positions.copy()
        a.resident_begin(first, 5, hold_positions=True)
        a.resident_run(4)
        a.resident_sync()
        ids, _ = a.resident_end()
        assert ids.shape == (5, 8) and np.array_equal(a.positions, before)
        _, nxt, _ = b.step(first)  # the first resident step is an ordinary step at the same position
        assert np.array_equal(ids[0], nxt)
    finally:
        a.close()
        b.close()


def test_decode_step_matches_packed_forward(gda, oracle):
    """The invariant of the reference's probes/gpt_lm_debug/compare_decode.c:14-18 on the device:
    prefill(n) + one cached decode step == last row of a packed forward over n+1 tokens."""
    from gradients_c_amd import decoder as D
    cfg = D.gpt_config(2048, 512, 3, 8, 64, 1536, 64, 1, 0, True, 9)
    a, b = D.GptDecoder(cfg, max_prefill_tokens=64), D.GptDecoder(cfg, max_prefill_tokens=64)
    try:
        ids = oracle.uniform_i32(41, 10, 0, 2047)
        a.prefill(ids[:40], [0, 40])
        lg_step, _, _ = a.step(ids[40:41])
        lg_full, _, _ = b.prefill(ids, [0, 41])
        assert np.abs(lg_step.astype(np.float32) - lg_full.astype(np.float32)).max() < 4e-3
    finally:
        a.close()
        b.close()


def test_checkpoint_written_by_the_reference_reproduces_its_generation(gda):
    """tests/golden/gpt_small_seed777.gdckpt was saved by the reference's gd_module_save_state from the model its
    own generation code then ran (tests/golden/make_gdckpt_fixture.py; vocabulary 64, width 64, 2 heads of 32, MLP
    128, context 64, 2 layers, window 0): a decoder created from ANOTHER seed, after loading the file, must give the
    reference's logits (F16 read back as F32, absolute 4e-3 as for the reference-program tests) and its token ids
    (near-ties excepted), stepwise and through the fused resident path; and every weight must hold the file's bytes."""
    import os
    from gradients_c_amd import decoder as D
    golden = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    ckpt = os.path.join(golden, "gpt_small_seed777.gdckpt")
    head = np.fromfile(os.path.join(golden, "gpt_small_seed777_in.bin"), np.int32)
    B, new_tokens, layers = (int(v) for v in head[:3])
    lens = head[3:3 + B]
    prompt = head[3 + B:]
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    assert prompt.size == cu[-1]
    out = np.fromfile(os.path.join(golden, "gpt_small_seed777_out.bin"), np.uint8)
    ref_ids = out[:4 * new_tokens * B].view(np.int32).reshape(new_tokens, B)
    ref_logits = out[4 * new_tokens * B:].view(np.float32).reshape(new_tokens, B, 64)

    dev = D.GptDecoder(D.gpt_config(64, 64, layers, 2, 32, 128, 64, B, 0, True, 31337), max_prefill_tokens=int(cu[-1]))
    try:
        lg0, _, _ = dev.prefill(prompt, cu)
        assert np.abs(ref_logits[0] - lg0.astype(np.float32)).max() > 0.05, "other seed, other model"
        dev.positions[:] = 0
        dev.load_checkpoint(ckpt)
        with D.Checkpoint(ckpt) as ck:
            for path, name, layer in (("gpt_lm.token_embedding", "embed", 0), ("gpt_lm.token_embedding", "lm_head", 0),
                                      ("gpt_lm.blocks.1.up_gate.weight", "w_upgate", 1),
                                      ("gpt_lm.blocks.0.qkv_proj.weight", "w_qkv", 0)):
                assert np.array_equal(dev.read_tensor(name, layer).view(np.uint16).ravel(),
                                      ck.read(path).view(np.uint16).ravel()), path
            down = ck.read("gpt_lm.blocks.1.down_proj.weight")
            assert np.array_equal(dev.read_tensor("w_down_t", 1).reshape(64, 128).view(np.uint16), down.T.view(np.uint16))
        near = 0
        for s in range(new_tokens):
            lg, nx, gp = dev.prefill(prompt, cu) if s == 0 else dev.step(ref_ids[s - 1])
            assert np.abs(ref_logits[s] - lg.astype(np.float32)).max() < 4e-3, s
            for b in np.nonzero(nx != ref_ids[s])[0]:
                assert gp[b] < 1e-3, f"step {s} row {b}: token differs and is not a near-tie"
                near += 1
        print("near-ties:", near)
        # the fused resident path on the loaded weights (it reads the [d_model, hidden] copy of the down weight)
        dev.positions[:] = 0
        _, nx, _ = dev.prefill(prompt, cu)
        ids, gaps, _ = dev.run_resident(ref_ids[0], new_tokens - 1)
        for s in range(1, new_tokens):
            for b in np.nonzero(ids[s - 1] != ref_ids[s])[0]:
                assert gaps[s - 1][b] < 1e-3, f"resident step {s} row {b}"
            if not np.array_equal(ids[s - 1], ref_ids[s]):
                break  # after a near-tie the sequences legitimately part
        # a load while a resident session is open is refused
        dev.resident_begin(ref_ids[0], 2)
        st = D.lib().gd_gpt_decoder_load_checkpoint(dev.handle, ckpt.encode(), 1)
        dev.resident_end()
        assert st == -4
    finally:
        dev.close()


def _reference_generate(oracle, ref, prompts, max_new, p, stop, rng, ctx_len):
    """The reference's generation loop (examples/gpt_lm/gpt_lm_shared.c:1444-1700 without the tokenizer) over the
    oracle decoder and the oracle's restatement of its sampler.  Returns the new tokens per row and the smallest
    margin seen (distance of a draw from a token boundary, or the greedy gap)."""
    B = len(prompts)
    room = ctx_len - 1 if max_new >= ctx_len else ctx_len - max_new
    seqs = [list(q[-room:]) for q in prompts]
    plen = [len(q) for q in seqs]
    cu = np.concatenate([[0], np.cumsum(plen)]).astype(np.int32)
    logits, _, _ = ref.prefill(np.concatenate(seqs).astype(np.int32), cu)
    finished, nxt, generated, worst = [False] * B, [0] * B, 0, np.inf

    def pick(b, row):
        nonlocal rng, worst
        capped = oracle.logits_softcap(row.astype(np.float32), p["softcap"])
        tok, rng, margin, left = oracle.sample_next_token(capped, seqs[b], p["temperature"], p["min_p"], p["penalty"], rng)
        if not np.isfinite(margin):
            top = np.sort(left[np.isfinite(left)])[-2:]
            margin = float(top[1] - top[0]) if top.size == 2 else np.inf
        worst = min(worst, margin)
        return tok

    for b in range(B):
        nxt[b] = pick(b, logits[b])
    while generated < max_new and not all(finished):
        appended = False
        for b in range(B):
            if finished[b]:
                continue
            if (stop >= 0 and nxt[b] == stop) or len(seqs[b]) >= ctx_len:
                finished[b] = True
                continue
            seqs[b].append(int(nxt[b]))
            appended = True
        if not appended:
            break
        generated += 1
        if generated >= max_new or all(finished):
            break
        ids = np.array([(stop if stop >= 0 else 0) if finished[b] else nxt[b] for b in range(B)], np.int32)
        logits, _, _ = ref.step(ids)
        for b in range(B):
            if not finished[b]:
                nxt[b] = pick(b, logits[b])
    return [np.array(seqs[b][plen[b]:], np.int32) for b in range(B)], worst


@pytest.mark.parametrize("params,stop,max_new", [
    (dict(temperature=0.8, min_p=0.05, penalty=1.3, softcap=20.0), 7, 24),
    (dict(temperature=1.0, min_p=0.0, penalty=1.0, softcap=0.0), -1, 12),
    (dict(temperature=0.0, min_p=0.0, penalty=1.2, softcap=0.0), 3, 40),
    (dict(temperature=1.5, min_p=0.0, penalty=1.0, softcap=0.0), 1, 70),
])
def test_generate_with_the_sampling_front_end(gda, oracle, params, stop, max_new):
    """gd_gpt_decoder_generate (packed prefill, device sampling, graph-replayed steps) against the reference's loop
    restated over the oracle: the same tokens row by row, unless a draw fell within 1e-5 of a token boundary (then
    the sequences may part and only the common prefix is compared).  Small vocabulary so that stop tokens and
    repeats occur; the last case runs rows into the end of the context."""
    from gradients_c_amd import decoder as D
    V, Dm, L, H, Dh, Hm, T, B = 96, 64, 2, 2, 32, 128, 48, 5
    if max_new == 70:
        T = 40
    seed = 4321
    dev = D.GptDecoder(D.gpt_config(V, Dm, L, H, Dh, Hm, T, B, 0, True, seed), max_prefill_tokens=B * T)
    ref = oracle.Decoder(V, Dm, L, H, Dh, Hm, T, B, 0, seed, True)
    try:
        lens = [9, 1, 30, 4, 17]
        flat = oracle.uniform_i32(sum(lens), 5, 0, V - 1)
        cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        prompts = [flat[cu[b]:cu[b + 1]] for b in range(B)]
        rng0 = D.lib().gd_gpt_generation_rng(seed, B, 0)
        assert rng0 == oracle.splitmix64(seed ^ 0xdec0de1234567890 ^ B ^ 0)
        got = dev.generate(flat, cu, max_new, params["temperature"], params["min_p"], params["penalty"],
                           params["softcap"], stop, rng0)
        want, worst = _reference_generate(oracle, ref, prompts, max_new, params, stop, rng0, T)
        exact = all(np.array_equal(g, w) for g, w in zip(got, want))
        print("rows:", [len(w) for w in want], "worst margin:", worst, "exact:", exact)
        if not exact:
            assert worst < 1e-3, (got, want)
        else:
            assert all(len(w) <= max_new for w in want)
        if max_new == 70:
            room = T - 1
            assert all(len(w) + min(len(q), room) <= T for w, q in zip(want, prompts))
        # a second call starts over from its prompts (caches, histories, flags and generator are reset)
        again = dev.generate(flat, cu, max_new, params["temperature"], params["min_p"], params["penalty"],
                             params["softcap"], stop, rng0)
        assert all(np.array_equal(a, g) for a, g in zip(again, got))
    finally:
        dev.close()
        ref.close()


def test_minimax_m3_architecture_prefill_and_steps(gda, oracle):
    """The reference's MiniMax-M3 architecture (gpt_lm_shared.c:588-600, 918-933): the packed prefill picks blocks and
    attends over them, the decode step is the dense one.  Block size 8, 3 blocks per row (first and last forced),
    context 128, so that the rule "context > 8 blocks and 2 x picked keys < context" holds; ragged prompts with a
    sequence of one token, one inside the first block and two long ones."""
    from gradients_c_amd import decoder as D
    V, Dm, L, H, Dh, Hm, T, B = 256, 128, 2, 4, 32, 256, 128, 4
    m3 = (8, 3, 1, 1)
    dev = D.GptDecoder(D.gpt_config(V, Dm, L, H, Dh, Hm, T, B, 0, True, 77, minimax_m3=m3), max_prefill_tokens=B * T)
    ref = oracle.Decoder(V, Dm, L, H, Dh, Hm, T, B, 0, 77, True)
    ref.set_minimax_m3(*m3)
    dense = oracle.Decoder(V, Dm, L, H, Dh, Hm, T, B, 0, 77, True)
    try:
        lens = [100, 1, 5, 90]
        cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        prompt = oracle.uniform_i32(int(cu[-1]), 8, 0, V - 1)
        lg_d, nx_d, gp_d = dev.prefill(prompt, cu)
        lg_r, nx_r, gp_r = ref.prefill(prompt, cu)
        lg_x, _, _ = dense.prefill(prompt, cu)
        err = np.abs(lg_d.astype(np.float32) - lg_r.astype(np.float32)).max()
        apart = np.abs(lg_x.astype(np.float32) - lg_r.astype(np.float32))
        print("minimax prefill: worst difference", err, "dense vs picked blocks", apart.max(axis=1))
        assert err < 4e-3
        assert apart[0].max() > 0.02 and apart[3].max() > 0.02      # long rows: picked blocks are not the dense result
        assert apart[1].max() < 1e-3 and apart[2].max() < 1e-3      # rows inside the first block: identical
        for l in range(L):
            got = dev.read_tensor("k_cache", l).reshape(B, T, H, Dh)[0, :100].astype(np.float32)
            want = ref.tensor("k_cache", l).reshape(B, T, H, Dh)[0, :100].astype(np.float32)
            assert np.abs(got - want).max() < 4e-3, l
        near = _assert_ids(nx_d, nx_r, gp_d, gp_r, "minimax prefill")
        tok = nx_r.copy()
        for s in range(6):
            lg_d, nx_d, gp_d = dev.step(tok)
            lg_r, nx_r, gp_r = ref.step(tok)
            assert np.abs(lg_d.astype(np.float32) - lg_r.astype(np.float32)).max() < 4e-3, s
            near += _assert_ids(nx_d, nx_r, gp_d, gp_r, f"minimax step {s}")
            tok = nx_r.copy()
        print("near-ties:", near)
    finally:
        dev.close()
        ref.close()
        dense.close()


def test_headline_step_shape_against_oracle(gda, oracle):
    """The step the benchmark times, whole: default architecture, B=64, every cache holding 511 rows, one fused
    resident step plus three graph replays at position 511 (positions held, each replay fed the previous pick).
    Device and oracle start from the same random F16 cache rows; logits within 4e-3, picks equal except reported
    near-ties (top-2 gap below 1e-3), appended K/V rows within 6e-3."""
    from gradients_c_amd import decoder as D
    V, Dm, L, H, Dh, Hm, T, B = 2048, 512, 3, 8, 64, 1536, 512, 64
    dev = D.GptDecoder(D.gpt_config(V, Dm, L, H, Dh, Hm, T, B, 0, False, 1002), max_prefill_tokens=B)
    ref = oracle.Decoder(V, Dm, L, H, Dh, Hm, T, B, 0, 1002, False)
    try:
        for l in range(L):
            for name, seed in (("k_cache", 7000 + l), ("v_cache", 7100 + l)):
                rows = oracle.normal_f16((B, T, H, Dh), seed, 0.5)
                ref.tensor(name, l)[:] = rows
                dev.write_tensor(name, l, rows)
        dev.positions[:] = T - 1
        tok = oracle.uniform_i32(B, 7200, 0, V - 1)
        dev.resident_begin(tok, 4, hold_positions=True, keep_logits=True)
        ties = 0
        for s in range(4):
            if s > 0:
                dev.resident_run(1)
            dev.resident_sync()
            lg_d = dev.read_tensor("last_logits")
            ref.positions[:] = T - 1
            lg_r, nx_r, gp_r = ref.step(tok)
            worst = np.abs(lg_d.astype(np.float32) - lg_r.astype(np.float32)).max()
            assert worst < 4e-3, (s, worst)
            nx_d = np.argmax(lg_d.astype(np.float32), axis=1).astype(np.int32)
            top2 = np.sort(lg_d.astype(np.float32), axis=1)[:, -2:]
            ties += _assert_ids(nx_d, nx_r, top2[:, 1] - top2[:, 0], gp_r, f"step {s}")
            for l in range(L):
                for name in ("k_cache", "v_cache"):
                    a, b = dev.read_tensor(name, l)[:, T - 1], ref.tensor(name, l)[:, T - 1]
                    assert np.abs(a.astype(np.float32) - b.astype(np.float32)).max() < 6e-3, (s, l, name)
            tok = nx_d
        ids, gaps = dev.resident_end()
        assert ids.shape == (4, B)
        # the picks the device recorded are the first maxima of the logits it kept, and each fed the next step
        assert np.array_equal(ids[3], tok)
        print("near-ties:", ties)
    finally:
        dev.close()
        ref.close()


def test_ragged_prefill_then_128_resident_steps(gda, oracle):
    """The run of BASELINE configs[4] at the scaled layer shapes (d_model 2048, 16 heads of 128, SwiGLU hidden 5632;
    two layers, vocabulary 2048, shorter prompts): packed prefill of 32 ragged prompts, then 128 fused resident steps
    with growing caches.  The oracle follows six of the 32 sequences (batch rows are independent) step by step, fed
    the device's own tokens: picks equal except reported near-ties."""
    from gradients_c_amd import decoder as D
    V, Dm, L, H, Dh, Hm, T, B, steps = 2048, 2048, 2, 16, 128, 5632, 192, 32, 128
    rng = np.random.default_rng(44)
    lens = rng.integers(1, 65, B).astype(np.int32)
    lens[3], lens[17] = 1, 64
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    prompt = oracle.uniform_i32(int(cu[-1]), 4401, 0, V - 1)
    rows = [3, 17, 0, 9, 22, 31]
    dev = D.GptDecoder(D.gpt_config(V, Dm, L, H, Dh, Hm, T, B, 0, False, 4400), max_prefill_tokens=int(cu[-1]))
    ref = oracle.Decoder(V, Dm, L, H, Dh, Hm, T, len(rows), 0, 4400, False)
    try:
        _, first, gap0 = dev.prefill(prompt, cu, want_logits=False)
        sub = np.concatenate([prompt[cu[r]:cu[r + 1]] for r in rows])
        sub_cu = np.concatenate([[0], np.cumsum(lens[rows])]).astype(np.int32)
        _, nx_r, gp_r = ref.prefill(sub, sub_cu)
        ties = _assert_ids(first[rows], nx_r, gap0[rows], gp_r, "prefill")
        ids, gaps, _ = dev.run_resident(first, steps)
        assert ids.shape == (steps, B) and ids.min() >= 0 and ids.max() < V
        tok = first[rows].copy()
        for s in range(steps):
            _, nx_r, gp_r = ref.step(tok)
            ties += _assert_ids(ids[s][rows], nx_r, gaps[s][rows], gp_r, f"step {s}")
            tok = ids[s][rows].copy()
        assert np.array_equal(dev.positions, lens + steps)
        for l in range(L):
            for i, r in enumerate(rows):
                n = lens[r] + steps
                for name in ("k_cache", "v_cache"):
                    a, b = dev.read_tensor(name, l)[r, :n], ref.tensor(name, l)[i, :n]
                    assert np.abs(a.astype(np.float32) - b.astype(np.float32)).max() < 8e-3, (l, r, name)
        print("near-ties:", ties)
    finally:
        dev.close()
        ref.close()


def test_resident_steps_over_long_ragged_caches_take_the_pieces_form(gda, oracle):
    """Graph-replayed decode steps whose attention runs in the form that cuts long rows into pieces merged inside the
    kernel (a (row, kv head) pair per compute unit, caches of 1024 rows or more): the default architecture with 32
    sequences, 1100-row caches and prompts of 1..1000 tokens, 12 fused resident steps (one eager, eleven replays of the
    captured graph: the rows' arrival counters must be back at zero after every replay).  The oracle follows five of
    the sequences, the longest and the shortest among them, fed the device's own tokens."""
    from gradients_c_amd import decoder as D
    V, Dm, L, H, Dh, Hm, T, B, steps = 2048, 512, 3, 8, 64, 1536, 1100, 32, 12
    rng = np.random.default_rng(45)
    lens = rng.integers(1, 1001, B).astype(np.int32)
    lens[5], lens[11] = 1, 1000
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    prompt = oracle.uniform_i32(int(cu[-1]), 4501, 0, V - 1)
    rows = [5, 11, 0, 20, 31]
    dev = D.GptDecoder(D.gpt_config(V, Dm, L, H, Dh, Hm, T, B, 0, False, 4500), max_prefill_tokens=int(cu[-1]))
    ref = oracle.Decoder(V, Dm, L, H, Dh, Hm, T, len(rows), 0, 4500, False)
    try:
        _, first, gap0 = dev.prefill(prompt, cu, want_logits=False)
        sub = np.concatenate([prompt[cu[r]:cu[r + 1]] for r in rows])
        sub_cu = np.concatenate([[0], np.cumsum(lens[rows])]).astype(np.int32)
        _, nx_r, gp_r = ref.prefill(sub, sub_cu)
        ties = _assert_ids(first[rows], nx_r, gap0[rows], gp_r, "prefill")
        ids, gaps, _ = dev.run_resident(first, steps)
        name = dev.ctx.backend().sdpa_decode_last_kernel()
        if B * H >= dev.ctx.backend().device_info()[1]:
            assert "rows merged by the last piece" in name, name
        tok = first[rows].copy()
        for s in range(steps):
            _, nx_r, gp_r = ref.step(tok)
            ties += _assert_ids(ids[s][rows], nx_r, gaps[s][rows], gp_r, f"step {s}")
            tok = ids[s][rows].copy()
        assert np.array_equal(dev.positions, lens + steps)
        print("near-ties:", ties, name)
    finally:
        dev.close()
        ref.close()


def test_prefill_with_the_rotation_in_the_projection_matches_the_separate_launches(gda, oracle):
    """A packed prefill of 12,100 tokens at head size 128 (d_model 512, 4 heads): 47 row tiles x 6 column tiles of the
    qkv projection are more than a round on 256 compute units, so 42 row tiles take the tile kernel's rotation + split +
    cache append epilogue and the remaining 1,348 rows the plain projection and the table-driven rotation kernel; the
    attention reads keys and values from the caches.  Against the same decoder with the tunable
    "prefill_rope_epilogue" = 0 (separate projection and rotation + append launches): first-layer values bit for bit,
    first-layer keys to one unit in the last place, last-layer caches and logits within the decoder tests' bar; and
    against the CPU oracle on the two shortest sequences."""
    from gradients_c_amd import decoder as D
    V, Dm, L, H, Dh, Hm, T, B = 2048, 512, 2, 4, 128, 1024, 2048, 8
    lens = np.array([2048, 1900, 1500, 1700, 1200, 2000, 1100, 652], np.int32)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    prompt = oracle.uniform_i32(int(cu[-1]), 4601, 0, V - 1)
    dev = D.GptDecoder(D.gpt_config(V, Dm, L, H, Dh, Hm, T, B, 0, False, 4600), max_prefill_tokens=int(cu[-1]))
    rows = [6, 7]
    ref = oracle.Decoder(V, Dm, L, H, Dh, Hm, T, len(rows), 0, 4600, False)
    try:
        be = dev.ctx.backend()
        lg_a, nx_a, gp_a = dev.prefill(prompt, cu)
        caches_a = [(dev.read_tensor("k_cache", l), dev.read_tensor("v_cache", l)) for l in range(L)]
        be.set_tunable("prefill_rope_epilogue", 0)
        lg_b, nx_b, gp_b = dev.prefill(prompt, cu)
        caches_b = [(dev.read_tensor("k_cache", l), dev.read_tensor("v_cache", l)) for l in range(L)]
        be.set_tunable("prefill_rope_epilogue", 1)
        for b in range(B):
            n = lens[b]
            ka, va, kb, vb = caches_a[0][0][b, :n], caches_a[0][1][b, :n], caches_b[0][0][b, :n], caches_b[0][1][b, :n]
            assert np.array_equal(va.view(np.uint16), vb.view(np.uint16)), b
            ulp = np.spacing(np.maximum(np.abs(ka), np.abs(kb)).astype(np.float16)).astype(np.float32)
            assert np.all(np.abs(ka.astype(np.float32) - kb.astype(np.float32)) <= ulp), b
            assert np.count_nonzero(ka.view(np.uint16) != kb.view(np.uint16)) <= max(2, ka.size // 300), b
            for which in (0, 1):
                xa, xb = caches_a[L - 1][which][b, :n].astype(np.float32), caches_b[L - 1][which][b, :n].astype(np.float32)
                assert np.abs(xa - xb).max() < 8e-3, (b, which)
        assert np.abs(lg_a.astype(np.float32) - lg_b.astype(np.float32)).max() < 8e-3
        _assert_ids(nx_a, nx_b, gp_a, gp_b, "fused against separate launches")
        sub = np.concatenate([prompt[cu[r]:cu[r + 1]] for r in rows])
        sub_cu = np.concatenate([[0], np.cumsum(lens[rows])]).astype(np.int32)
        lg_r, nx_r, gp_r = ref.prefill(sub, sub_cu)
        assert np.abs(lg_a[rows].astype(np.float32) - lg_r.astype(np.float32)).max() < 8e-3
        _assert_ids(nx_a[rows], nx_r, gp_a[rows], gp_r, "fused against the oracle")
        for i, r in enumerate(rows):
            for l in range(L):
                kd, kr = caches_a[l][0][r, :lens[r]], ref.tensor("k_cache", l)[i, :lens[r]]
                vd, vr = caches_a[l][1][r, :lens[r]], ref.tensor("v_cache", l)[i, :lens[r]]
                assert np.abs(kd.astype(np.float32) - kr.astype(np.float32)).max() < 8e-3, (l, r)
                assert np.abs(vd.astype(np.float32) - vr.astype(np.float32)).max() < 8e-3, (l, r)
    finally:
        dev.close()
        ref.close()
