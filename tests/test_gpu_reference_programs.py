"""The reference's OWN test programs, compiled from its sources (oracle/Makefile, target ref-tests)
against the unmodified reference core and linked with gradients.c_amd/libgd_backend_hip.so as the
backend.  They run with GD_HIP_HOST_VISIBLE=1 because the reference core insists on host-visible
arenas.  The binaries live in oracle/_ref/ (built where the reference tree is mounted, not tracked);
the tests are skipped when they have not been built.

  test_kv_cache_decode  literal append vectors (at / positions / packed) and the three sdpa_decode
                        position forms agreeing to 1e-6 (reference tests/test_kv_cache_decode.c)
  test_memory           arena / ring-slot / fence contract (reference tests/test_memory.c)
  test_transfer         upload / download / F32<->F16 transfer contract (reference tests/test_transfer.c)
  test_tensor           tensor descriptors, fill / rand_uniform, views, scopes (reference tests/test_tensor.c)

  ref_gpt_generate      oracle/ref_gpt_generate.c around the reference's own examples/gpt_lm/gpt_lm_shared.c:
                        packed ragged prefill, cached decode steps, greedy pick (64 new tokens at batch 1)

The reference's per-operator test programs also call the training (backward) entry points in the
same main(), which this backend answers with GD_ERR_UNSUPPORTED, so they cannot pass unmodified; their
forward cases are restated as data in tests/golden/reference_test_cases.json instead.
"""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF_DIR = os.path.join(ROOT, "oracle", "_ref")


@pytest.mark.parametrize("program", ["test_kv_cache_decode", "test_memory", "test_transfer", "test_tensor"])
def test_reference_program_passes_on_the_hip_backend(program):
    exe = os.path.join(REF_DIR, program)
    if not os.path.exists(exe):
        pytest.skip(f"{exe} not built (needs the reference tree: make -C oracle ref-tests)")
    env = dict(os.environ, GD_HIP_HOST_VISIBLE="1")
    r = subprocess.run([exe], env=env, capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert f"{program}: ok" in r.stdout


def _run_reference_generator(tmp_path, lens, prompt, new_tokens, layers, seed):
    exe = os.path.join(REF_DIR, "ref_gpt_generate")
    if not os.path.exists(exe):
        pytest.skip(f"{exe} not built (needs the reference tree: make -C oracle ref-tests)")
    import numpy as np
    src, dst = tmp_path / "in.bin", tmp_path / "out.bin"
    np.concatenate([[len(lens), new_tokens, layers], lens, prompt]).astype(np.int32).tofile(src)
    env = dict(os.environ, GD_HIP_HOST_VISIBLE="1")
    r = subprocess.run([exe, str(src), str(dst), str(seed)], env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    raw = np.fromfile(dst, np.uint8)
    n = new_tokens * len(lens)
    ids = raw[: 4 * n].view(np.int32).reshape(new_tokens, len(lens))
    logits = raw[4 * n:].view(np.float32).reshape(new_tokens, len(lens), 2048)
    return ids, logits


@pytest.mark.parametrize("lens,new_tokens", [([32], 65), ([9, 1, 30, 17], 9)])
def test_reference_generation_code_on_this_backend_matches_oracle_and_decoder(gda, oracle, tmp_path, lens, new_tokens):
    """The reference's own gpt_lm prefill + cached decode (its operator call sequence, its weight init,
    its greedy pick), executing on the HIP backend, against (a) the CPU oracle decoder and (b) this
    repository's C decoder: same seeds, same ragged prompts.  Default reference dimensions: vocabulary
    2048, width 512, 8 heads of 64, MLP 1024, context 512, window 256, tied LM head."""
    import numpy as np
    from gradients_c_amd import decoder as D
    layers, seed, B = 3, 4242, len(lens)
    lens = np.asarray(lens, np.int32)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    prompt = oracle.uniform_i32(int(cu[-1]), 9, 0, 2047)
    ref_ids, ref_logits = _run_reference_generator(tmp_path, lens, prompt, new_tokens, layers, seed)

    cpu = oracle.Decoder(2048, 512, layers, 8, 64, 1024, 512, B, 256, seed, True)
    dev = D.GptDecoder(D.gpt_config(2048, 512, layers, 8, 64, 1024, 512, B, 256, True, seed),
                       max_prefill_tokens=int(cu[-1]))
    try:
        mismatches = 0
        for s in range(new_tokens):
            if s == 0:
                lg_c, nx_c, gp_c = cpu.prefill(prompt, cu)
                lg_d, nx_d, gp_d = dev.prefill(prompt, cu)
            else:
                lg_c, nx_c, gp_c = cpu.step(ref_ids[s - 1])
                lg_d, nx_d, gp_d = dev.step(ref_ids[s - 1])
            # the reference program reads the F16 logits back as F32
            assert np.abs(ref_logits[s] - lg_c.astype(np.float32)).max() < 4e-3, ("oracle", s)
            assert np.abs(ref_logits[s] - lg_d.astype(np.float32)).max() < 4e-3, ("decoder", s)
            for nx, gp, who in ((nx_c, gp_c, "oracle"), (nx_d, gp_d, "decoder")):
                for b in np.nonzero(nx != ref_ids[s])[0]:
                    assert gp[b] < 1e-3, f"{who} step {s} row {b}: token differs and is not a near-tie"
                    mismatches += 1
        print("near-ties:", mismatches)
    finally:
        dev.close()
