"""Text in, text out: gradients.c_amd/gpt_lm_infer (csrc/apps/gpt_lm_infer.c, the counterpart of the reference's
examples/gpt_lm/infer.c) on a checkpoint and a tokenizer that the reference's own code wrote.

tests/golden/gpt_tok420_seed99.gdckpt: saved by the reference's gd_module_save_state with trainer-style metadata;
tests/golden/gpt_tok420_seed99_out.bin: what the reference's generation code produced from it for the prompt
"the quick brown fox" (ids from the reference's encoder), greedy, 12 tokens (tests/golden/make_infer_fixture.py).
"""
import os
import re
import subprocess

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(ROOT, "tests", "golden")
EXE = os.path.join(ROOT, "gradients.c_amd", "gpt_lm_infer")
CKPT = os.path.join(GOLDEN, "gpt_tok420_seed99.gdckpt")
VOCAB = os.path.join(GOLDEN, "tokenizer_small.json")


def run(*args):
    """Exit code, stdout as bytes (a randomly initialised model emits bytes that are no valid UTF-8), stderr."""
    r = subprocess.run([EXE, *args], capture_output=True, timeout=120)
    return r.returncode, r.stdout, r.stderr.decode(errors="replace")


def parse(stdout):
    ids = [int(v) for v in re.search(rb"^ids:(.*)$", stdout, re.M).group(1).split()]
    text = re.search(rb"^generated_text=(.*)$", stdout, re.M | re.S).group(1).rsplit(b"\ngenerate:", 1)[0]
    return ids, text


def test_greedy_text_equals_the_reference_generation(gda):
    from gradients_c_amd import tokenizer as T
    raw = np.fromfile(os.path.join(GOLDEN, "gpt_tok420_seed99_out.bin"), np.uint8)
    ref_ids = raw[:48].view(np.int32)
    ref_logits = raw[48:].view(np.float32).reshape(12, 420)
    top2 = np.sort(ref_logits, axis=1)[:, -2:]
    assert (top2[:, 1] - top2[:, 0]).min() > 0.1          # no near-tie in the reference run: ids must be identical
    rc, out, err = run("--checkpoint", CKPT, "--tokenizer-path", VOCAB, "--prompt", "the quick brown fox",
                       "--max-new-tokens", "12", "--ids")
    assert rc == 0, (rc, err, out[-400:])
    ids, text = parse(out)
    assert ids == ref_ids.tolist()
    tok = T.Tokenizer(VOCAB, 1, 1)
    assert text == tok.decode(ref_ids)
    assert b"layers=2 d_model=64 heads=2 vocab=420 context=64 prompt_tokens=6" in out   # all from the checkpoint


def test_sampled_run_equals_the_library_call(gda):
    from gradients_c_amd import decoder as D, tokenizer as T
    args = ("--checkpoint", CKPT, "--tokenizer-path", VOCAB, "--prompt", "hello <eot> 123 tokenizer test",
            "--max-new-tokens", "20", "--temperature", "0.9", "--min-p", "0.02", "--repetition-penalty", "1.2",
            "--logits-softcap", "15", "--seed", "5", "--ids")
    rc, out, err = run(*args)
    assert rc == 0, (rc, err, out[-400:])
    ids, text = parse(out)
    tok = T.Tokenizer(VOCAB, 1, 1)
    prompt = tok.encode("hello <eot> 123 tokenizer test")
    assert tok.token_id("<eot>") in prompt
    cfg = D.config_from_checkpoint(CKPT, batch=1)
    dev = D.GptDecoder(cfg, max_prefill_tokens=prompt.size)
    try:
        dev.load_checkpoint(CKPT)
        want = dev.generate(prompt, [0, prompt.size], 20, 0.9, 0.02, 1.2, 15.0, -1,
                            D.lib().gd_gpt_generation_rng(5, 1, 0))[0]
    finally:
        dev.close()
    assert ids == want.tolist() and len(set(ids)) > 3
    assert text == tok.decode(want)
    # the same seed gives the same text, another seed another
    assert parse(run(*args)[1])[0] == ids
    other = list(args)
    other[other.index("--seed") + 1] = "6"
    assert parse(run(*other)[1])[0] != ids
    # special texts as ordinary text: a longer prompt
    rc, out2, _ = run(*args, "--no-special")
    assert rc == 0 and b"prompt_tokens=%d" % T.Tokenizer(VOCAB, 1, 0).encode("hello <eot> 123 tokenizer test").size in out2


def test_errors_are_reported(gda):
    rc, out, err = run("--checkpoint", os.path.join(GOLDEN, "absent.gdckpt"), "--tokenizer-path", VOCAB, "--prompt", "x")
    assert rc != 0 and "io error" in err
    rc, out, err = run("--checkpoint", CKPT, "--tokenizer-path", os.path.join(GOLDEN, "absent.json"), "--prompt", "x")
    assert rc != 0 and "tokenizer" in err
    rc, out, err = run("--checkpoint", os.path.join(GOLDEN, "gpt_small_seed777.gdckpt"), "--tokenizer-path", VOCAB,
                       "--prompt", "x", "--heads", "2", "--context", "64")
    assert rc != 0 and "420 tokens, the model 64" in err     # vocabulary of the tokenizer exceeds the model's
    rc, out, err = run("--prompt", "x")
    assert rc == 2
