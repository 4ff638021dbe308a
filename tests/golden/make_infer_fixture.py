"""Writes the fixture of the text-in / text-out test with the reference's OWN code.

Runs oracle/_ref/ref_gpt_generate_tok420 (oracle/ref_gpt_generate.c around the reference's gpt_lm_shared.c at
vocabulary 420, d_model 64, 2 heads of 32, hidden 128, context 64, 2 layers; built by `make -C oracle ref-tests`) on a
machine with an MI355X.  The prompt is the text PROMPT encoded by the reference's tokenizer (its ids are taken from
tests/golden/tokenizer_cases.npz, which the reference's encoder produced); the reference initialises its model from
the seed, saves it with gd_module_save_state together with trainer-style metadata, and generates greedily.  Outputs:

  gpt_tok420_seed99.gdckpt    checkpoint + metadata (key=value lines as examples/gpt_lm/main.c:1836-1864 writes them)
  gpt_tok420_seed99_out.bin   int32 ids[new_tokens][1], float32 logits[new_tokens][1][420]
"""
import os
import subprocess
import sys
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
PROMPT_INDEX = 5          # "the quick brown fox" in make_tokenizer_fixture.TEXTS
NEW_TOKENS, LAYERS, SEED = 12, 2, 99

METADATA = ("model=gpt_lm\nvocab_size=420\ncontext_length=64\nd_model=64\nn_layers=2\nn_heads=2\nhead_dim=32\n"
            "mlp_hidden=128\nffn_activation=swiglu\narchitecture=gpt\nsdpa_window=0\ndropout=0\nlogits_softcap=0\n"
            "tokenizer_path=tests/golden/tokenizer_small.json\n")


def main():
    out_dir = sys.argv[1] if len(sys.argv) > 1 else HERE
    os.makedirs(out_dir, exist_ok=True)
    exe = os.path.join(ROOT, "oracle", "_ref", "ref_gpt_generate_tok420")
    cases = np.load(os.path.join(HERE, "tokenizer_cases.npz"))
    assert bytes(cases[f"text_{PROMPT_INDEX}"]) == b"the quick brown fox"
    prompt = cases[f"ids_0_{PROMPT_INDEX}"]
    dst = os.path.join(out_dir, "gpt_tok420_seed99_out.bin")
    ckpt = os.path.join(out_dir, "gpt_tok420_seed99.gdckpt")
    with tempfile.TemporaryDirectory() as tmp:
        src, meta = os.path.join(tmp, "in.bin"), os.path.join(tmp, "meta.txt")
        np.concatenate([[1, NEW_TOKENS, LAYERS], [prompt.size], prompt]).astype(np.int32).tofile(src)
        with open(meta, "w") as f:
            f.write(METADATA)
        env = dict(os.environ, GD_HIP_HOST_VISIBLE="1")
        r = subprocess.run([exe, src, dst, str(SEED), ckpt, meta], env=env, capture_output=True, text=True, timeout=300)
    print(r.stdout, r.stderr)
    if r.returncode != 0:
        raise SystemExit(r.returncode)
    print("wrote", ckpt, os.path.getsize(ckpt), "bytes")


if __name__ == "__main__":
    main()
