"""Writes the checkpoint fixture of the .gdckpt loader tests with the reference's OWN code.

Runs oracle/_ref/ref_gpt_generate_small (oracle/ref_gpt_generate.c around the reference's
examples/gpt_lm/gpt_lm_shared.c, compiled from the reference tree by `make -C oracle ref-tests` at vocabulary 64,
d_model 64, 2 heads of 32, hidden 128, context 64, 2 layers) on a machine with an MI355X: the reference initialises
its model from the seed, saves it with gd_module_save_state (src/nn/module_io.c) and generates from a fixed ragged
prompt.  Outputs, into the directory given as argv[1] (default: this directory):

  gpt_small_seed777.gdckpt    the checkpoint as the reference wrote it
  gpt_small_seed777_in.bin    int32: batch, new_tokens, layers, prompt lengths, packed prompt ids
  gpt_small_seed777_out.bin   int32 ids[new_tokens][batch], float32 logits[new_tokens][batch][64]
"""
import os
import subprocess
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))


def main():
    out_dir = sys.argv[1] if len(sys.argv) > 1 else HERE
    os.makedirs(out_dir, exist_ok=True)
    exe = os.path.join(ROOT, "oracle", "_ref", "ref_gpt_generate_small")
    lens = np.array([5, 3], np.int32)
    prompt = (np.arange(int(lens.sum()), dtype=np.int64) * 37 + 11) % 64
    new_tokens, layers, seed = 6, 2, 777
    src = os.path.join(out_dir, "gpt_small_seed777_in.bin")
    dst = os.path.join(out_dir, "gpt_small_seed777_out.bin")
    ckpt = os.path.join(out_dir, "gpt_small_seed777.gdckpt")
    np.concatenate([[len(lens), new_tokens, layers], lens, prompt]).astype(np.int32).tofile(src)
    env = dict(os.environ, GD_HIP_HOST_VISIBLE="1")
    r = subprocess.run([exe, src, dst, str(seed), ckpt], env=env, capture_output=True, text=True, timeout=300)
    print(r.stdout, r.stderr)
    if r.returncode != 0:
        raise SystemExit(r.returncode)
    print("wrote", ckpt, os.path.getsize(ckpt), "bytes")


if __name__ == "__main__":
    main()
