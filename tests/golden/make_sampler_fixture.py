"""Writes tests/golden/sampler_cases.npz with the reference's OWN host sampler.

Runs oracle/_ref/ref_sampler (oracle/ref_sampler.c around the reference's examples/gpt_lm/gpt_lm_shared.c, built by
`make -C oracle ref-tests`; pure host code, no GPU needed) on seeded logits, histories and parameter sets.  Per case
the file holds the inputs (logits, hist_len, history, params = temperature, min_p, penalty, softcap, rng as two
uint32 halves) and what the reference produced (tokens, rng_after, logits_after)."""
import os
import subprocess
import sys
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))

PARAMS = [  # temperature, min_p, penalty, softcap
    (0.8, 0.05, 1.3, 20.0),
    (1.0, 0.0, 1.0, 0.0),
    (0.0, 0.0, 1.5, 0.0),
    (2.5, 0.5, 1.0, 5.0),
    (0.3, 1.0, 1.1, 0.0),
    (float("nan"), 0.0, float("inf"), -1.0),
    (1.7, 0.0, 0.5, 30.0),
]


def main():
    exe = os.path.join(ROOT, "oracle", "_ref", "ref_sampler")
    out = {}
    with tempfile.TemporaryDirectory() as tmp:
        for case, par in enumerate(PARAMS):
            rng = np.random.default_rng(100 + case)
            rows, vocab, cap = 12, 96, 16
            logits = rng.normal(0, 4, (rows, vocab)).astype(np.float16).astype(np.float32)
            logits[1, 5] = np.nan
            logits[1, 9] = np.inf
            logits[2, :] = np.nan                       # nothing finite: token 0, no draw
            logits[3, 7] = logits[3, 70] = 11.0         # tied leaders
            logits[4, :] = -np.inf
            logits[4, 33] = -2.0                        # one finite value
            logits[5, :] = 0.0                          # uniform
            hist_len = rng.integers(0, cap + 1, rows).astype(np.int32)
            history = rng.integers(0, 30, (rows, cap)).astype(np.int32)
            history[6, 0] = -4
            history[6, 1] = vocab + 2                   # out of range entries are ignored
            state = np.uint64(0x9e3779b97f4a7c15 * (case + 1) % (1 << 64))
            src, dst = os.path.join(tmp, "in.bin"), os.path.join(tmp, "out.bin")
            with open(src, "wb") as f:
                np.array([rows, vocab, cap], np.int32).tofile(f)
                np.array(par, np.float32).tofile(f)
                np.array([state], np.uint64).tofile(f)
                logits.tofile(f)
                hist_len.tofile(f)
                history.tofile(f)
            r = subprocess.run([exe, src, dst], capture_output=True, text=True, timeout=60)
            if r.returncode != 0:
                raise SystemExit(r.stdout + r.stderr)
            raw = np.fromfile(dst, np.uint8)
            tokens = raw[:4 * rows].view(np.int32)
            after = raw[4 * rows:12 * rows].view(np.uint64)
            logits_after = raw[12 * rows:].view(np.float32).reshape(rows, vocab)
            out.update({f"c{case}_logits": logits, f"c{case}_hist_len": hist_len, f"c{case}_history": history,
                        f"c{case}_params": np.array(par, np.float32),
                        f"c{case}_rng": np.array([state], np.uint64).view(np.uint32),
                        f"c{case}_tokens": tokens.copy(), f"c{case}_rng_after": after.copy().view(np.uint32),
                        f"c{case}_logits_after": logits_after.copy()})
    path = os.path.join(sys.argv[1] if len(sys.argv) > 1 else HERE, "sampler_cases.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(PARAMS), "cases")


if __name__ == "__main__":
    main()
