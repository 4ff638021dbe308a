"""Writes tests/golden/minimax_cases.npz with the reference's OWN in-test models of the MiniMax-M3 operators.

Runs oracle/_ref/ref_minimax (oracle/ref_minimax.c around the reference's tests/test_minimax_m3_sparse_attention.c,
built by `make -C oracle ref-tests`; pure host code): ref_topk picks the blocks, ref_sparse_fwd / ref_sparse_fwd_gqa
attend over them.  Cases 0 and 1 are the two forward cases of the reference's test program itself (its fill_tokens
inputs); the others are seeded random inputs at several shapes.  Per case the file holds the inputs (head, scale,
cu, q, k, v as uint16 bits, topk_in if given) and the reference's results (topk, out)."""
import os
import subprocess
import sys
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))


def fill_tokens(count, base):
    """tests/test_minimax_m3_sparse_attention.c:119-126"""
    i = np.arange(count, dtype=np.uint32)
    x = np.float32(base) + np.float32(0.046875) * ((i * 13 + 5) % 17).astype(np.float32) \
        - np.float32(0.03125) * (i % 7).astype(np.float32)
    return x.astype(np.float16)


def cases():
    out = []
    # the reference's test_sparse_fwd_bwd forward part (:695-763)
    N, H, Dh = 6, 2, 4
    out.append(dict(B=2, Hq=H, Hkv=H, Dh=Dh, block=2, topk=2, init=1, local=1, scale=0.5, cu=[0, 3, 6],
                    q=fill_tokens(N * H * Dh, -0.25), k=fill_tokens(N * H * Dh, 0.125), v=fill_tokens(N * H * Dh, -0.375)))
    # the reference's test_sparse_gqa forward part (:603-678): block lists given by the test
    N, Hq, Hkv, Dh, TOPK = 5, 4, 2, 4, 8
    given = np.full((Hkv, N, TOPK), -1, np.int32)
    for i in range(N):
        valid = (i + 2) // 2
        given[:, i, 0] = 0
        given[:, i, 1] = valid - 1 if valid > 1 else -1
    out.append(dict(B=1, Hq=Hq, Hkv=Hkv, Dh=Dh, block=2, topk=TOPK, init=0, local=0, scale=0.5, cu=[0, N],
                    q=fill_tokens(N * Hq * Dh, -0.1875), k=fill_tokens(N * Hkv * Dh, 0.09375),
                    v=fill_tokens(N * Hkv * Dh, -0.28125), topk_in=given))
    rng = np.random.default_rng(2024)
    for (lens, H, Dh, block, topk, init, local) in [([37, 5, 64], 2, 16, 8, 4, 1, 1), ([70], 3, 8, 4, 4, 0, 0),
                                                    ([130, 1, 33], 2, 64, 16, 3, 2, 2), ([256], 1, 32, 128, 2, 1, 1),
                                                    ([90, 90], 2, 16, 8, 1, 0, 1), ([50], 2, 16, 8, 4, 0, 3)]:
        N = sum(lens)
        out.append(dict(B=len(lens), Hq=H, Hkv=H, Dh=Dh, block=block, topk=topk, init=init, local=local,
                        scale=float(1.0 / np.sqrt(Dh)), cu=np.concatenate([[0], np.cumsum(lens)]).tolist(),
                        q=rng.normal(0, 1, N * H * Dh).astype(np.float16), k=rng.normal(0, 1, N * H * Dh).astype(np.float16),
                        v=rng.normal(0, 1, N * H * Dh).astype(np.float16)))
    return out


def main():
    exe = os.path.join(ROOT, "oracle", "_ref", "ref_minimax")
    store = {}
    with tempfile.TemporaryDirectory() as tmp:
        for n, c in enumerate(cases()):
            src, dst = os.path.join(tmp, "in.bin"), os.path.join(tmp, "out.bin")
            given = c.get("topk_in")
            head = np.array([c["B"], c["Hq"], c["Hkv"], c["Dh"], c["block"], c["topk"], c["init"], c["local"],
                             0 if given is None else 1], np.int32)
            with open(src, "wb") as f:
                head.tofile(f)
                np.array([c["scale"]], np.float32).tofile(f)
                np.array(c["cu"], np.int32).tofile(f)
                for name in ("q", "k", "v"):
                    c[name].view(np.uint16).tofile(f)
                if given is not None:
                    given.tofile(f)
            r = subprocess.run([exe, src, dst], capture_output=True, text=True, timeout=300)
            if r.returncode != 0:
                raise SystemExit(r.stdout + r.stderr)
            N = c["cu"][-1]
            raw = np.fromfile(dst, np.uint8)
            nt = c["Hkv"] * N * c["topk"]
            store[f"c{n}_head"] = head
            store[f"c{n}_scale"] = np.array([c["scale"]], np.float32)
            store[f"c{n}_cu"] = np.array(c["cu"], np.int32)
            for name in ("q", "k", "v"):
                store[f"c{n}_{name}"] = c[name].view(np.uint16)
            if given is not None:
                store[f"c{n}_topk_in"] = given
            store[f"c{n}_topk"] = raw[:4 * nt].view(np.int32).reshape(c["Hkv"], N, c["topk"]).copy()
            store[f"c{n}_out"] = raw[4 * nt:].view(np.float32).reshape(N, c["Hq"], c["Dh"]).copy()
    path = os.path.join(sys.argv[1] if len(sys.argv) > 1 else HERE, "minimax_cases.npz")
    np.savez_compressed(path, **store)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
