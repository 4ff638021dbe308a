"""Writes the tokenizer fixtures with the reference's OWN tokenizer code.

Runs oracle/_ref/ref_tokenizer (oracle/ref_tokenizer.c linked with the reference's src/tokenizer/*.c by
`make -C oracle ref-tests`; pure host code, no GPU needed): trains a 420-entry byte-level BPE vocabulary on the corpus
below with the reference's trainer, saves it with the reference's writer and encodes the test texts with the
reference's encoder under (split_digits, allow_special) = (1,1), (1,0), (0,1).  Outputs, next to this script:

  tokenizer_small.json    the vocabulary file as the reference wrote it
  tokenizer_cases.npz     texts (uint8 arrays), expected ids per configuration, vocabulary hash, special ids
"""
import os
import subprocess
import sys
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
SPECIALS = ["<eot>", "<pad>", "<|user|>"]

CORPUS = """the quick brown fox jumps over the lazy dog. The dog sleeps; the fox does not.
hello hello hello <eot>
byte-level BPE tokenizer test 123 123 123 and 4567 tokens, tokenizer tokenizer tokenizer
<|user|> what is 12 + 30? <eot> it is 42. <eot>
naive cafe, naïve café, über, straße, 日本語 の テキスト, русский текст
tabs\tand\ttabs,  double  spaces,   triple   spaces
punctuation!!! ... --- ??? (parentheses) [brackets] {braces} "quotes" 'single'
snake_case camelCase SCREAMING_CASE kebab-case 3.14159 2024-11-25 10:30:00
""" * 6


TEXTS = [
    "hello <eot> 123 hello",
    "hello <eot>",
    "",
    " ",
    "  leading and trailing  ",
    "the quick brown fox",
    "The Quick Brown Fox 2024",
    "a1b22c333 d4444",
    "x=3.14159;y=-2e10",
    "<eot><eot> <pad><|user|>hi<eot>",
    "<eo t> <eot <|user| >",
    "café naïve 日本語のテキスト русский",
    "tabs\tand\nnewlines\r\n\n\nend",
    "   \t \n  mixed   whitespace\t\t",
    "!!!???...---",
    "snake_case camelCase kebab-case",
    "tokenizer tokenizer tokenizer tokenizer",
    "z" * 300,
    " " * 270 + "x",
    "ab" * 200 + " 9" * 50,
    "emoji \U0001f600\U0001f680 and  nbsp",
    "1 2 3  4   5 <pad> 6",
    "<|user|> what is 12 + 30? <eot> it is 42. <eot>",
]


def main():
    exe = os.path.join(ROOT, "oracle", "_ref", "ref_tokenizer")
    out_dir = sys.argv[1] if len(sys.argv) > 1 else HERE
    raw_texts = [t.encode("utf-8") for t in TEXTS] + [bytes(range(1, 256)), bytes([0xff, 0xfe, 0x80, 0x20, 0x80])]
    with tempfile.TemporaryDirectory() as tmp:
        corpus, texts, res = (os.path.join(tmp, n) for n in ("corpus.txt", "texts.bin", "out.bin"))
        with open(corpus, "wb") as f:
            f.write(CORPUS.encode("utf-8"))
        with open(texts, "wb") as f:
            np.array([len(raw_texts)], np.int32).tofile(f)
            for t in raw_texts:
                np.array([len(t)], np.int32).tofile(f)
                f.write(t)
        json_path = os.path.join(out_dir, "tokenizer_small.json")
        r = subprocess.run([exe, corpus, "420", json_path, texts, res] + SPECIALS, capture_output=True, text=True,
                           timeout=120)
        print(r.stdout, r.stderr)
        if r.returncode != 0:
            raise SystemExit(r.returncode)
        raw = np.fromfile(res, np.uint8)
    at = 0

    def take(dtype, n=1):
        nonlocal at
        size = np.dtype(dtype).itemsize * n
        v = raw[at:at + size].view(dtype)
        at += size
        return v

    out = {"hash": take(np.uint64).view(np.uint32).copy(), "vocab_size": take(np.int32).copy()}
    n_specials = int(take(np.int32)[0])
    out["special_ids"] = take(np.int32, n_specials).copy()
    out["specials"] = np.frombuffer("\n".join(SPECIALS).encode(), np.uint8)
    for c in range(3):
        for i, t in enumerate(raw_texts):
            n = int(take(np.int32)[0])
            out[f"ids_{c}_{i}"] = take(np.int32, n).copy()
            dlen = int(take(np.int32)[0])
            assert dlen == len(t), (c, i, dlen, len(t))        # the reference's decode gives the text back
    assert at == raw.size
    for i, t in enumerate(raw_texts):
        out[f"text_{i}"] = np.frombuffer(t, np.uint8)
    path = os.path.join(out_dir, "tokenizer_cases.npz")
    np.savez_compressed(path, **out)
    print("wrote", json_path, os.path.getsize(json_path), "bytes;", path, os.path.getsize(path), "bytes;", len(raw_texts), "texts")


if __name__ == "__main__":
    main()
