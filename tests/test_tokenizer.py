"""The byte-level BPE tokenizer against the reference's own tokenizer, without a GPU.

tests/golden/tokenizer_small.json is a vocabulary the reference's trainer produced and its writer saved;
tests/golden/tokenizer_cases.npz holds what the reference's encoder returned for 25 texts under three configurations
(tests/golden/make_tokenizer_fixture.py ran them through oracle/_ref/ref_tokenizer).  The remaining checks are the
reference's own test (tests/test_tokenizer.c:120-175: round trip, special matched / literal, bad id) and properties
that hold for any byte-level BPE (decode(encode(x)) == x, pieces never span a special, merges only inside a piece).
"""
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
VOCAB = os.path.join(HERE, "golden", "tokenizer_small.json")
CONFIGS = [(1, 1), (1, 0), (0, 1)]
GD_ERR_INVALID_ARGUMENT, GD_ERR_UNSUPPORTED, GD_ERR_IO = -1, -6, -9


@pytest.fixture(scope="module")
def T(host):
    import importlib
    return importlib.import_module("gradients_c_amd_host.tokenizer")


@pytest.fixture(scope="module")
def cases():
    return np.load(os.path.join(HERE, "golden", "tokenizer_cases.npz"))


def test_vocabulary_loads_like_the_reference(T, cases):
    tok = T.Tokenizer(VOCAB)                                     # NULL configuration: split_digits from the file
    assert tok.vocab_size == int(cases["vocab_size"][0]) == 420
    assert tok.hash == int(cases["hash"].view(np.uint64)[0])
    with open(VOCAB) as f:
        assert f'"hash": "{tok.hash:016x}"' in f.read()
    specials = bytes(cases["specials"]).decode().split("\n")
    assert [tok.token_id(s) for s in specials] == list(cases["special_ids"]) == [256, 257, 258]
    # the digest covers split_digits, nothing else of the configuration
    assert T.Tokenizer(VOCAB, 1, 0).hash == tok.hash and T.Tokenizer(VOCAB, 0, 1).hash != tok.hash


def test_encoding_equals_the_reference_encoder(T, cases):
    n_texts = sum(1 for k in cases.files if k.startswith("text_"))
    assert n_texts == 25
    for c, (split, special) in enumerate(CONFIGS):
        tok = T.Tokenizer(VOCAB, split, special)
        for i in range(n_texts):
            text = bytes(cases[f"text_{i}"])
            got = tok.encode(text)
            assert np.array_equal(got, cases[f"ids_{c}_{i}"]), (c, i, text[:40], got[:12], cases[f"ids_{c}_{i}"][:12])
            assert tok.decode(got) == text, (c, i)


def test_reference_test_program_cases(T):
    tok = T.Tokenizer(VOCAB, 1, 1)
    eot = tok.token_id("<eot>")
    ids = tok.encode("hello <eot> 123 hello")
    assert eot in ids and tok.decode(ids) == b"hello <eot> 123 hello"
    literal = T.Tokenizer(VOCAB, 1, 0)
    ids = literal.encode("hello <eot>")
    assert eot not in ids and literal.decode(ids) == b"hello <eot>"
    import gradients_c_amd_host as pkg
    for bad in ([-1], [420], [5, 100000]):
        with pytest.raises(pkg.GdError) as err:
            tok.decode(bad)
        assert err.value.status == GD_ERR_INVALID_ARGUMENT
    with pytest.raises(pkg.GdError) as err:
        tok.token_id("<nope>")
    assert err.value.status == GD_ERR_INVALID_ARGUMENT
    assert tok.encode("").size == 0 and tok.decode([]) == b""


def test_round_trip_and_piece_rules_on_random_bytes(T):
    rng = np.random.default_rng(12)
    alphabet = list(b"ab z09 \n\t.-<>|eotpadusr") + [0xc3, 0xa9, 0xe6, 0x97, 0xa5, 0xff]
    for split, special in CONFIGS:
        tok = T.Tokenizer(VOCAB, split, special)
        specials = {tok.token_id(s) for s in ("<eot>", "<pad>", "<|user|>")}
        for _ in range(300):
            text = bytes(rng.choice(alphabet, int(rng.integers(0, 120))).tolist())
            ids = tok.encode(text)
            assert tok.decode(ids) == text
            if not special:
                assert not specials & set(ids.tolist())
            if split:                                            # a digit never shares a token with anything
                for t in ids:
                    piece = tok.decode([t])
                    assert len(piece) == 1 or not any(48 <= b <= 57 for b in piece) or int(t) in specials, piece
        # every single byte encodes to itself (ids 0-255 are the bytes)
        for b in range(1, 256):
            assert tok.encode(bytes([b])).tolist() == [b]


def test_greedy_merge_order_on_a_hand_made_vocabulary(T, tmp_path):
    """Lowest merged id first, leftmost among equals: with merges ab -> 256, bc -> 257, (256)c -> 258 the text
    "abc" is ab+c -> 258; with the first two swapped it is a+bc (the pair a,257 has no merge)."""
    def vocab(merges, extra=""):
        lines = ['{', '  "format": "gd-bpe-tokenizer-v1",', '  "split_digits": false,', '  "tokens": [']
        lines += ['    {"id":%d,"kind":"byte","hex":"%02x"},' % (i, i) for i in range(256)]
        for n, (l, r, hx) in enumerate(merges):
            lines.append('    {"id":%d,"kind":"merge","left":%d,"right":%d,"hex":"%s"},' % (256 + n, l, r, hx))
        return "\n".join(lines) + extra + "\n  ]\n}\n"

    a, b, c = 97, 98, 99
    p = tmp_path / "t1.json"
    p.write_text(vocab([(a, b, "6162"), (b, c, "6263"), (256, c, "616263")]))
    tok = T.Tokenizer(str(p))
    assert tok.encode("abc").tolist() == [258]                   # whole piece is a token: direct hit
    assert tok.encode("abcab").tolist() == [258, 256]
    assert tok.encode("xabc").tolist() == [120, 258]
    p.write_text(vocab([(b, c, "6263"), (a, b, "6162"), (257, c, "616263")]))
    tok = T.Tokenizer(str(p))
    assert tok.encode("xabc").tolist() == [120, a, 256]          # bc merges first, then a|bc has no merge
    assert tok.encode("abab").tolist() == [257, 257]
    assert tok.encode("aab").tolist() == [a, 257]
    # split_digits comes from the file when no configuration is given
    assert tok.encode("a12").tolist() == [a, 49, 50]
    p.write_text(vocab([(49, 50, "3132")]))
    assert T.Tokenizer(str(p)).encode("a12").tolist() == [a, 256]
    assert T.Tokenizer(str(p), 1, 1).encode("a12").tolist() == [a, 49, 50]


def test_loader_refuses_malformed_files(T, tmp_path):
    import gradients_c_amd_host as pkg
    good = open(VOCAB).read()

    def status_of(text):
        p = tmp_path / "bad.json"
        p.write_text(text)
        with pytest.raises(pkg.GdError) as err:
            T.Tokenizer(str(p))
        return err.value.status

    assert status_of(good.replace('{"id":7,', '{"id":8,', 1)) == GD_ERR_INVALID_ARGUMENT        # ids out of sequence
    assert status_of(good.replace('"hex":"41"', '"hex":"4"', 1)) == GD_ERR_INVALID_ARGUMENT      # odd hex length
    assert status_of(good.replace('"hex":"41"', '"hex":"4g"', 1)) == GD_ERR_INVALID_ARGUMENT     # not hex
    assert status_of(good.replace('"hex":"41"', '"hex":"4142"', 1)) == GD_ERR_INVALID_ARGUMENT   # byte token of 2 bytes
    assert status_of(good.replace('"text":"<pad>"', '"text":"<pa\\u0064>"', 1)) == GD_ERR_UNSUPPORTED
    assert status_of(good.replace('"text":"<pad>"', '"text":"<pad>', 1)) == GD_ERR_INVALID_ARGUMENT  # unterminated
    assert status_of(good.replace('"text":"<pad>"', '"text":""', 1)) == GD_ERR_INVALID_ARGUMENT  # empty token
    assert status_of("\n".join(good.split("\n")[:100])) == GD_ERR_INVALID_ARGUMENT               # fewer than 256 tokens
    assert status_of("") == GD_ERR_INVALID_ARGUMENT
    with pytest.raises(pkg.GdError) as err:
        T.Tokenizer(str(tmp_path / "absent.json"))
    assert err.value.status == GD_ERR_IO
    # escapes the reference's writer produces are read back
    p = tmp_path / "esc.json"
    p.write_text(good.replace('"text":"<pad>"', '"text":"<\\"p\\\\a\\n\\t\\rd>"', 1))
    tok = T.Tokenizer(str(p))
    assert tok.decode([257]) == b'<"p\\a\n\t\rd>' and tok.encode('x<"p\\a\n\t\rd>y').tolist()[1] == 257
