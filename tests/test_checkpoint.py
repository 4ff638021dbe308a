"""The .gdckpt reader and the decoder's checkpoint loader, without a GPU.

The file under test is tests/golden/gpt_small_seed777.gdckpt, written by the reference's own gd_module_save_state
(tests/golden/make_gdckpt_fixture.py).  The library is the device-less build of the product's C sources (tests/host).
Damaged files are made here by editing bytes of that fixture; the expected status of each follows the reference's
reader (src/nn/module_io.c:424-459, 491-561, 868-899) as its tests exercise it (tests/test_module_io.c:60-190:
round trip of values and metadata, strict load refusing a shape mismatch, non-strict load).
"""
import os
import struct

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
CKPT = os.path.join(HERE, "golden", "gpt_small_seed777.gdckpt")
GD_ERR_INVALID_ARGUMENT, GD_ERR_BUSY, GD_ERR_BAD_STATE, GD_ERR_IO = -1, -4, -5, -9
DIMS = dict(vocab=64, d_model=64, n_layers=2, n_heads=2, head_dim=32, mlp_hidden=128, max_seq=64, batch=2)
ENTRY_FIXED = 96


def small_config(D, **over):
    d = dict(DIMS, **over)
    return D.gpt_config(d["vocab"], d["d_model"], d["n_layers"], d["n_heads"], d["head_dim"], d["mlp_hidden"],
                        d["max_seq"], d["batch"], 0, over.get("tie", True), over.get("seed", 5))


def parse(raw):
    """Independent pure-Python walk over header and directory (the format is fixed by the file itself: the offsets
    below were read off the fixture's bytes and the reference writer, not off the C reader under test)."""
    assert raw[:8] == b"GDCKPT1\0"
    version, header_size, count, dir_off, dir_size, meta_off, meta_len, data_off = struct.unpack_from("<II6Q", raw, 8)
    entries, at = [], dir_off
    for _ in range(count):
        path_len, flags, dtype, rank = struct.unpack_from("<4I", raw, at)
        shape = struct.unpack_from("<8Q", raw, at + 16)
        offset, nbytes = struct.unpack_from("<2Q", raw, at + 80)
        path = raw[at + ENTRY_FIXED:at + ENTRY_FIXED + path_len].decode()
        entries.append(dict(at=at, path=path, flags=flags, dtype=dtype, rank=rank, shape=shape[:rank], offset=offset,
                            nbytes=nbytes))
        at += ENTRY_FIXED + path_len
    assert at == dir_off + dir_size
    return dict(version=version, header_size=header_size, count=count, dir_off=dir_off, dir_size=dir_size,
                meta_off=meta_off, meta_len=meta_len, data_off=data_off, entries=entries)


@pytest.fixture(scope="module")
def raw():
    with open(CKPT, "rb") as f:
        return f.read()


def expected_paths(layers):
    paths = ["gpt_lm.token_embedding", "gpt_lm.lm_head_bias", "gpt_lm.final_norm_w"]
    for l in range(layers):
        paths += [f"gpt_lm.blocks.{l}.{n}" for n in (
            "attn_norm_w", "mlp_norm_w", "qkv_proj.weight", "qkv_proj.bias", "attn_proj.weight", "attn_proj.bias",
            "up_gate.weight", "up_gate.bias", "down_proj.weight", "down_proj.bias")]
    return paths


NAMES = {"attn_norm_w": "attn_norm", "mlp_norm_w": "mlp_norm", "qkv_proj.weight": "w_qkv", "qkv_proj.bias": "b_qkv",
         "attn_proj.weight": "w_attn", "attn_proj.bias": "b_attn", "up_gate.weight": "w_upgate",
         "up_gate.bias": "b_upgate", "down_proj.weight": "w_down", "down_proj.bias": "b_down"}


def decoder_tensor_of(path):
    """(decoder tensor name, layer) of a checkpoint path."""
    tail = path[len("gpt_lm."):]
    if tail == "token_embedding":
        return "embed", 0
    if tail == "lm_head_bias":
        return "lm_bias", 0
    if tail == "final_norm_w":
        return "final_norm", 0
    _, layer, name = tail.split(".", 2)
    return NAMES[name], int(layer)


# ---- reader -------------------------------------------------------------------------------------------------------

def test_reader_lists_what_the_reference_wrote(host, raw):
    _, D = host
    want = parse(raw)
    with D.Checkpoint(CKPT) as ck:
        assert len(ck) == want["count"] == 23
        got = ck.entries()
        assert sorted(ck.paths()) == sorted(expected_paths(2))
        for e, w in zip(got, want["entries"]):
            assert e.path.decode() == w["path"]
            assert (e.flags, e.dtype, e.rank) == (w["flags"], w["dtype"], w["rank"]) == (1, 1, w["rank"])
            assert tuple(e.shape[i] for i in range(e.rank)) == w["shape"]
            assert (e.data_offset, e.nbytes) == (w["offset"], w["nbytes"])
            data = ck.read(w["path"])
            assert data.dtype == np.float16 and data.shape == w["shape"]
            assert data.tobytes() == raw[w["offset"]:w["offset"] + w["nbytes"]]
        assert ck.metadata() == raw[want["meta_off"]:want["meta_off"] + want["meta_len"]]
        assert ck.metadata() == b'{"writer":"gd_module_save_state","model":"gpt_lm"}'
        with pytest.raises(KeyError):
            ck.read("gpt_lm.blocks.2.attn_norm_w")


def test_reader_ranges(host):
    _, D = host
    import ctypes as C
    with D.Checkpoint(CKPT) as ck:
        p = D.lib().gd_checkpoint_find(ck.handle, b"gpt_lm.final_norm_w")
        buf = np.zeros(256, np.uint8)
        assert D.lib().gd_checkpoint_read(ck.handle, p, 120, buf.ctypes.data_as(C.c_void_p), 8) == 0
        assert D.lib().gd_checkpoint_read(ck.handle, p, 121, buf.ctypes.data_as(C.c_void_p), 8) == GD_ERR_INVALID_ARGUMENT
        assert D.lib().gd_checkpoint_read(ck.handle, p, 129, buf.ctypes.data_as(C.c_void_p), 0) == GD_ERR_INVALID_ARGUMENT
        assert D.lib().gd_checkpoint_read(ck.handle, p, 128, buf.ctypes.data_as(C.c_void_p), 0) == 0
        foreign = D.CheckpointEntry()
        assert D.lib().gd_checkpoint_read(ck.handle, C.byref(foreign), 0, buf.ctypes.data_as(C.c_void_p),
                                          0) == GD_ERR_INVALID_ARGUMENT


def test_fixture_weights_are_the_seeded_initialisation(host, oracle):
    """The reference initialised the saved model from seed 777: its bytes must equal the oracle's restatement of that
    initialisation (this also pins the oracle's weight streams against bytes the reference itself wrote)."""
    _, D = host
    ref = oracle.Decoder(64, 64, 2, 2, 32, 128, 64, 2, 0, 777, True)
    try:
        with D.Checkpoint(CKPT) as ck:
            for path in ck.paths():
                name, layer = decoder_tensor_of(path)
                assert np.array_equal(ck.read(path).view(np.uint16).ravel(),
                                      ref.tensor(name, layer).view(np.uint16).ravel()), path
    finally:
        ref.close()


# ---- loader -------------------------------------------------------------------------------------------------------

def snapshot(dev, layers=2):
    out = {}
    for name in ("embed", "lm_head", "lm_bias", "final_norm"):
        out[name, 0] = dev.read_tensor(name).copy()
    for l in range(layers):
        for name in list(NAMES.values()) + ["w_down_t"]:
            out[name, l] = dev.read_tensor(name, l).copy()
    return out


@pytest.mark.parametrize("tie", [True, False])
def test_loader_replaces_every_weight(host, tie):
    _, D = host
    dev = D.GptDecoder(small_config(D, tie=tie, seed=5))
    try:
        before = snapshot(dev)
        dev.load_checkpoint(CKPT)
        after = snapshot(dev)
        with D.Checkpoint(CKPT) as ck:
            for path in ck.paths():
                key = decoder_tensor_of(path)
                want = ck.read(path)
                assert np.array_equal(after[key].view(np.uint16).ravel(), want.view(np.uint16).ravel()), path
                if "weight" in path or "embedding" in path:
                    assert not np.array_equal(before[key], after[key]), path
            for l in (0, 1):
                down = ck.read(f"gpt_lm.blocks.{l}.down_proj.weight")  # [hidden, d_model]
                assert np.array_equal(after["w_down_t", l].reshape(64, 128).view(np.uint16), down.T.view(np.uint16))
            # the reference's head is its embedding table
            assert np.array_equal(after["lm_head", 0].view(np.uint16).ravel(),
                                  ck.read("gpt_lm.token_embedding").view(np.uint16).ravel())
    finally:
        dev.close()


def damaged(tmp_path, raw, name, edit):
    data = bytearray(raw)
    cut = edit(data)
    if cut is not None:
        data = cut
    p = tmp_path / name
    p.write_bytes(bytes(data))
    return str(p)


def put(fmt, offset, *values):
    def edit(data):
        struct.pack_into(fmt, data, offset, *values)
    return edit


def test_reader_refuses_damaged_files(host, raw, tmp_path):
    pkg, D = host
    info = parse(raw)
    e0, e1 = info["entries"][0], info["entries"][1]
    size = len(raw)

    def rename_to_second(data):
        a = [e for e in info["entries"] if e["path"] == "gpt_lm.blocks.1.attn_norm_w"][0]
        data[a["at"] + ENTRY_FIXED:a["at"] + ENTRY_FIXED + len(a["path"])] = b"gpt_lm.blocks.0.attn_norm_w"

    cases = [
        ("magic", put("<B", 3, 0x58), GD_ERR_BAD_STATE),
        ("version", put("<I", 8, 2), GD_ERR_BAD_STATE),
        ("header_size", put("<I", 12, 128), GD_ERR_BAD_STATE),
        ("dir_before_header", put("<Q", 24, 32), GD_ERR_BAD_STATE),
        ("metadata_before_dir", put("<Q", 40, 8), GD_ERR_BAD_STATE),
        ("data_before_metadata", put("<Q", 56, info["meta_off"] - 1), GD_ERR_BAD_STATE),
        ("count_too_large", put("<Q", 16, 1 << 33), GD_ERR_INVALID_ARGUMENT),
        ("count_one_more", put("<Q", 16, info["count"] + 1), GD_ERR_BAD_STATE),
        ("count_one_less", put("<Q", 16, info["count"] - 1), GD_ERR_BAD_STATE),
        ("dir_size_short", put("<Q", 32, info["dir_size"] - 1), GD_ERR_BAD_STATE),
        ("path_len_zero", put("<I", e0["at"], 0), GD_ERR_BAD_STATE),
        ("path_len_huge", put("<I", e0["at"], 256), GD_ERR_BAD_STATE),
        ("rank_nine", put("<I", e0["at"] + 12, 9), GD_ERR_BAD_STATE),
        ("flags_unknown", put("<I", e0["at"] + 4, 3), GD_ERR_BAD_STATE),
        ("dim_negative", put("<Q", e0["at"] + 16, 1 << 63), GD_ERR_BAD_STATE),
        ("data_before_data_section", put("<Q", e1["at"] + 80, info["data_off"] - 2), GD_ERR_BAD_STATE),
        ("nbytes_not_shape", put("<Q", e1["at"] + 88, e1["nbytes"] + 2), GD_ERR_BAD_STATE),
        ("dtype_unknown", put("<I", e1["at"] + 8, 77), GD_ERR_BAD_STATE),
        ("data_past_end", put("<Q", e1["at"] + 80, size - 2), GD_ERR_BAD_STATE),
        ("path_repeated", rename_to_second, GD_ERR_BAD_STATE),
        ("nul_in_path", put("<B", e0["at"] + ENTRY_FIXED + 2, 0), GD_ERR_BAD_STATE),
        ("dir_size_beyond_file", put("<Q", 32, 1 << 60), GD_ERR_IO),  # refused before anything is allocated for it
        ("cut_in_header", lambda d: d[:40], GD_ERR_IO),
        ("cut_in_magic", lambda d: d[:5], GD_ERR_IO),
        ("cut_in_directory", lambda d: d[:info["dir_off"] + 50], GD_ERR_IO),
        ("empty", lambda d: d[:0], GD_ERR_IO),
    ]
    for name, edit, status in cases:
        path = damaged(tmp_path, raw, name, edit)
        with pytest.raises(pkg.GdError) as err:
            D.Checkpoint(path)
        assert err.value.status == status, name
    with pytest.raises(pkg.GdError) as err:
        D.Checkpoint(str(tmp_path / "absent.gdckpt"))
    assert err.value.status == GD_ERR_IO
    with pytest.raises(pkg.GdError) as err:
        D.Checkpoint("")
    assert err.value.status == GD_ERR_INVALID_ARGUMENT


def test_metadata_reader_checks_the_header_only(host, raw, tmp_path):
    """gd_checkpoint_read_metadata of the reference reads the header and the blob, not the directory."""
    pkg, D = host
    import ctypes as C
    info = parse(raw)
    path = damaged(tmp_path, raw, "bad_dir_good_meta", put("<I", info["entries"][0]["at"], 0))
    blob, n = C.c_void_p(), C.c_size_t()
    assert D.lib().gd_checkpoint_read_metadata(path.encode(), C.byref(blob), C.byref(n)) == 0
    assert C.string_at(blob, n.value) == b'{"writer":"gd_module_save_state","model":"gpt_lm"}'
    assert C.string_at(blob, n.value + 1)[-1:] == b"\0"
    D._libc_free(blob)
    for name, edit, status in [("m_magic", put("<B", 0, 0x58), GD_ERR_BAD_STATE),
                               ("m_cut", lambda d: d[:info["meta_off"] + 3], GD_ERR_IO),
                               ("m_len_beyond_file", put("<Q", 48, 1 << 60), GD_ERR_IO),
                               ("m_offset_beyond_file", put("<Q", 40, 1 << 40), GD_ERR_BAD_STATE)]:
        p = damaged(tmp_path, raw, name, edit)
        assert D.lib().gd_checkpoint_read_metadata(p.encode(), C.byref(blob), C.byref(n)) == status, name
        assert not blob.value and n.value == 0
    assert D.lib().gd_checkpoint_read_metadata(None, C.byref(blob), C.byref(n)) == GD_ERR_INVALID_ARGUMENT
    assert D.lib().gd_checkpoint_read_metadata(path.encode(), None, C.byref(n)) == GD_ERR_INVALID_ARGUMENT


def test_loader_strictness_and_untouched_weights_on_refusal(host, raw, tmp_path):
    pkg, D = host
    info = parse(raw)
    by_path = {e["path"]: e for e in info["entries"]}

    def rename(path, new):
        e = by_path[path]
        assert len(new) == len(path)

        def edit(data):
            data[e["at"] + ENTRY_FIXED:e["at"] + ENTRY_FIXED + len(path)] = new.encode()
        return edit

    def expect_refused(dev, path, status=GD_ERR_BAD_STATE, strict=True):
        before = snapshot(dev, dev.cfg.n_layers)
        with pytest.raises(pkg.GdError) as err:
            dev.load_checkpoint(path, strict=strict)
        assert err.value.status == status
        after = snapshot(dev, dev.cfg.n_layers)
        assert all(np.array_equal(before[k], after[k]) for k in before), "a refused file changed weights"

    # a parameter under another name: unexpected + missing when strict; skipped otherwise
    other = damaged(tmp_path, raw, "renamed", rename("gpt_lm.blocks.1.attn_proj.bias", "gpt_lm.blocks.1.attn_proj.bits"))
    # the last tensor marked as a buffer: ignored, so its parameter is missing
    last = info["entries"][-1]
    as_buffer = damaged(tmp_path, raw, "as_buffer", put("<I", last["at"] + 4, 2))
    dev = D.GptDecoder(small_config(D, seed=9))
    try:
        expect_refused(dev, other)
        expect_refused(dev, as_buffer)
        expect_refused(dev, str(tmp_path / "absent.gdckpt"), GD_ERR_IO)
        kept = dev.read_tensor("b_attn", 1).copy()
        dev.load_checkpoint(other, strict=False)
        with D.Checkpoint(CKPT) as ck:
            assert np.array_equal(dev.read_tensor("w_attn", 1).ravel(), ck.read("gpt_lm.blocks.1.attn_proj.weight").ravel())
        assert np.array_equal(dev.read_tensor("b_attn", 1), kept)
        assert D.lib().gd_gpt_decoder_load_checkpoint(dev.handle, None, 1) == GD_ERR_INVALID_ARGUMENT
        assert D.lib().gd_gpt_decoder_load_checkpoint(None, CKPT.encode(), 1) == GD_ERR_INVALID_ARGUMENT
    finally:
        dev.close()
    # decoders of another shape: metadata mismatch (also when not strict, as in the reference), missing layers,
    # unexpected layers
    for over, strict in [(dict(mlp_hidden=256), True), (dict(mlp_hidden=256), False), (dict(vocab=96), True),
                         (dict(n_layers=3), True), (dict(n_layers=1), True)]:
        dev = D.GptDecoder(small_config(D, **over))
        try:
            expect_refused(dev, CKPT, strict=strict)
        finally:
            dev.close()
    # not strict: a one-layer decoder takes its layer from the two-layer file, a three-layer one keeps its third
    dev = D.GptDecoder(small_config(D, n_layers=3, seed=9))
    try:
        third = dev.read_tensor("w_qkv", 2).copy()
        dev.load_checkpoint(CKPT, strict=False)
        with D.Checkpoint(CKPT) as ck:
            assert np.array_equal(dev.read_tensor("w_qkv", 1).ravel(), ck.read("gpt_lm.blocks.1.qkv_proj.weight").ravel())
        assert np.array_equal(dev.read_tensor("w_qkv", 2), third)
    finally:
        dev.close()
    # same element count, other dtype code in the file (BF16): refused
    e = by_path["gpt_lm.blocks.0.up_gate.weight"]
    bf16 = damaged(tmp_path, raw, "bf16", put("<I", e["at"] + 8, 2))
    dev = D.GptDecoder(small_config(D))
    try:
        expect_refused(dev, bf16)
    finally:
        dev.close()


# ---- model dimensions from the file ------------------------------------------------------------------------------

def with_metadata(raw, blob):
    """The fixture with another metadata blob: the data section moves, so every directory entry's offset and the
    header's data offset move with it (test-side rewrite of the container, independent of the C reader)."""
    info = parse(raw)
    data = bytearray(raw[:info["meta_off"]]) + blob
    new_data_off = (len(data) + 255) // 256 * 256
    data += bytes(new_data_off - len(data)) + raw[info["data_off"]:]
    delta = new_data_off - info["data_off"]
    struct.pack_into("<Q", data, 48, len(blob))
    struct.pack_into("<Q", data, 56, new_data_off)
    for e in info["entries"]:
        struct.pack_into("<Q", data, e["at"] + 80, e["offset"] + delta)
    return bytes(data)


TRAINER_METADATA = (b"model=gpt_lm\nvocab_size=64\ncontext_length=64\nd_model=64\nn_layers=2\nn_heads=2\nhead_dim=32\n"
                    b"mlp_hidden=128\nffn_activation=swiglu\narchitecture=gpt\nsdpa_window=16\ndropout=0.1\n"
                    b"logits_softcap=20\ntokenizer_path=data/tokenizer-v2048.json\n")


def test_config_from_checkpoint(host, raw, tmp_path):
    pkg, D = host
    # the fixture's own metadata has no key=value lines: heads come from the caller
    cfg = D.config_from_checkpoint(CKPT, batch=2, max_seq=48, n_heads=2)
    assert (cfg.vocab, cfg.d_model, cfg.n_layers, cfg.n_heads, cfg.head_dim, cfg.mlp_hidden) == (64, 64, 2, 2, 32, 128)
    assert (cfg.max_seq, cfg.batch, cfg.sdpa_window, cfg.tie_lm_head) == (48, 2, 0, 1)
    assert D.config_from_checkpoint(CKPT, batch=1, max_seq=8, head_dim=16).n_heads == 4
    for bad in (dict(), dict(n_heads=3), dict(n_heads=2, head_dim=16)):
        with pytest.raises(pkg.GdError) as err:
            D.config_from_checkpoint(CKPT, batch=2, max_seq=48, **bad)
        assert err.value.status == GD_ERR_BAD_STATE
    # with the metadata the reference's trainer writes, the file alone is enough
    p = tmp_path / "trainer.gdckpt"
    p.write_bytes(with_metadata(raw, TRAINER_METADATA))
    with D.Checkpoint(str(p)) as ck:
        assert ck.metadata() == TRAINER_METADATA
        assert ck.read("gpt_lm.blocks.1.down_proj.bias").tobytes() == D.Checkpoint(CKPT).read(
            "gpt_lm.blocks.1.down_proj.bias").tobytes()
    cfg = D.config_from_checkpoint(str(p), batch=3)
    assert (cfg.vocab, cfg.d_model, cfg.n_layers, cfg.n_heads, cfg.head_dim, cfg.mlp_hidden) == (64, 64, 2, 2, 32, 128)
    assert (cfg.max_seq, cfg.batch, cfg.sdpa_window) == (64, 3, 16)
    assert D.config_from_checkpoint(str(p), batch=3, max_seq=32).max_seq == 32
    dev = D.GptDecoder(cfg)
    try:
        dev.load_checkpoint(str(p))
    finally:
        dev.close()
    # the second architecture of the reference's example
    q = tmp_path / "m3.gdckpt"
    q.write_bytes(with_metadata(raw, TRAINER_METADATA.replace(b"architecture=gpt\n", b"architecture=minimax_m3\n"
                                b"minimax_m3_block_size=64\nminimax_m3_topk_blocks=4\nminimax_m3_init_blocks=2\n"
                                b"minimax_m3_local_blocks=0\n")))
    m3 = D.config_from_checkpoint(str(q), batch=1)
    assert (m3.m3_block_size, m3.m3_topk_blocks, m3.m3_init_blocks, m3.m3_local_blocks) == (64, 4, 2, 0)
    q.write_bytes(with_metadata(raw, TRAINER_METADATA.replace(b"architecture=gpt\n", b"architecture=minimax_m3\n")))
    m3 = D.config_from_checkpoint(str(q), batch=1)
    assert (m3.m3_block_size, m3.m3_topk_blocks, m3.m3_init_blocks, m3.m3_local_blocks) == (128, 3, 1, 1)
    assert (cfg.m3_block_size, cfg.m3_topk_blocks) == (0, 0)
    # metadata that contradicts the directory
    for key, value in ((b"d_model=64", b"d_model=96"), (b"n_layers=2", b"n_layers=3"), (b"vocab_size=64", b"vocab_size=65"),
                       (b"mlp_hidden=128", b"mlp_hidden=64"), (b"n_heads=2", b"n_heads=3")):
        q = tmp_path / "contradiction.gdckpt"
        q.write_bytes(with_metadata(raw, TRAINER_METADATA.replace(key, value)))
        with pytest.raises(pkg.GdError) as err:
            D.config_from_checkpoint(str(q), batch=1)
        assert err.value.status == GD_ERR_BAD_STATE, key
    with pytest.raises(pkg.GdError) as err:
        D.config_from_checkpoint(str(tmp_path / "absent.gdckpt"), batch=1)
    assert err.value.status == GD_ERR_IO
