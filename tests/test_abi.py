"""CPU checks of the C-ABI library: it loads without a GPU, exports every symbol that
include/gd_backend_hip.h declares, and refuses to pretend there is a device."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "gd_backend_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gd_backend_\w+)\s*\(", text)))


def test_header_declares_the_decode_path_entry_points():
    names = _declared_symbols()
    for must in ("gd_backend_create_default", "gd_backend_buffer_create", "gd_backend_scope_begin",
                 "gd_backend_record_fence", "gd_backend_upload", "gd_backend_download", "gd_backend_fill",
                 "gd_backend_embedding_forward", "gd_backend_rms_norm_forward", "gd_backend_matmul_nt",
                 "gd_backend_matmul", "gd_backend_linear", "gd_backend_add", "gd_backend_qkv_split_rope_forward",
                 "gd_backend_kv_cache_append_at", "gd_backend_kv_cache_append_positions",
                 "gd_backend_kv_cache_append_packed", "gd_backend_sdpa_decode", "gd_backend_sdpa_decode_at",
                 "gd_backend_sdpa_decode_positions", "gd_backend_swiglu_split_forward", "gd_backend_sdpa_varlen",
                 "gd_backend_argmax_rows", "gd_backend_swiglu_split_linear"):
        assert must in names


def test_library_exports_every_declared_symbol(gda):
    lib = ctypes.CDLL(gda.LIB_PATH)
    missing = [n for n in _declared_symbols() if not hasattr(lib, n)]
    assert not missing, missing


def test_library_exports_the_host_core_decoder_and_checkpoint_symbols(gda):
    """Every function the other public headers declare (host core, decoder, checkpoint reader) is exported too;
    functions defined in a header (static inline) are not library symbols."""
    lib = ctypes.CDLL(gda.LIB_PATH)
    for header in ("gradients_infer.h", "gd_gpt_decoder.h", "gd_checkpoint.h", "gd_tokenizer.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        text = re.sub(r"static inline[^{;]*\{.*?\n\}", "", text, flags=re.S)
        text = "\n".join(l for l in text.splitlines() if not l.lstrip().startswith("#"))
        names = sorted(set(re.findall(r"\b(gd_\w+)\s*\(", text)))
        assert len(names) >= 7, header
        missing = [n for n in names if not hasattr(lib, n)]
        assert not missing, (header, missing)
    for must in ("gd_gpt_decoder_load_checkpoint", "gd_checkpoint_read_metadata", "gd_checkpoint_open",
                 "gd_gpt_decoder_generate", "gd_bpe_tokenizer_load", "gd_tokenizer_encode", "gd_tokenizer_decode"):
        assert hasattr(lib, must)


def test_python_binding_covers_the_header(gda):
    assert set(_declared_symbols()) == set(gda.EXPORTED_SYMBOLS)


def test_struct_layouts_match_the_c_abi(gda):
    # sizes follow from the field lists of reference src/core/backend.h:21-28,45-50,132-140,528-537,671-689
    assert ctypes.sizeof(gda.TensorView) == 8 + 8 + 8 + 4 + 4 + 64 + 64
    assert ctypes.sizeof(gda.MatrixView) == 40
    assert ctypes.sizeof(gda.VectorView) == 24
    assert ctypes.sizeof(gda.RmsNormArgs) == 48
    assert ctypes.sizeof(gda.SdpaVarlenArgs) == 24
    assert ctypes.sizeof(gda.SdpaDecodeArgs) == 16
    assert ctypes.sizeof(gda.EmbeddingArgs) == 24


def test_no_device_means_unsupported_not_fallback(gda):
    import subprocess
    import sys
    # in a child process with the GPU hidden, creation must fail with GD_ERR_UNSUPPORTED
    code = ("import sys; sys.path.insert(0, %r); from conftest import load_package; g = load_package()\n"
            "try:\n    g.Backend()\nexcept g.GdError as e:\n    sys.exit(0 if e.status == g.UNSUPPORTED else 3)\n"
            "sys.exit(4)\n") % os.path.join(ROOT, "tests")
    env = dict(os.environ, HIP_VISIBLE_DEVICES="-1", ROCR_VISIBLE_DEVICES="-1")
    r = subprocess.run([sys.executable, "-c", code], env=env)
    assert r.returncode == 0


def test_product_package_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "gradients.c_amd")
    for dirpath, _, files in os.walk(pkg):
        if os.sep + "build" in dirpath:
            continue
        for f in files:
            if f.endswith((".py", ".c", ".h", ".hip", ".cpp")) or f == "Makefile":
                text = open(os.path.join(dirpath, f), errors="replace").read()
                assert "gd_oracle" not in text and "libgd_oracle" not in text and "oracle/" not in text, f
                # nor the device-less test backend: the product has no CPU path
                assert "null_backend" not in text and "libgradients_host" not in text and "tests/host" not in text, f
