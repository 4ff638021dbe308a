"""The operator registry generator (gradients.c_amd/csrc/tools/gen_ops.c) and what it wrote: the enumeration keeps
the reference's numbers (src/ops/op_kind.h:5-41), the greedy pick is appended as 34, the committed generated files
are what the generator produces from the tree, and the rules it shares with the reference's generator (scan rule,
.def grammar, numbers never move) hold on a small made-up tree."""
import ctypes
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "gradients.c_amd", "csrc")

# reference src/ops/op_kind.h:5-41
REFERENCE_IDS = {
    "matmul": 1, "linear": 2, "relu": 3, "add": 4, "mul": 5, "sub": 6, "reduce_mean": 7, "reduce_sum": 8,
    "cross_entropy": 9, "sigmoid": 10, "mse": 11, "huber": 12, "dropout": 13, "sdpa_decode": 14, "sdpa_varlen": 15,
    "concat": 16, "reshape": 17, "permute": 18, "split": 19, "rms_norm": 20, "rope": 21, "embedding": 22,
    "linear_transposed_weight": 23, "powlu": 24, "kv_cache_append": 25, "lm_cross_entropy": 26, "qkv_split_rope": 27,
    "powlu_split_linear": 28, "tanh": 29, "swiglu": 30, "swiglu_split_linear": 31, "minimax_m3_index_topk": 32,
    "minimax_m3_sparse_attention": 33,
}


@pytest.fixture(scope="module")
def gen(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("gen") / "gen_ops")
    subprocess.run(["gcc", "-O1", "-std=gnu11", "-Wall", "-Wextra", "-Werror", "-o", exe,
                    os.path.join(CSRC, "tools", "gen_ops.c")], check=True)
    return exe


def _enum(path):
    text = open(path).read()
    return {m.group(1).lower(): int(m.group(2)) for m in re.finditer(r"GD_OP_([A-Z0-9_]+) = (\d+),", text)}


def test_committed_enumeration_keeps_the_reference_numbers_and_appends_the_greedy_pick():
    ids = _enum(os.path.join(CSRC, "ops", "op_kind.h"))
    for name, number in REFERENCE_IDS.items():
        assert ids[name] == number, name
    assert ids["argmax_rows"] == 34
    assert ids["invalid"] == 0 and ids["count"] == max(v for k, v in ids.items() if k != "count") + 1
    assert len(set(ids.values())) == len(ids)


def test_generated_files_are_up_to_date(gen):
    done = subprocess.run([gen, CSRC, "--check"], capture_output=True, text=True)
    assert done.returncode == 0, done.stderr


def test_unsupported_table_is_the_boundary_minus_what_the_backend_defines(gda):
    """Every symbol of backend_symbols.def is exported by the backend library: by a source file of the backend, or by
    the generated GD_ERR_UNSUPPORTED entry, never by both."""
    listed = [l.split("#")[0].strip() for l in open(os.path.join(CSRC, "backends", "hip", "backend_symbols.def"))]
    listed = [l for l in listed if l]
    stubs = re.findall(r"^GD_UNSUPPORTED_ENTRY\((\w+)\)", open(os.path.join(CSRC, "backends", "hip", "backend_hip_unsupported.c")).read(), re.M)
    assert len(listed) > 100 and set(stubs) < set(listed) and len(stubs) == len(set(stubs))
    lib = ctypes.CDLL(gda.LIB_PATH)
    assert not [n for n in listed if not hasattr(lib, n)]
    for must_be_real in ("gd_backend_sdpa_decode", "gd_backend_kv_cache_append_positions", "gd_backend_matmul_nt",
                         "gd_backend_rms_norm_forward", "gd_backend_add", "gd_backend_concat_to_full"):
        assert must_be_real in listed and must_be_real not in stubs
    # declared at the reference's boundary (src/core/backend.h:259,772,776) although its core calls only the batched
    # forms: a build that pulls them in must fail at run time with GD_ERR_UNSUPPORTED, not at link time
    for declared_only in ("gd_backend_adamw", "gd_backend_amp_unscale", "gd_backend_broadcast_to"):
        assert declared_only in stubs
    assert len(listed) >= 109


def test_lookups_of_the_library(gda):
    lib = ctypes.CDLL(gda.LIB_PATH)
    lib.gd_op_kind_name.restype = ctypes.c_char_p
    lib.gd_op_kind_from_name.argtypes = [ctypes.c_char_p]
    assert lib.gd_op_kind_name(14) == b"sdpa_decode" and lib.gd_op_kind_name(34) == b"argmax_rows"
    assert lib.gd_op_kind_name(0) is None and lib.gd_op_kind_name(999) is None
    assert lib.gd_op_kind_from_name(b"kv_cache_append") == 25 and lib.gd_op_kind_from_name(b"nothing") == 0
    built = {name for name, number in REFERENCE_IDS.items() if lib.gd_op_kind_built(number)}
    assert {"sdpa_decode", "sdpa_varlen", "kv_cache_append", "rms_norm", "qkv_split_rope", "linear",
            "linear_transposed_weight", "swiglu", "swiglu_split_linear", "add", "embedding", "reshape",
            "minimax_m3_index_topk", "minimax_m3_sparse_attention"} <= built
    assert not built & {"relu", "cross_entropy", "dropout", "mse", "permute"}   # reserved numbers: training operators
    assert lib.gd_op_kind_built(34) == 1


def test_rules_on_a_made_up_tree(gen, tmp_path):
    csrc = tmp_path / "csrc"
    for name, files in (("alpha", ["core_alpha.c", "op_alpha.def"]), ("beta", ["autograd_beta.c"]),
                        ("kernels_only", ["hip.txt"]), ("Bad-Name", ["core_Bad-Name.c"])):
        (csrc / "ops" / name).mkdir(parents=True)
        for f in files:
            (csrc / "ops" / name / f).write_text("api = binary   # trailing comment\nbackend=unary\nunknown=1\n" if f.endswith(".def") else "")
    (csrc / "backends" / "hip").mkdir(parents=True)
    (csrc / "backends" / "hip" / "backend_symbols.def").write_text("# list\ngd_backend_one\ngd_backend_two  # stays a stub\n")
    (csrc / "backends" / "hip" / "impl.c").write_text(
        "gd_status gd_backend_one(int a,\n                         int b)\n{\n    return gd_backend_two(a);\n}\n")
    (csrc / "ops" / "op_kind.h").write_text("GD_OP_GONE = 1,\nGD_OP_BETA = 2,\n")
    subprocess.run([gen, str(csrc)], check=True, capture_output=True)
    ids = _enum(csrc / "ops" / "op_kind.h")
    assert ids == {"invalid": 0, "gone": 1, "beta": 2, "alpha": 3, "count": 4}      # kept, reserved, appended
    registry = (csrc / "ops" / "op_registry.c").read_text()
    assert '{GD_OP_ALPHA, "alpha", 1, "binary", "unary"}' in registry and '{GD_OP_GONE, "gone", 0, "custom", "custom"}' in registry
    stubs = (csrc / "backends" / "hip" / "backend_hip_unsupported.c").read_text()
    assert "GD_UNSUPPORTED_ENTRY(gd_backend_two)" in stubs and "GD_UNSUPPORTED_ENTRY(gd_backend_one)" not in stubs
    # a second run changes nothing; a new directory takes the next number and moves none
    assert subprocess.run([gen, str(csrc), "--check"]).returncode == 0
    (csrc / "ops" / "aaa").mkdir()
    (csrc / "ops" / "aaa" / "core_aaa.c").write_text("")
    assert subprocess.run([gen, str(csrc), "--check"], capture_output=True).returncode == 3
    subprocess.run([gen, str(csrc)], check=True, capture_output=True)
    assert _enum(csrc / "ops" / "op_kind.h") == {"invalid": 0, "gone": 1, "beta": 2, "alpha": 3, "aaa": 4, "count": 5}
    shutil.rmtree(csrc / "ops" / "alpha")
    subprocess.run([gen, str(csrc)], check=True, capture_output=True)
    assert _enum(csrc / "ops" / "op_kind.h")["alpha"] == 3 and '{GD_OP_ALPHA, "alpha", 0,' in (csrc / "ops" / "op_registry.c").read_text()
