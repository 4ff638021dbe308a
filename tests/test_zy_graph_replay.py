"""The library's opt-in for the HIP runtime's node-by-node graph replay (GD_HIP_GRAPH_NODE_REPLAY=1, what bench.py
runs under): a process that asks for it generates the same tokens as one that leaves the runtime's default.  The
variable is read when the runtime starts, so each setting gets a process of its own: gradients.c_amd/gpt_lm_infer on the
checkpoint and tokenizer fixtures of tests/test_gpu_infer_program.py."""
import os
import re
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(ROOT, "tests", "golden")
EXE = os.path.join(ROOT, "gradients.c_amd", "gpt_lm_infer")


def _generate(node_replay, *extra):
    env = {k: v for k, v in os.environ.items() if k not in ("GD_HIP_GRAPH_NODE_REPLAY", "DEBUG_CLR_GRAPH_PACKET_CAPTURE")}
    if node_replay:
        env["GD_HIP_GRAPH_NODE_REPLAY"] = "1"
    r = subprocess.run([EXE, "--checkpoint", os.path.join(GOLDEN, "gpt_tok420_seed99.gdckpt"), "--tokenizer-path",
                        os.path.join(GOLDEN, "tokenizer_small.json"), "--prompt", "the quick brown fox",
                        "--max-new-tokens", "40", "--ids", *extra], capture_output=True, timeout=120, env=env)
    assert r.returncode == 0, (r.returncode, r.stderr.decode(errors="replace"), r.stdout[-400:])
    return [int(v) for v in re.search(rb"^ids:(.*)$", r.stdout, re.M).group(1).split()]


def test_node_by_node_graph_replay_generates_the_same_tokens():
    default = _generate(False)
    nodes = _generate(True)
    assert len(default) == 40 and nodes == default
