"""The reference's OWN test programs, compiled from its sources (oracle/Makefile, target ref-tests)
against the unmodified reference core and linked with gradients.c_amd/libgd_backend_hip.so as the
backend.  They run with GD_HIP_HOST_VISIBLE=1 because the reference core insists on host-visible
arenas.  The binaries live in oracle/_ref/ (built where the reference tree is mounted, not tracked);
the tests are skipped when they have not been built.

  test_kv_cache_decode  literal append vectors (at / positions / packed) and the three sdpa_decode
                        position forms agreeing to 1e-6 (reference tests/test_kv_cache_decode.c)
  test_memory           arena / ring-slot / fence contract (reference tests/test_memory.c)
  test_transfer         upload / download / F32<->F16 transfer contract (reference tests/test_transfer.c)
  test_tensor           tensor descriptors, fill / rand_uniform, views, scopes (reference tests/test_tensor.c)

The reference's per-operator test programs also call the training (backward) entry points in the
same main(), which this backend answers with GD_ERR_UNSUPPORTED, so they cannot pass unmodified; their
forward cases are restated as data in tests/golden/reference_test_cases.json instead.
"""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF_DIR = os.path.join(ROOT, "oracle", "_ref")


@pytest.mark.parametrize("program", ["test_kv_cache_decode", "test_memory", "test_transfer", "test_tensor"])
def test_reference_program_passes_on_the_hip_backend(program):
    exe = os.path.join(REF_DIR, program)
    if not os.path.exists(exe):
        pytest.skip(f"{exe} not built (needs the reference tree: make -C oracle ref-tests)")
    env = dict(os.environ, GD_HIP_HOST_VISIBLE="1")
    r = subprocess.run([exe], env=env, capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert f"{program}: ok" in r.stdout
