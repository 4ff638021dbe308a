"""bench.py refuses, before it touches the GPU, a profiled run whose flags would queue more dispatch packets than a
hardware queue's ring holds (rocprofv3's queue interception has crashed such runs inside hipGraphLaunch).  Pure
arithmetic on the flags: runs on the CPU."""
import importlib.util
import os

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


PROFILED = {"ROCP_TOOL_LIBRARIES": "/opt/rocm/lib/rocprofiler-sdk/librocprofiler-sdk-tool.so"}


def _args(bench, *flags):
    return bench.build_parser().parse_args(list(flags))


def test_profiler_detection(bench):
    assert not bench.profiler_attached({"PATH": "/usr/bin", "LD_PRELOAD": "/usr/local/lib/other.so"})
    assert bench.profiler_attached(PROFILED)
    assert bench.profiler_attached({"LD_PRELOAD": "/opt/rocm/lib/librocprofiler-sdk-tool.so.1"})
    assert bench.profiler_attached({"ROCPROF_OUTPUT_PATH": "out"})


def test_step_arithmetic(bench):
    total, parts = bench.planned_dispatches(_args(bench, "--workload", "4"))
    assert parts["configs[4]"] >= 128 * (5 * 24 + 2) and total == sum(parts.values())
    few, _ = bench.planned_dispatches(_args(bench, "--workload", "4", "--decode-steps", "80"))
    assert total - few == 48 * (5 * 24 + 2)
    head, parts = bench.planned_dispatches(_args(bench, "--headline-only", "--batches", "1"))
    assert parts["configs[2]"] >= (20 + 200) * 17 and "configs[3]" not in parts
    full, parts = bench.planned_dispatches(_args(bench))
    assert {"configs[0]", "configs[1]", "configs[2]", "configs[3]", "configs[4]", "roofline"} <= set(parts) and full > head


@pytest.mark.parametrize("flags,refused", [
    ((), True),                                                            # the driver's line: all five configs
    (("--headline-only", "--no-cpu-baseline"), True),                      # five batches of 200 steps x 17 launches
    (("--headline-only", "--no-cpu-baseline", "--batches", "1"), False),
    (("--workload", "4"), True),                                           # 128 steps x 122 launches
    (("--workload", "4", "--decode-steps", "80"), False),
    (("--workload", "3", "--steps", "40", "--warmup", "5", "--batches", "1"), False),
    (("--workload", "3", "--steps", "200"), True),
    (("--workload", "4", "--prefill-only"), False),
    (("--kernel-only",), False),
    (("--sampled",), False),
    (("--minimax-kernels",), False),
    (("--probe", "tile_gemm", "--steps", "2"), False),
])
def test_flags_that_would_wrap_the_ring_are_refused_only_under_a_profiler(bench, flags, refused):
    a = _args(bench, *flags)
    bench.refuse_if_profiled_run_would_wrap_the_queue(a, env={"PATH": "/usr/bin"})      # no profiler: never refused
    if refused:
        with pytest.raises(SystemExit) as e:
            bench.refuse_if_profiled_run_would_wrap_the_queue(a, env=PROFILED)
        assert "dispatch packets" in str(e.value.code) and e.value.code != 0
    else:
        bench.refuse_if_profiled_run_would_wrap_the_queue(a, env=PROFILED)
