"""The benchmark executable: flag handling (CPU) and, on the GPU, the reference's log lines and its own check."""
import os
import re
import subprocess

import pytest

from decoding_attention_amd import build as da_build

EXE = da_build.CLI_PATH

pytestmark = pytest.mark.skipif(not os.path.exists(EXE), reason="benchmark executable not built")


def _run(*args, timeout=120):
    return subprocess.run([EXE, *args], capture_output=True, text=True, timeout=timeout)


def test_help_lists_the_reference_flags():
    res = _run("--help")
    assert res.returncode == 0
    for name in ("b", "sq", "sk", "hq", "hk", "d", "dv", "is_causal", "is_alibi", "is_bf16", "warmup_iterations",
                 "profiling_iterations", "sleep_duration", "enable_check", "cpu_procs", "gpu_rank"):
        assert re.search(rf"^\s+-{name} \(", res.stdout, re.M), name


@pytest.mark.parametrize("args,message", [
    (["-bogus=1"], "unknown command line flag 'bogus'"),
    (["-b=x"], "illegal value 'x' specified for uint32 flag 'b'"),
    (["-is_alibi=maybe"], "illegal value 'maybe' specified for bool flag 'is_alibi'"),
    (["-sk"], "missing its argument"),
    (["-sq=2"], "-sq must be 1"),
    (["-is_causal"], "-sq must be 1"),
])
def test_bad_flags_are_rejected_before_any_gpu_call(args, message):
    res = _run(*args)
    assert res.returncode == 1
    assert message in res.stderr


PROFILE_LINE = re.compile(
    r"^\[DA \d{4}-\d\d-\d\d \d\d:\d\d:\d\d \d+:\d+ benchmark_decoding_attn\.cpp:\d+ run_case\] Decoding-Attention exit, "
    r"profiling time: ([\d.]+) ms \(100\.00%\), throughput: ([\d.]+) TFLOPS \(100\.00%\), bandwidth: ([\d.]+) GB/s "
    r"\(100\.00%\)$", re.M)


def _parse_like_the_reference_tool(log):
    """Field positions the reference's tools/performance/cpp/performance.py:77-90 reads from an 'exit' line."""
    for line in log.splitlines():
        if "exit" in line and "Naive" not in line:
            items = line.split(" ")
            return items[6], float(items[14]), float(items[18])
    raise AssertionError("no profile line")


@pytest.mark.gpu
@pytest.mark.parametrize("flags,tol", [
    (["-b=2", "-sk=256"], 2e-3),                                               # the reference's default smoke shape
    (["-b=2", "-sk=256", "-is_bf16=true"], 1e-2),
    (["-b=2", "-sk=256", "-hq=64", "-hk=8", "-is_alibi"], 2e-3),               # GQA + ALiBi, bool flag without value
    (["--b", "2", "--sk", "256", "-hq=128", "-hk=1", "-d=576", "-dv=512"], 2e-3),  # MLA, spaced values
])
def test_check_mode_and_log_format(flags, tol):
    res = _run(*flags, "-enable_check=true", "-sleep_duration=0", "-seed=7", "-profiling_iterations=3")
    assert res.returncode == 0, res.stderr
    m = re.search(r"Max diff: ([\d.]+), avg diff: ([\d.]+)", res.stderr)
    assert m, res.stderr
    assert float(m.group(1)) <= tol and float(m.group(2)) <= tol / 10
    assert PROFILE_LINE.search(res.stderr), res.stderr
    name, tflops, gbps = _parse_like_the_reference_tool(res.stderr)
    assert name == "Decoding-Attention" and tflops > 0 and gbps > 0
    assert res.stderr.rstrip().endswith("Done")
