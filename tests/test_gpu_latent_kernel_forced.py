"""The planner sends small latent problems, and those with few heads, to the grouped-head kernel; the latent kernel
then only sees large shapes.  Its one-, two- and four-wave forms, page forms and 8-bit forms must hold at every
size all the same, so the latent cases of the other test files run once more in a process whose planner keeps the
latent form on the latent kernel (the tunables are read once per process)."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

FILES = ["tests/test_gpu_parity.py", "tests/test_gpu_fp8kv.py", "tests/test_gpu_int8kv.py", "tests/test_gpu_paged.py",
         "tests/test_gpu_graph.py", "tests/test_gpu_random.py"]


def test_latent_cases_on_the_latent_kernel():
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, DA_MLA_GROUP_HEADS="0", DA_MLA_GROUP_SMALL="0")
    cmd = [sys.executable, "-m", "pytest", *FILES, "-q", "-x", "-m", "gpu", "-k", "mla or latent or random",
           "-p", "no:cacheprovider"]
    r = subprocess.run(cmd, env=env, cwd=root, capture_output=True, text=True, timeout=900)
    tail = r.stdout[-3000:] + r.stderr[-2000:]
    assert r.returncode == 0 and " passed" in r.stdout and "failed" not in r.stdout, tail
