"""RK_NPU_HIP_GEMM_PLAN="rows:ksplit" (a tuning aid) forces the tile height and the K split of
dense GEMMs.  The library's own plan splits K over workgroups only where 32-row tiles are too few,
so the reduce kernels behind 64- and 128-row tiles run only under a forced plan (or for int4
weights with K beyond 2^17 under many rows): each forced plan must give the oracle's results too.
The variable is read once per process, hence one child process per plan."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("plan", ["128:2", "64:3", "32:4", "128:1"])
def test_forced_dense_plan_matches_the_oracle(plan):
    env = dict(os.environ, RK_NPU_HIP_GEMM_PLAN=plan)
    child = subprocess.run([sys.executable, os.path.join(ROOT, "tests", "plan_override_child.py")], env=env,
                           capture_output=True, text=True, timeout=240)
    assert child.returncode == 0, child.stdout[-2000:] + child.stderr[-4000:]
    assert child.stdout.strip().endswith("OK " + plan), child.stdout[-2000:]
