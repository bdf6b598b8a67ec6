"""Tuning switches that are read once per process, hence one child process per value, each checked
against the oracle:

RK_NPU_HIP_GEMM_PLAN="rows:ksplit" forces the tile height and the K split of dense GEMMs; the reduce
kernels behind some tile heights run only under a forced plan (or for shapes the library's own plan
happens to split).  RK_NPU_HIP_GEMV_COLS forces the columns per workgroup of the decode kernels."""
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


@pytest.mark.parametrize("cols", ["32", "16", "8"])
def test_forced_gemv_width_matches_the_oracle(cols):
    """RK_NPU_HIP_GEMV_COLS forces the columns per workgroup of the decode kernels: every width with
    1, 2, 4 and 8 rows, int8 and int4 weights, rows given as int8 / fp16 / fp32 or quantized by a launch
    of their own -- among them the eight-row, 32-column instantiations that the library's own choice
    leaves to the streaming kernel on matrices wide enough for 32 columns per workgroup."""
    env = dict(os.environ, RK_NPU_HIP_GEMV_COLS=cols)
    child = subprocess.run([sys.executable, os.path.join(ROOT, "tests", "gemv_cols_child.py")], env=env,
                           capture_output=True, text=True, timeout=240)
    assert child.returncode == 0, child.stdout[-2000:] + child.stderr[-4000:]
    assert child.stdout.strip().endswith("OK " + cols), child.stdout[-2000:]
