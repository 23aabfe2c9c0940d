"""The C++ host layer (Tensor<dtype, device>, tensor_mm / tensor_softmax / tensor_causal_conv1d and
the cu_* launchers) through its own harness binary, which mirrors the reference's test
functions.  Host-only cases and the fail-stop cases run anywhere; GPU cases run on the GPU box.
"""
import os
import re
import subprocess
from pathlib import Path

import pytest

REPO = Path(__file__).resolve().parent.parent
HARNESS = REPO / "anygpu_amd" / "lib" / "anygpu_host_tests"
GOLDEN = REPO / "tests" / "golden"


def run_harness(*args, timeout=300):
    if not HARNESS.exists():
        pytest.fail(f"{HARNESS} is not built; run __graft_entry__.build() first")
    env = dict(os.environ, ANYGPU_GOLDEN_DIR=str(GOLDEN))
    return subprocess.run([str(HARNESS), *args], cwd=REPO, env=env, capture_output=True, text=True, timeout=timeout)


def verdicts(stdout):
    return dict(re.findall(r"TestCase \[(\w+)\]: (PASSED|FAILED)", stdout))


def test_host_cases_pass():
    proc = run_harness("--host")
    v = verdicts(proc.stdout)
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-2000:]
    assert len(v) >= 12 and all(r == "PASSED" for r in v.values()), v
    # config 1 of the baseline (fp32 matmul 256x512 @ 512x1024 on the CPU path) is one of them
    assert v["test_cpu_mm_f32_256x512_512x1024"] == "PASSED"


@pytest.mark.parametrize("case,message", [
    ("death_mm_shape_mismatch", "matrix multiplication requires compatible matrices"),
    ("death_softmax_not_2d", "softmax expects 2 dimensional tensors"),
    ("death_conv1d_channel_mismatch", "xt and wt need to have the same dims"),
    ("death_missing_dat_file", "Unable to open file"),
])
def test_precondition_failures_are_fail_stop(case, message):
    # the reference's error convention: print file/line and the message, exit(1)
    proc = run_harness(case)
    assert proc.returncode == 1
    assert message in proc.stdout
    assert "PASSED" not in proc.stdout and "FAILED" not in proc.stdout


def test_harness_usage_and_unknown_names():
    assert run_harness().returncode == 2
    assert run_harness("--bogus").returncode == 2
    proc = run_harness("no_such_case")
    assert proc.returncode == 1 and "no such test case" in proc.stderr
    listing = run_harness("--list").stdout.split()
    assert "test_mm_f16_640x1280_1280x320" in listing and "test_softmax_f32" in listing


@pytest.mark.gpu
def test_gpu_cases_pass():
    print("running host-layer GPU cases", flush=True)
    proc = run_harness("--gpu", timeout=600)
    v = verdicts(proc.stdout)
    assert proc.returncode == 0, proc.stdout[-3000:] + proc.stderr[-2000:]
    assert len(v) >= 17 and all(r == "PASSED" for r in v.values()), v
