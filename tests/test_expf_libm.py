"""The exponential the HIP kernels evaluate where the reference calls expf (softmax of the routing
in serial order, sigmoid of the hyper-connection read): picoforge_amd/csrc/pf_expf_libm.h compiled
for the host and compared with the host C library's expf bit for bit (tests/check_expf.c).  The GPU
tests then compare the kernels with the CPU oracle, which calls that library."""
import re
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]


@pytest.fixture(scope="module")
def checker(tmp_path_factory):
    exe = tmp_path_factory.mktemp("expf") / "check_expf"
    subprocess.run(["gcc", "-std=c11", "-O2", "-ffp-contract=off", "-Wall", "-Wextra", "-o", str(exe),
                    str(ROOT / "tests" / "check_expf.c"), "-lm"], check=True)
    return exe


def run(exe, *args):
    out = subprocess.run([str(exe), *args], capture_output=True, text=True, check=True).stdout
    checked, bad = map(int, re.search(r"checked (\d+) mismatches (\d+)", out).groups())
    return checked, bad, out


def test_sampled_arguments_and_the_threshold_neighbourhoods(checker):
    checked, bad, out = run(checker)
    assert checked > 20_000_000 and bad == 0, out


def test_all_arguments(checker):
    """All 2^32 bit patterns (NaNs skipped).  A C library built without fused multiply-add rounds two
    of them the other way by one ulp; the build this image runs matches on all."""
    checked, bad, out = run(checker, "--all")
    assert checked == 2 ** 32 - 2 * (2 ** 23 - 1) and bad <= 2, out
