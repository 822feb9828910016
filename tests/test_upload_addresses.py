"""Every byte the upload kernels read lies inside their source buffer and every byte they write inside the
destination allocation.

The kernels that lay a layer out in device memory (scale/payload splits, tile orders) take their addresses from
picoforge_amd/csrc/pf_upload_addr.h; tests/check_upload_addresses.cpp compiles the same header for the host and
walks every thread of every launch, with the allocation sizes pf_hip_moe_create uses.  Runs without a GPU."""
import subprocess
from pathlib import Path

import pytest

from test_decode_addresses import LAYERS

ROOT = Path(__file__).resolve().parents[1]


@pytest.fixture(scope="module")
def walker(tmp_path_factory):
    exe = tmp_path_factory.mktemp("upload") / "check_upload_addresses"
    subprocess.run(["g++", "-std=c++17", "-O2", "-Wall", "-o", str(exe), str(ROOT / "tests" / "check_upload_addresses.cpp")], check=True)
    return exe


@pytest.mark.parametrize("label,dims,tensor_types", LAYERS, ids=[l[0] for l in LAYERS])
def test_every_access_of_the_upload_kernels_stays_inside_its_buffer(walker, label, dims, tensor_types):
    run = subprocess.run([str(walker)] + [str(v) for v in dims] + [str(t) for t in tensor_types], capture_output=True, text=True)
    print(run.stdout, run.stderr)
    assert run.returncode == 0, run.stderr
    assert int(run.stdout.split()[0]) > 100000
