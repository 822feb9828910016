"""Every byte range the decode kernels can read lies inside the weight buffers the library allocates.

The kernels take their offsets from picoforge_amd/csrc/pf_decode_addr.h; tests/check_decode_addresses.cpp
compiles the same header for the host and walks every (tensor, expert, row, segment, pass, warm-up line) of
a launch.  Runs without a GPU."""
import subprocess
from pathlib import Path

import pytest

from picoforge_amd import abi

ROOT = Path(__file__).resolve().parents[1]
F32, Q4K, IQ2, Q2K, Q8, MX = abi.GGUF_F32, abi.GGUF_Q4_K, abi.GGUF_IQ2_XXS, abi.GGUF_Q2_K, abi.GGUF_Q8_0, abi.GGUF_MXFP4


def types(gate, down, shared):
    return [F32, gate, gate, down, shared, shared, shared, F32]


LAYERS = [
    # hidden, experts, top_k, inter, shared, down_physical, tensor types
    ("q4k benchmark shape", (2048, 512, 10, 512, 512, 512), types(Q4K, Q4K, Q4K)),
    ("iq2_xxs benchmark shape", (2048, 512, 10, 512, 512, 512), types(IQ2, IQ2, IQ2)),
    ("q2 profile, benchmark shape", (2048, 512, 10, 512, 512, 512), types(IQ2, Q2K, Q8)),
    ("q4 profile, benchmark shape", (2048, 512, 10, 512, 512, 512), types(Q4K, MX, Q8)),
    ("q2 profile, checkpoint widths", (2560, 512, 10, 640, 640, 768), types(IQ2, Q2K, Q8)),
    ("q4 profile, checkpoint widths", (2560, 512, 10, 640, 640, 640), types(Q4K, MX, Q8)),
    ("q4k, widest shapes", (2560, 64, 10, 768, 768, 768), types(Q4K, Q4K, Q4K)),
    ("small layer", (512, 32, 6, 256, 256, 256), types(IQ2, IQ2, IQ2)),
    ("wide shared expert", (1024, 96, 5, 256, 1024, 256), types(IQ2, IQ2, IQ2)),
]


@pytest.fixture(scope="module")
def walker(tmp_path_factory):
    exe = tmp_path_factory.mktemp("addr") / "check_decode_addresses"
    subprocess.run(["g++", "-std=c++17", "-O2", "-Wall", "-o", str(exe), str(ROOT / "tests" / "check_decode_addresses.cpp")], check=True)
    return exe


@pytest.mark.parametrize("label,dims,tensor_types", LAYERS, ids=[l[0] for l in LAYERS])
def test_every_read_of_the_decode_kernels_stays_inside_its_buffer(walker, label, dims, tensor_types):
    run = subprocess.run([str(walker)] + [str(v) for v in dims] + [str(t) for t in tensor_types], capture_output=True, text=True)
    print(run.stdout, run.stderr)
    assert run.returncode == 0, run.stderr
    assert int(run.stdout.split()[0]) > 50000
