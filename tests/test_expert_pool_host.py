"""The expert pool's host side on the CPU, under the sanitizers.

tests/check_expert_pool.c links picoforge_amd/csrc/qwen4_expert_pool.c against a stand-in for the HIP shim (plain
memory): the bookkeeping, the persistent reader threads and their hand-over per acquire run without a GPU, once
with AddressSanitizer and UndefinedBehaviorSanitizer and once with ThreadSanitizer."""
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]


@pytest.mark.parametrize("sanitizer", ["address,undefined", "thread"])
def test_pool_reads_through_persistent_readers(tmp_path, sanitizer):
    exe = tmp_path / "check_expert_pool"
    subprocess.run(["gcc", "-std=c11", "-g", "-O1", f"-fsanitize={sanitizer}", "-fno-sanitize-recover=all", "-pthread", "-o", str(exe),
                    str(ROOT / "tests" / "check_expert_pool.c"), str(ROOT / "picoforge_amd" / "csrc" / "qwen4_expert_pool.c")], check=True)
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    print(run.stdout, run.stderr)
    assert run.returncode == 0, run.stderr
    assert "misses" in run.stdout
