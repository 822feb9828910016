"""The reference's own MoE test harness links against the shipped library in place of src/qwen4_moe.c.

tests/test_qwen4_moe.c of the reference reaches the block through QW4_F_FORWARD, which defaults to
qwen4_moe_forward (tests/test_qwen4_moe.c:13-15), and is built from the harness, src/qwen4_moe.c and the
reference's non-MoE units (tools/qwen4.mk:59-61).  Here the harness and those other units are compiled where
they lie and libpicoforge_moe.so stands in for src/qwen4_moe.c: every symbol must resolve, and the MoE entry
points must come from the library.  Runs where the reference tree is mounted; no GPU needed (nothing is run)."""
import subprocess
from pathlib import Path

import pytest

from picoforge_amd import binding

REF = Path("/root/reference")
OTHER_UNITS = ["qwen4_base.c", "qwen4_conv.c", "qwen4_gdn.c", "qwen4_config.c", "qwen4_weights.c", "qwen4_packed.c",
               "gguf_plan.c", "gguf.c", "gguf_reader.c", "util.c"]          # QW4_RECURRENT of tools/qwen4.mk:15-17
MOE_SYMBOLS = ["qwen4_moe_create", "qwen4_moe_destroy", "qwen4_moe_work_size", "qwen4_moe_work_create", "qwen4_moe_work_reset",
               "qwen4_moe_work_destroy", "qwen4_moe_route", "qwen4_moe_forward", "qw4_moe_group_pairs", "qw4_moe_observe"]


@pytest.mark.skipif(not (REF / "tests" / "test_qwen4_moe.c").exists(), reason="reference tree not mounted")
def test_reference_moe_harness_links_against_the_library(tmp_path):
    exe = tmp_path / "test_moe"
    lib_dir = binding.PRODUCT_LIB.parent
    cmd = ["gcc", "-std=c11", "-D_DEFAULT_SOURCE", "-O1", "-ffp-contract=off", "-fno-fast-math", f"-I{REF / 'src'}",
           str(REF / "tests" / "test_qwen4_moe.c")] + [str(REF / "src" / u) for u in OTHER_UNITS] + \
          [f"-L{lib_dir}", "-lpicoforge_moe", "-lm", f"-Wl,-rpath,{lib_dir}", "-o", str(exe)]
    run = subprocess.run(cmd, capture_output=True, text=True)
    assert run.returncode == 0, run.stderr[-2000:]
    undefined = subprocess.run(["nm", "-u", str(exe)], capture_output=True, text=True, check=True).stdout
    for name in MOE_SYMBOLS:
        assert f"U {name}" in undefined, f"{name} is not taken from the library"
    needed = subprocess.run(["readelf", "-d", str(exe)], capture_output=True, text=True, check=True).stdout
    assert "libpicoforge_moe.so" in needed
