"""The C-ABI library loads, exports every declared symbol, and its structures have the layouts
the ctypes mirror (and the reference's headers) assume.  No compute calls: runs without a GPU."""
import ctypes as C
import re
import subprocess
import sys
from pathlib import Path

import pytest

import picoforge_amd as pf
from picoforge_amd import abi, binding

ROOT = Path(__file__).resolve().parents[1]
HEADERS = ["qwen4_packed.h", "qwen4_moe.h", "qwen4_hc.h", "pf_gguf.h", "pf_moe_hip.h"]


def declared_functions(header):
    text = (ROOT / "include" / header).read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"^\s*(?:const\s+)?[A-Za-z_][\w\s\*]*?\b(\w+)\s*\([^;{]*\)\s*;", text, flags=re.M)
    return [n for n in names if n != "void"]   # the observer typedef's return type is not a function


def test_every_declared_symbol_is_exported():
    lib = C.CDLL(str(binding.PRODUCT_LIB))
    missing = []
    total = 0
    for header in HEADERS:
        names = declared_functions(header)
        assert names, header
        total += len(names)
        missing += [f"{header}:{n}" for n in names if not hasattr(lib, n)]
    assert not missing, missing
    assert total >= 57


def test_product_never_links_the_oracle():
    out = subprocess.run(["nm", "-D", str(binding.PRODUCT_LIB)], capture_output=True, text=True, check=True).stdout
    assert "orc_" not in out
    needed = subprocess.run(["readelf", "-d", str(binding.PRODUCT_LIB)], capture_output=True, text=True).stdout
    assert "liborc" not in needed and "libqwen4_ref" not in needed
    for source in (ROOT / "picoforge_amd").rglob("*"):
        if source.suffix in (".c", ".h", ".hip", ".py"):
            assert "oracle/" not in source.read_text(), source


def test_struct_layouts_match_a_c_compiler(tmp_path):
    probe = tmp_path / "probe.c"
    probe.write_text(r'''
#include <stdio.h>
#include <stddef.h>
#include "qwen4_moe.h"
#include "qwen4_hc.h"
#include "pf_moe_hip.h"
int main(void) {
    printf("%zu %zu %zu %zu %zu %zu %zu %zu %zu %zu %zu %zu\n", sizeof(Qwen4Error), sizeof(Qwen4F32), sizeof(Qwen4U32Mut),
           sizeof(Qwen4MoeConfig), sizeof(GgufTensor), sizeof(QW4PackedLayout), sizeof(QW4PackedCpuView),
           sizeof(Qwen4MoeWeights), sizeof(Qwen4MoeRoutes), sizeof(QW4MoeGrouping), sizeof(PfHipMoeDesc),
           sizeof(Qwen4HcShape));
    printf("%zu %zu %zu %zu\n", offsetof(Qwen4Error, row), offsetof(Qwen4Error, subject),
           offsetof(Qwen4MoeConfig, trunk_type), offsetof(QW4PackedLayout, k_storage));
    return 0;
}''')
    exe = tmp_path / "probe"
    subprocess.run(["gcc", "-std=c11", "-I", str(ROOT / "include"), str(probe), "-o", str(exe)], check=True)
    sizes, offsets = [list(map(int, line.split())) for line in
                      subprocess.run([str(exe)], capture_output=True, text=True, check=True).stdout.splitlines()]
    mirror = [abi.Qwen4Error, abi.Qwen4F32, abi.Qwen4U32Mut, abi.Qwen4MoeConfig, abi.GgufTensor,
              abi.QW4PackedLayout, abi.QW4PackedCpuView, abi.Qwen4MoeWeights, abi.Qwen4MoeRoutes,
              abi.QW4MoeGrouping, binding.PfHipMoeDesc, abi.Qwen4HcShape]
    assert sizes == [C.sizeof(t) for t in mirror]
    assert offsets == [abi.Qwen4Error.row.offset, abi.Qwen4Error.subject.offset,
                       abi.Qwen4MoeConfig.trunk_type.offset, abi.QW4PackedLayout.k_storage.offset]


@pytest.mark.skipif(not (Path("/root/reference/src/qwen4_types.h")).exists(), reason="reference tree not mounted")
def test_struct_layouts_match_the_reference_headers(tmp_path):
    """Same probe compiled against the reference's own headers: identical sizes and enum values."""
    body = r'''
int main(void) {
    printf("%zu %zu %zu %zu %zu %zu %zu %zu %zu %d %d %d\n", sizeof(Qwen4Error), sizeof(Qwen4F32), sizeof(Qwen4U32Mut),
           sizeof(Qwen4MoeConfig), sizeof(GgufTensor), sizeof(QW4PackedLayout), sizeof(QW4PackedCpuView),
           sizeof(Qwen4MoeWeights), sizeof(Qwen4MoeRoutes), (int)QW4_NONFINITE, (int)QW4_GPU_ERROR, (int)QW4_CAPACITY);
    return 0;
}'''
    outputs = []
    for name, include, header in (("mine", ROOT / "include", "qwen4_moe.h"),
                                  ("ref", Path("/root/reference/src"), "qwen4_moe.h")):
        src = tmp_path / f"{name}.c"
        src.write_text(f'#include <stdio.h>\n#include "{header}"\n' + body)
        exe = tmp_path / name
        subprocess.run(["gcc", "-std=c11", "-I", str(include), str(src), "-o", str(exe)], check=True)
        outputs.append(subprocess.run([str(exe)], capture_output=True, text=True, check=True).stdout)
    assert outputs[0] == outputs[1]
    shapes = []
    for name, include, header in (("mine_hc", ROOT / "include", "qwen4_hc.h"),
                                  ("ref_hc", Path("/root/reference/src"), "qwen4_ops.h")):
        src = tmp_path / f"{name}.c"
        src.write_text(f'#include <stdio.h>\n#include <stddef.h>\n#include "{header}"\n' +
                       'int main(void) { printf("%zu %zu %zu\\n", sizeof(Qwen4HcShape), offsetof(Qwen4HcShape, low_rank), '
                       'offsetof(Qwen4HcShape, rms_eps)); return 0; }')
        exe = tmp_path / name
        subprocess.run(["gcc", "-std=c11", "-I", str(include), str(src), "-o", str(exe)], check=True)
        shapes.append(subprocess.run([str(exe)], capture_output=True, text=True, check=True).stdout)
    assert shapes[0] == shapes[1]


def test_product_fails_loudly_without_a_device():
    """Without a GPU the compute entry points return an error status; nothing is computed on the CPU."""
    api = pf.load_product()
    if api.hip.device_count() > 0:
        pytest.skip("a device is present")
    import numpy as np
    cfg = abi.moe_config(8, 4, 2, 5, 3)
    weights = pf.LayerWeights.synthetic(cfg, abi.GGUF_F32, seed=1)
    with pytest.raises(pf.MoeError) as caught:
        pf.MoeLayer(api, cfg, weights, 2)
    assert caught.value.status == abi.QW4_GPU_ERROR
    from helpers import call_route
    st, p, ids, w, _ = call_route(api, cfg, np.zeros((1, 4), dtype=np.float32))
    assert st in (abi.QW4_GPU_ERROR, abi.QW4_UNSUPPORTED) and (p == -99).all()


def test_shim_entry_points_refuse_bad_arguments_before_touching_a_device():
    """Null handles, zero dimensions and pitches narrower than a row are refused by the C-ABI shim itself
    (PF_HIP_E_ARGUMENT = 1): no device is needed to find that out."""
    hip = pf.load_product().hip
    word = C.c_uint32()
    ms = C.c_float()
    buf = (C.c_float * 64)()
    p = C.cast(buf, C.c_void_p)
    assert hip.hc_read_device(None, 8, 4, p, 8, 4, p, 4, 1, 2, 4, p, None) == 1
    assert hip.hc_read_device(p, 8, 4, p, 8, 4, p, 4, 1, 0, 4, p, None) == 1          # no streams
    assert hip.hc_read_device(p, 8, 2, p, 8, 4, p, 4, 1, 2, 4, p, None) == 1          # stream pitch below hidden
    assert hip.hc_read_device(p, 8, 4, p, 8, 4, p, 4, 1, 2, 4, None, None) == 1       # no error word
    assert hip.hc_read_device(p, 8, 4, p, 8, 4, p, 4, 0, 2, 4, p, None) == 0          # no tokens: nothing to do
    assert hip.hc_add_device(p, 8, 4, None, 4, p, 2, 1, 2, 4, p, None) == 1
    assert hip.hc_add_device(p, 8, 4, p, 4, p, 1, 1, 2, 4, p, None) == 1              # inject pitch below streams
    assert hip.hc_add_device(p, 8, 4, p, 4, p, 2, 0, 2, 4, p, None) == 0
    assert hip.moe_forward_hc_device(None, None, p, 8, 4, p, 8, 4, p, 8, 4, p, 2, 1, None) == 1
    assert hip.moe_forward_device(None, None, p, 4, p, 4, 1, None) == 1
    assert hip.moe_kernel_family(None, None, 1) == 0
    assert hip.hc_read_host(None, 32, 16, p, 32, 16, p, 16, 1, 2, 4, C.byref(word)) == 1
    assert hip.hc_read_host(p, 32, 16, p, 32, 16, p, 16, 0, 2, 4, C.byref(word)) == 0
