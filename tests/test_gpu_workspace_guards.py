"""No kernel writes outside the workspace buffer it was given.

A workspace created with PF_WORK_GUARD=1 has 4096 bytes of a fixed pattern behind each of its buffers (logits,
routes, activations, digit images, union tables, the prefill path's fp16 forms and grouping tables, ...).  The
layers of the checkpoint profiles and of the single-format configurations, at the benchmark widths and at the
checkpoints' widths, run batches of 1, 4 and 16 tokens (decode kernels), 48 tokens (matrix cores) and the
general kernels; afterwards every guard must still hold the pattern, and the outputs must match the CPU path."""
import ctypes as C

import numpy as np
import pytest

import picoforge_amd as pf
from picoforge_amd import abi

from helpers import assert_parity, forward_with, make_layer_inputs

pytestmark = pytest.mark.gpu

SHAPES = [
    ("q4k, benchmark widths", abi.GGUF_Q4_K, (2048, 64, 10, 512, 512, 512)),
    ("iq2_xxs, benchmark widths", abi.GGUF_IQ2_XXS, (2048, 64, 10, 512, 512, 512)),
    ("q2 profile, benchmark widths", "q2", (2048, 64, 10, 512, 512, 512)),
    ("q4 profile, benchmark widths", "q4", (2048, 64, 10, 512, 512, 512)),
    ("q2 profile, checkpoint widths", "q2", (2560, 64, 10, 640, 640, 768)),
    ("q4 profile, checkpoint widths", "q4", (2560, 64, 10, 640, 640, 640)),
]


def guards(product, layer):
    damaged, first = C.c_int(), C.c_int()
    rc = product.hip.work_check_guards(product.device_work(layer.work), C.byref(damaged), C.byref(first))
    assert rc == 0
    return damaged.value, first.value


@pytest.mark.parametrize("label,expert_type,dims", SHAPES, ids=[s[0] for s in SHAPES])
def test_no_kernel_writes_beyond_its_workspace_buffer(product, oracle, monkeypatch, label, expert_type, dims):
    h, e, k, i, s, phys = dims
    cfg = abi.moe_config(h, e, k, i, s, down_physical=phys)
    weights, x = make_layer_inputs(cfg, expert_type, 48, seed=97)
    want = forward_with(oracle, cfg, weights, x[:16])
    monkeypatch.setenv("PF_WORK_GUARD", "1")
    for fused in ("0", "1"):
        monkeypatch.setenv("PF_MOE_DECODE_FUSED", fused)
        with pf.MoeLayer(product, cfg, weights, 48) as layer:
            for tokens in (1, 4, 16):
                print(f"guards: {label}, {tokens} tokens, one-launch expert stage {fused}", flush=True)
                _, y, ids, w = layer.forward(x[:tokens])
                assert_parity(y, ids, w, want[0][:tokens], want[1][:tokens], want[2][:tokens], label=f"{label} T={tokens}")
                assert guards(product, layer) == (0, -1), f"{label}: a guard was overwritten by the {tokens}-token forward"
            if fused == "0":
                print(f"guards: {label}, 48 tokens", flush=True)
                layer.forward(x)
                assert guards(product, layer) == (0, -1), f"{label}: a guard was overwritten by the 48-token forward"
                layer.force_general()
                layer.forward(x[:5])
                assert guards(product, layer) == (0, -1), f"{label}: a guard was overwritten by the general kernels"


def test_the_guards_notice_a_write(product, monkeypatch):
    """The check itself: bytes written behind a buffer are reported (a copy from the host, no kernel involved)."""
    monkeypatch.setenv("PF_WORK_GUARD", "1")
    cfg = abi.moe_config(512, 32, 6, 256, 256)
    weights, x = make_layer_inputs(cfg, abi.GGUF_Q4_K, 2, seed=5)
    with pf.MoeLayer(product, cfg, weights, 2) as layer:
        assert guards(product, layer) == (0, -1)
        hip = product.hip
        logits = hip.work_logits(product.device_work(layer.work))      # the workspace's first buffer: 2 x 32 floats, 256 bytes
        junk = np.zeros(4, dtype=np.uint8)
        hip.check(hip.memcpy_h2d(C.c_void_p(logits + 256 + 100), junk.ctypes.data, 4), "poke")
        assert guards(product, layer) == (1, 0)
    monkeypatch.delenv("PF_WORK_GUARD")
    with pf.MoeLayer(product, cfg, weights, 2) as layer:
        assert guards(product, layer) == (0, -1)                          # no guards: nothing to report
