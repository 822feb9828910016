"""pf_hip_moe_forward_static: the forward whose scratch is the library's static device array.

Called through the C-ABI twice in a row, the second time with fewer tokens, and compared with
pf_hip_moe_forward_device on a workspace (same kernels: bit for bit) and with the CPU oracle
(ids exact, outputs within 1e-3 + 1e-4 relative)."""
import ctypes as C

import numpy as np
import pytest

import picoforge_amd as pf
from picoforge_amd import abi

from helpers import assert_parity, forward_with, make_layer_inputs

pytestmark = pytest.mark.gpu


def device_forward(hip, moe, work, x, k, static):
    t, h = x.shape
    d_x = hip.to_device(x)
    d_y = hip.to_device(np.full((t, h), -99.0, dtype=np.float32))
    d_ids = hip.to_device(np.full((t, k), 0xFFFFFFFF, dtype=np.uint32))
    d_w = hip.to_device(np.full((t, k), -99.0, dtype=np.float32))
    d_err = hip.to_device(np.zeros(1, dtype=np.uint32))
    if static:
        hip.check(hip.moe_forward_static(moe, d_x, h, d_y, h, d_ids, d_w, d_err, t, None), "forward_static")
        hip.check(hip.synchronize(), "sync")
        ids = hip.from_device(d_ids, (t, k), np.uint32)
        w = hip.from_device(d_w, (t, k), np.float32)
        err = int(hip.from_device(d_err, (1,), np.uint32)[0])
    else:
        hip.check(hip.work_clear_status(work), "clear")
        hip.check(hip.moe_forward_device(moe, work, d_x, h, d_y, h, t, None), "forward_device")
        hip.check(hip.synchronize(), "sync")
        ids = hip.from_device(hip.work_ids(work), (t, k), np.uint32)
        w = hip.from_device(hip.work_route_weights(work), (t, k), np.float32)
        err = int(hip.from_device(hip.work_error_word(work), (1,), np.uint32)[0])
    y = hip.from_device(d_y, (t, h), np.float32)
    for p in (d_x, d_y, d_ids, d_w, d_err):
        hip.free(p)
    return y, ids, w, err


@pytest.mark.parametrize("h,e,k,i,s,gtype", [(2048, 512, 10, 512, 512, abi.GGUF_Q4_K), (512, 32, 6, 256, 256, abi.GGUF_IQ2_XXS),
                                             (64, 16, 4, 24, 12, abi.GGUF_F32)])
def test_static_scratch_forward_matches_the_workspace_forward(product, oracle, h, e, k, i, s, gtype):
    print(f"case static scratch h={h} e={e} type={gtype}", flush=True)
    hip = product.hip
    cfg = abi.moe_config(h, e, k, i, s)
    weights, x = make_layer_inputs(cfg, gtype, 4, seed=31 + h, std=0.02 if gtype != abi.GGUF_F32 else 0.2)
    want = forward_with(oracle, cfg, weights, x)
    with pf.MoeLayer(product, cfg, weights, 4) as layer:
        moe, work = layer.device_handles()
        for tokens in (4, 1):        # two calls in a row on the shared array, the second one smaller
            print(f"  tokens={tokens}", flush=True)
            y0, ids0, w0, err0 = device_forward(hip, moe, work, x[:tokens], k, static=False)
            y1, ids1, w1, err1 = device_forward(hip, moe, None, x[:tokens], k, static=True)
            assert err0 == 0 and err1 == 0
            np.testing.assert_array_equal(ids1, ids0)
            np.testing.assert_array_equal(w1.view(np.uint32), w0.view(np.uint32))
            np.testing.assert_array_equal(y1.view(np.uint32), y0.view(np.uint32))
            assert_parity(y1, ids1, w1, want[0][:tokens], want[1][:tokens], want[2][:tokens], label=f"static T={tokens}")


def test_static_scratch_forward_refuses_what_does_not_fit(product):
    hip = product.hip
    cfg = abi.moe_config(512, 32, 6, 256, 256)
    weights, x = make_layer_inputs(cfg, abi.GGUF_Q4_K, 5, seed=3)
    with pf.MoeLayer(product, cfg, weights, 8) as layer:
        moe, _ = layer.device_handles()
        d_x = hip.to_device(x)
        d_y = hip.to_device(np.zeros_like(x))
        d_err = hip.to_device(np.zeros(1, dtype=np.uint32))
        rc = hip.moe_forward_static(moe, d_x, 512, d_y, 512, None, None, d_err, 5, None)
        assert rc == 2 and b"at most 4 tokens" in hip.last_error()            # PF_HIP_E_UNSUPPORTED
        assert hip.moe_forward_static(moe, d_x, 512, d_y, 512, None, None, None, 1, None) == 1   # no error word
        assert hip.moe_forward_static(moe, d_x, 100, d_y, 512, None, None, d_err, 1, None) == 1  # pitch below hidden
        assert hip.moe_forward_static(moe, d_x, 512, d_y, 512, None, None, d_err, 0, None) == 0  # empty batch
        for p in (d_x, d_y, d_err):
            hip.free(p)
    # a layer whose scratch for four tokens exceeds the array
    cfg = abi.moe_config(512, 16, 15, 2048, 256)
    weights, x = make_layer_inputs(cfg, abi.GGUF_Q4_K, 4, seed=4)
    with pf.MoeLayer(product, cfg, weights, 4) as layer:
        moe, _ = layer.device_handles()
        d_x = hip.to_device(x)
        d_y = hip.to_device(np.zeros_like(x))
        d_err = hip.to_device(np.zeros(1, dtype=np.uint32))
        rc = hip.moe_forward_static(moe, d_x, 512, d_y, 512, None, None, d_err, 4, None)
        assert rc == 2 and b"static scratch holds" in hip.last_error(), hip.last_error()
        for p in (d_x, d_y, d_err):
            hip.free(p)
