"""GPU parity of the optional one-token decode path whose expert stage is ONE launch (PF_MOE_DECODE_FUSED=1 at workspace
creation: every workgroup computes a tile's activations, publishes them as a tagged line in memory, waits for the
lines of the other workgroups and multiplies eight output rows) against the CPU path and against the same layer
run as three dependent kernels, the default."""
import numpy as np
import pytest

import picoforge_amd as pf
from picoforge_amd import abi, workloads

from helpers import ATOL, RTOL, assert_parity, forward_with, make_layer_inputs

pytestmark = pytest.mark.gpu


def launches(product, layer, tokens=1):
    return product.hip.moe_decode_launches(*layer.device_handles(), tokens)


@pytest.mark.parametrize("gtype", [abi.GGUF_Q4_K, abi.GGUF_IQ2_XXS])
def test_fused_expert_stage_matches_oracle_and_three_kernels(product, oracle, gtype, monkeypatch):
    """The measured shape, one token a call: the two-launch forward against the CPU path (ids bit-exact, outputs
    within 1e-3 + 1e-4 |ref|) and against the three-kernel forward of the same layer, whose sums differ only in
    their order; every call repeated, a second time after other calls, bit for bit (a forward's lines carry its own
    tag: nothing of the forward before is mistaken for them)."""
    cfg = workloads.measured_config()
    weights, x = make_layer_inputs(cfg, gtype, 12, seed=31)
    want = forward_with(oracle, cfg, weights, x[:6])
    monkeypatch.setenv("PF_MOE_DECODE_FUSED", "1")
    with pf.MoeLayer(product, cfg, weights, 1) as fused:
        assert launches(product, fused) == 2, "the one-launch expert stage does not take this layer"
        monkeypatch.delenv("PF_MOE_DECODE_FUSED")
        with pf.MoeLayer(product, cfg, weights, 1) as plain:
            assert launches(product, plain) == 3
            first = []
            for t in range(len(x)):
                print(f"fused decode type={gtype} token {t}", flush=True)
                _, y, ids, w = fused.forward(x[t:t + 1])
                _, y3, ids3, w3 = plain.forward(x[t:t + 1])
                np.testing.assert_array_equal(ids, ids3)
                np.testing.assert_array_equal(w, w3)
                err = np.abs(y.astype(np.float64) - y3)
                assert (err <= 2e-5 + 2e-5 * np.abs(y3)).all(), f"token {t}: two against three launches differ by {err.max():.3e}"
                if t < 6:
                    assert_parity(y, ids, w, want[0][t:t + 1], want[1][t:t + 1], want[2][t:t + 1], label=f"fused token {t}")
                first.append((y, ids, w))
            for rounds in range(3):
                for t in range(len(x)):
                    _, y, ids, w = fused.forward(x[t:t + 1])
                    np.testing.assert_array_equal(y, first[t][0], err_msg=f"token {t}, repeat {rounds}: not bit for bit")
                    np.testing.assert_array_equal(ids, first[t][1])


@pytest.mark.parametrize("h,e,k,i,s", [(512, 32, 6, 256, 256), (1024, 64, 8, 512, 256), (2048, 128, 4, 256, 512),
                                       (1536, 96, 15, 256, 256)])
@pytest.mark.parametrize("gtype", [abi.GGUF_Q4_K, abi.GGUF_IQ2_XXS])
def test_fused_expert_stage_on_other_shapes(product, oracle, h, e, k, i, s, gtype, monkeypatch):
    """Hidden widths below 2048 (more workgroups with a tile than with output rows, and the other way round), shared
    experts wider and narrower than the routed ones."""
    monkeypatch.setenv("PF_MOE_DECODE_FUSED", "1")
    cfg = abi.moe_config(h, e, k, i, s)
    weights, x = make_layer_inputs(cfg, gtype, 5, seed=h + e)
    want = forward_with(oracle, cfg, weights, x)
    with pf.MoeLayer(product, cfg, weights, 1) as layer:
        assert launches(product, layer) == 2
        for t in range(len(x)):
            print(f"fused decode {h}/{e}/{k}/{i}/{s} type={gtype} token {t}", flush=True)
            _, y, ids, w = layer.forward(x[t:t + 1])
            assert_parity(y, ids, w, want[0][t:t + 1], want[1][t:t + 1], want[2][t:t + 1], label=f"token {t}")


def test_fused_expert_stage_under_graph_replay(product, oracle, monkeypatch):
    """A captured sequence of forwards, each on another input, replayed several times with eager forwards between the
    replays: the last forward's output and routes of every replay against the CPU path."""
    from bench import Tools
    tools, hip = Tools(), product.hip
    cfg = workloads.measured_config()
    weights, x = make_layer_inputs(cfg, abi.GGUF_Q4_K, 8, seed=77)
    want = forward_with(oracle, cfg, weights, x[-1:])
    monkeypatch.setenv("PF_MOE_DECODE_FUSED", "1")
    with pf.MoeLayer(product, cfg, weights, 1) as layer:
        moe, work = layer.device_handles()
        assert hip.moe_decode_launches(moe, work, 1) == 2
        d_x = hip.to_device(x.reshape(len(x), 1, cfg.hidden_size))
        d_y = hip.to_device(np.full((1, cfg.hidden_size), -99.0, dtype=np.float32))
        plan = tools.plan_moe([moe], [work], d_x, len(x), d_y, 1, 1, len(x), cfg.hidden_size)
        for replay in range(4):
            print(f"fused decode, graph replay {replay}", flush=True)
            tools.run(plan, 1)
            y = hip.from_device(d_y, (1, cfg.hidden_size), np.float32)
            ids = hip.from_device(hip.work_ids(work), (1, cfg.top_k), np.uint32)
            w = hip.from_device(hip.work_route_weights(work), (1, cfg.top_k), np.float32)
            assert int(hip.from_device(hip.work_error_word(work), (1,), np.uint32)[0]) == 0
            assert_parity(y, ids, w, *want, label=f"replay {replay}")
            layer.forward(x[replay:replay + 1])            # eager work between the replays
        tools.destroy(plan)
        hip.free(d_x)
        hip.free(d_y)


def test_three_kernels_by_default(product, oracle, monkeypatch):
    monkeypatch.delenv("PF_MOE_DECODE_FUSED", raising=False)
    cfg = abi.moe_config(512, 32, 6, 256, 256)
    weights, x = make_layer_inputs(cfg, abi.GGUF_Q4_K, 2, seed=3)
    want = forward_with(oracle, cfg, weights, x[:1])
    with pf.MoeLayer(product, cfg, weights, 1) as layer:
        assert launches(product, layer) == 3
        _, y, ids, w = layer.forward(x[:1])
        assert_parity(y, ids, w, *want, label="three kernels")
    assert ATOL == 1e-3 and RTOL == 1e-4
