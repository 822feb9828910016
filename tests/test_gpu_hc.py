"""GPU parity of the hyper-connection read and add either side of the MoE block, and of the
chained read -> MoE -> add, through the C-ABI against the CPU oracle.

Both steps are bit-exact: the add is one rounded product and one rounded sum; the read keeps the
CPU loop's order and evaluates the sigmoid's exponential with the C library's own expf algorithm
in IEEE double steps, so on a host whose C library is glibc 2.27 or later (this image) every bit
of the read matches the oracle, which calls that library.
"""
import ctypes as C

import numpy as np
import pytest

import picoforge_amd as pf
from picoforge_amd import abi

from hc_cases import SHAPES, call_add, call_read, hc_shape, pitched, random_case, run_error_case
from helpers import ATOL, RTOL, make_layer_inputs

pytestmark = pytest.mark.gpu

def assert_same_bits(got, want, what):
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32), err_msg=what)


def test_known_answers_of_the_reference_c_test(product):
    normed = np.array([[[1, 2, 3], [10, 20, 30]]], dtype=np.float32)
    st, mixed, _ = call_read(product, normed, np.zeros_like(normed))
    assert st == abi.QW4_OK
    np.testing.assert_array_equal(mixed, [[2.75, 5.5, 8.25]])
    st, _ = call_add(product, normed, np.array([[3, -2, 1]], dtype=np.float32), np.ones((1, 2), dtype=np.float32))
    assert st == abi.QW4_OK
    np.testing.assert_array_equal(normed.ravel(), [4, 0, 4, 13, 18, 31])


@pytest.mark.parametrize("t,h,w", SHAPES + [(70, 4, 4096), (5, 7, 260), (2, 20, 96), (40, 20, 2048)])
@pytest.mark.parametrize("scale", [1.0, 30.0])
def test_read_and_add_match_oracle(product, oracle, t, h, w, scale):
    print(f"case hc T={t} streams={h} hidden={w} scale={scale}", flush=True)
    normed, logits, block, inject = random_case(t, h, w, 31 + t + w, scale=scale)
    if t:
        logits.ravel()[:4] = (0.0, -0.0, 89.0, -104.0)
    st_o, want, _ = call_read(oracle, normed, logits)
    st_p, got, _ = call_read(product, normed, logits)
    assert st_o == st_p == abi.QW4_OK
    assert_same_bits(got, want, "read")
    res_o, res_p = normed.copy(), normed.copy()
    assert call_add(oracle, res_o, block, inject)[0] == call_add(product, res_p, block, inject)[0] == abi.QW4_OK
    np.testing.assert_array_equal(res_p.view(np.uint32), res_o.view(np.uint32))


def test_sigmoid_of_the_read_matches_the_c_library_on_a_sweep(product, oracle):
    """One stream of ones: mixed = sigmoid(logit) exactly.  Two million logits: random bit patterns within
    +-110, every float next to the underflow threshold of expf, and the reference test's special values
    (tests/test_qwen4_fast_kernels.py:2742)."""
    rng = np.random.default_rng(5)
    x = rng.integers(0, 2 ** 32, 2_000_000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    keep = np.isfinite(x) & (np.abs(x) < 110.0)
    x = np.where(keep, x, rng.uniform(-110.0, 110.0, x.size).astype(np.float32))
    edge = np.float32(-103.97208)
    near = [edge]
    for _ in range(2000):
        near.append(np.nextafter(near[-1], np.float32(0)))
    x[:2001] = near
    x[2001:2009] = (0.0, -0.0, 89.0, -104.0, 88.72284, -88.72284, 1e-30, -1e-30)
    logits = x.reshape(1000, 1, 2000)
    ones = np.ones_like(logits)
    st_o, want, _ = call_read(oracle, ones, logits)
    st_p, got, _ = call_read(product, ones, logits)
    assert st_o == st_p == abi.QW4_OK
    assert_same_bits(got, want, "sigmoid sweep")


@pytest.mark.parametrize("t,h,w", [(3, 4, 64), (7, 3, 33), (6, 4, 256)])
def test_pitched_views_touch_only_their_elements(product, oracle, t, h, w):
    normed, logits, block, inject = random_case(t, h, w, 41)
    _, want, _ = call_read(oracle, normed, logits)
    _, view_n = pitched(normed, 1, 3)
    _, view_g = pitched(logits, 2, 5)
    mixed = np.full((t, w + 9), -99.0, dtype=np.float32)
    st, _, _ = call_read(product, normed, logits, mixed,
                         views=(abi.f32_cube(view_n), abi.f32_cube(view_g), abi.f32_view(mixed, cols=w)))
    assert st == abi.QW4_OK
    assert_same_bits(np.ascontiguousarray(mixed[:, :w]), want, "read through pitched views")
    assert (mixed[:, w:] == -99.0).all()
    dense = normed.copy()
    call_add(oracle, dense, block, inject)
    big_r, view_r = pitched(normed, 2, 7)
    wide_b = np.full((t, w + 3), 55.0, dtype=np.float32)
    wide_b[:, :w] = block
    st, _ = call_add(product, view_r, block, inject,
                     views=(abi.f32_cube(view_r), abi.f32_view(wide_b, cols=w), abi.f32_view(inject)))
    assert st == abi.QW4_OK
    np.testing.assert_array_equal(view_r, dense)
    assert (big_r[:, h:, :] == -77.0).all() and (big_r[:, :, w:] == -77.0).all()


@pytest.mark.parametrize("op,which,index", [("read", 0, (1, 2, 3)), ("read", 1, (0, 0, 0)), ("add", 0, (1, 3, 63)),
                                            ("add", 1, (0, 5)), ("add", 2, (1, 3))])
@pytest.mark.parametrize("value", [np.nan, np.inf, -np.inf])
def test_nonfinite_inputs_are_reported_and_outputs_untouched(product, oracle, op, which, index, value):
    def mutate(views, arrays, shape):
        arrays[which][index] = value
    st_o, _, _ = run_error_case(oracle, op, mutate)
    st_p, out, err = run_error_case(product, op, mutate)
    assert st_p == st_o == abi.QW4_NONFINITE and err.code == abi.QW4_NONFINITE
    if op == "read":
        assert (out == -99.0).all()
    else:   # the residual keeps its values (the poisoned element included)
        expect = random_case(2, 4, 64, 15)[0]
        if which == 0:
            expect[index] = value
        np.testing.assert_array_equal(out.view(np.uint32), expect.view(np.uint32))


def test_overflow_is_reported_and_outputs_untouched(product):
    big = np.float32(3e38)
    normed = np.full((2, 4, 8), 1.0, dtype=np.float32)
    normed[1, :, 3] = big
    st, mixed, _ = call_read(product, normed, np.full_like(normed, 40.0))
    assert st == abi.QW4_NONFINITE and (mixed == -99.0).all()
    residual = np.full((2, 4, 8), 1.0, dtype=np.float32)
    residual[1, 2, 5] = big
    block = np.full((2, 8), big, dtype=np.float32)
    block[0] = 1.0
    before = residual.copy()
    st, _ = call_add(product, residual, block, np.ones((2, 4), dtype=np.float32))
    assert st == abi.QW4_NONFINITE
    np.testing.assert_array_equal(residual, before)


# ---- the chain read -> MoE -> add ---------------------------------------------------------------
CHAIN = [
    # hidden, experts, top_k, inter, shared_inter, expert type, tokens, streams
    (8, 4, 2, 5, 3, abi.GGUF_F32, 3, 2),                 # general kernels
    (64, 16, 4, 24, 12, abi.GGUF_F32, 7, 3),
    (512, 32, 6, 256, 256, abi.GGUF_Q4_K, 1, 4),         # decode kernels
    (512, 32, 6, 256, 256, abi.GGUF_IQ2_XXS, 4, 4),
    (1024, 96, 5, 512, 256, abi.GGUF_Q4_K, 3, 1),
    (256, 16, 4, 256, 256, abi.GGUF_Q4_K, 33, 4),        # prefill kernels
    (512, 32, 6, 256, 256, abi.GGUF_Q4_K, 11, 4),        # Q4_K decode kernels, one token per grid row
    (512, 8, 3, 256, 512, abi.GGUF_IQ2_XXS, 70, 4),
    (768, 40, 5, 256, 256, abi.GGUF_Q4_K, 129, 2),
    (512, 32, 6, 256, 256, abi.GGUF_Q4_K, 2, 6),         # more streams than the last kernel folds in: separate add
    (256, 16, 4, 256, 256, abi.GGUF_IQ2_XXS, 33, 5),
    (512, 32, 6, 256, 256, "q2", 3, 4),                  # checkpoint profiles on the decode kernels
    (512, 32, 6, 256, 256, "q4", 9, 4),                  # ... a chunk, four tokens per launch
    (2560, 48, 10, 640, 640, "q2", 1, 4),                # the checkpoints' widths (Q2_K down stored 768 wide): decode
    (2560, 48, 10, 640, 640, "q4", 40, 4),               # ... and a chunk
]


def chain_inputs(cfg, tokens, streams, seed):
    """Residual streams whose gated mix has unit RMS, as the block sees after the norm."""
    rng = np.random.default_rng(seed)
    h = cfg.hidden_size
    normed = rng.standard_normal((tokens, streams, h)).astype(np.float32) * np.float32(1.8)
    logits = rng.standard_normal((tokens, streams, h)).astype(np.float32)
    residual = rng.standard_normal((tokens, streams, h)).astype(np.float32)
    inject = rng.uniform(0.0, 2.0 / streams, (tokens, streams)).astype(np.float32)
    return normed, logits, residual, inject


@pytest.mark.parametrize("h,e,k,i,s,gtype,tokens,streams", CHAIN)
def test_chained_forward_matches_oracle_stage_by_stage(product, oracle, h, e, k, i, s, gtype, tokens, streams):
    print(f"case chain h={h} e={e} k={k} type={gtype} T={tokens} streams={streams}", flush=True)
    cfg = abi.moe_config(h, e, k, i, s, down_physical=(i + 255) // 256 * 256 if gtype == "q2" else i)
    weights, _ = make_layer_inputs(cfg, gtype, 1, seed=3 * h + tokens, std=0.02 if gtype != abi.GGUF_F32 else 0.2)
    normed, logits, residual, inject = chain_inputs(cfg, tokens, streams, 900 + h + tokens)
    # the device's own mixed rows, so that every later stage is compared on identical inputs
    st, mixed, _ = call_read(product, normed, logits, shape=hc_shape(streams, h))
    assert st == abi.QW4_OK
    _, mixed_cpu, _ = call_read(oracle, normed, logits, shape=hc_shape(streams, h))
    assert_same_bits(mixed, mixed_cpu, "read")
    with pf.MoeLayer(oracle, cfg, weights, tokens) as cpu:
        _, y_ref, ids_ref, w_ref = cpu.forward(mixed)
    want = residual.copy()
    assert call_add(oracle, want, y_ref, inject, shape=hc_shape(streams, h))[0] == abi.QW4_OK
    with pf.MoeLayer(product, cfg, weights, tokens) as layer:
        fused = residual.copy()
        _, ids, w = layer.forward_hc(normed, logits, fused, inject)
        unfused = residual.copy()
        _, ids_u, w_u = layer.forward_hc(normed, logits, unfused, inject, fused=False)
        _, y_dev, _, _ = layer.forward(mixed)
    np.testing.assert_array_equal(ids, ids_ref, err_msg="expert ids differ")
    np.testing.assert_array_equal(ids_u, ids_ref)
    np.testing.assert_allclose(w, w_ref, atol=2e-6, rtol=2e-5)
    # residual + weight * y: the block's tolerance scaled by the injection weight
    scale = np.abs(inject)[:, :, None]
    bound = scale * (ATOL + RTOL * np.abs(y_ref)[:, None, :]) + 1e-6 * np.abs(want)
    err = np.abs(fused.astype(np.float64) - want)
    assert (err <= bound).all(), float((err / bound).max())
    print(f"  max abs err of the residual {err.max():.2e} (block output {np.abs(y_dev - y_ref).max():.2e})", flush=True)
    # folding the add into the block's last kernel changes no bit
    np.testing.assert_array_equal(fused.view(np.uint32), unfused.view(np.uint32))


def test_chained_forward_validation_and_errors(product):
    cfg = abi.moe_config(64, 16, 4, 24, 12)
    weights, _ = make_layer_inputs(cfg, abi.GGUF_F32, 1, seed=5, std=0.2)
    normed, logits, residual, inject = chain_inputs(cfg, 3, 2, 77)
    with pf.MoeLayer(product, cfg, weights, 3) as layer:
        before = residual.copy()
        bad = normed.copy()
        bad[1, 1, 5] = np.nan
        st, ids, _ = layer.forward_hc(bad, logits, residual, inject, check=False)
        assert st == abi.QW4_NONFINITE
        np.testing.assert_array_equal(residual, before)
        assert (ids == 0xFFFFFFFF).all()
        # sticky until reset, as qwen4_moe_forward
        assert layer.forward_hc(normed, logits, residual, inject, check=False)[0] == abi.QW4_BAD_STATE
        assert layer.reset() == abi.QW4_OK
        # wrong hidden size, too many tokens, residual inside an input
        wide = np.zeros((3, 2, 128), dtype=np.float32)
        assert layer.forward_hc(wide, wide.copy(), wide.copy(), inject, check=False)[0] == abi.QW4_SHAPE
        more = chain_inputs(cfg, 4, 2, 78)
        assert layer.forward_hc(*more, check=False)[0] == abi.QW4_CAPACITY
        assert layer.forward_hc(normed, logits, normed, inject, check=False)[0] == abi.QW4_INVALID_ARGUMENT
        np.testing.assert_array_equal(residual, before)
        assert layer.forward_hc(normed, logits, residual, inject)[0] == abi.QW4_OK
        assert not np.array_equal(residual, before)


def test_device_resident_chain_accumulates_like_the_host_calls(product):
    """pf_hip_moe_forward_hc_device enqueued three times on device buffers (through the benchmark's plan,
    which replays it from a HIP graph) adds the same bits as three host-buffer calls, fused or not."""
    from bench import Tools
    tools = Tools()
    cfg = abi.moe_config(512, 32, 6, 256, 256)
    weights, _ = make_layer_inputs(cfg, abi.GGUF_Q4_K, 1, seed=8)
    hip = product.hip
    for tokens in (1, 4, 40):
        normed, logits, residual, inject = chain_inputs(cfg, tokens, 4, 300 + tokens)
        with pf.MoeLayer(product, cfg, weights, tokens) as layer:
            want = residual.copy()
            for _ in range(3):
                layer.forward_hc(normed, logits, want, inject)
            moe, work = layer.device_handles()
            d_n, d_g, d_i = hip.to_device(normed), hip.to_device(logits), hip.to_device(inject)
            for fused in (1, 0):
                d_r = hip.to_device(residual)
                plan = tools.plan_hc(moe, work, d_n, d_g, 1, d_r, d_i, 4, tokens, 3, fused, cfg.hidden_size)
                tools.run(plan, 1)
                tools.destroy(plan)
                got = hip.from_device(d_r, residual.shape, np.float32)
                hip.free(d_r)
                np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32),
                                              err_msg=f"tokens={tokens} fused={fused}")
            for p in (d_n, d_g, d_i):
                hip.free(p)
