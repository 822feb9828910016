"""GPU parity of qwen4_moe_forward: the HIP path through the C-ABI against the CPU oracle."""
import ctypes as C
import sys

import numpy as np
import pytest

import picoforge_amd as pf
from picoforge_amd import abi

from helpers import assert_parity, forward_with, make_layer_inputs, top_margin

pytestmark = pytest.mark.gpu

SMALL = [
    # hidden, experts, top_k, inter, shared_inter, expert type, tokens
    (8, 4, 2, 5, 3, abi.GGUF_F32, 2),
    (8, 4, 2, 5, 3, abi.GGUF_F32, 33),
    (64, 16, 4, 24, 12, abi.GGUF_F32, 7),
    (256, 16, 4, 256, 256, abi.GGUF_Q4_K, 7),
    (512, 32, 6, 256, 512, abi.GGUF_Q4_K, 5),
    (256, 16, 4, 256, 256, abi.GGUF_IQ2_XXS, 7),
    (768, 24, 3, 512, 256, abi.GGUF_IQ2_XXS, 4),
    (64, 1088, 3, 24, 12, abi.GGUF_F32, 6),       # more experts than a wave's registers hold: every token routed in serial order
]


@pytest.mark.parametrize("h,e,k,i,s,gtype,tokens", SMALL)
def test_small_layers_match_oracle(product, oracle, h, e, k, i, s, gtype, tokens):
    print(f"case h={h} e={e} k={k} i={i} s={s} type={gtype} T={tokens}", flush=True)
    cfg = abi.moe_config(h, e, k, i, s)
    std = 0.02 if gtype != abi.GGUF_F32 else 0.2
    weights, x = make_layer_inputs(cfg, gtype, tokens, seed=11 + h + tokens, std=std)
    want = forward_with(oracle, cfg, weights, x)
    got = forward_with(product, cfg, weights, x)
    assert_parity(*got, *want, label=f"h{h} e{e} type{gtype}")


# shapes the specialised decode kernels cover, 1..4 tokens per call; the last ones have rows whose 64-value
# segments are not a power of two in number (40, 12, 20), so some lanes take two segments
DECODE = [
    (512, 32, 6, 256, 256, abi.GGUF_Q4_K), (512, 32, 6, 256, 256, abi.GGUF_IQ2_XXS),
    (1024, 96, 5, 512, 256, abi.GGUF_Q4_K), (1024, 96, 5, 256, 1024, abi.GGUF_IQ2_XXS),
    (2048, 64, 10, 1024, 512, abi.GGUF_Q4_K),
    (512, 32, 14, 1536, 512, abi.GGUF_Q4_K),      # the widest activation rows: more than 64 KB of LDS in the down kernel
    (2560, 64, 10, 768, 768, abi.GGUF_Q4_K), (2560, 64, 10, 768, 256, abi.GGUF_IQ2_XXS), (1280, 40, 4, 256, 768, abi.GGUF_Q4_K),
]


@pytest.mark.parametrize("h,e,k,i,s,gtype", DECODE)
def test_decode_kernels_match_oracle_and_general_kernels(product, oracle, h, e, k, i, s, gtype):
    print(f"case decode h={h} e={e} k={k} i={i} s={s} type={gtype}", flush=True)
    cfg = abi.moe_config(h, e, k, i, s)
    weights, x = make_layer_inputs(cfg, gtype, 4, seed=h + e + gtype)
    x[3] = x[2]                                   # two identical tokens share every expert
    want = forward_with(oracle, cfg, weights, x)
    with pf.MoeLayer(product, cfg, weights, 4) as layer:
        assert product.hip.moe_kernel_family(*layer.device_handles(), 1) == 1, "the decode kernels do not cover this layer"
        for tokens in (1, 2, 3, 4):
            print(f"  tokens={tokens}", flush=True)
            _, y, ids, w = layer.forward(x[:tokens])
            assert_parity(y, ids, w, want[0][:tokens], want[1][:tokens], want[2][:tokens], label=f"decode T={tokens}")
        if (k * cfg.down_physical + s) * 4 <= 64 * 1024:   # the general kernels stage a token's activation rows in LDS
            layer.force_general()
            _, y, ids, w = layer.forward(x)
            assert_parity(y, ids, w, *want, label="general kernels on a decode shape")


@pytest.mark.parametrize("h,e,k,i,s,gtype", DECODE)
def test_decode_kernels_on_batches_of_up_to_sixteen_tokens(product, oracle, h, e, k, i, s, gtype):
    """From six tokens the down products run 64 output rows a workgroup with the digits as scalar operands: batches
    on either side of that switch, whole and ragged, against the oracle."""
    print(f"case decode batches h={h} e={e} k={k} i={i} s={s} type={gtype}", flush=True)
    cfg = abi.moe_config(h, e, k, i, s)
    weights, x = make_layer_inputs(cfg, gtype, 16, seed=3 * h + e + gtype)
    x[9] = x[8]                                   # two identical tokens share every expert
    want = forward_with(oracle, cfg, weights, x)
    with pf.MoeLayer(product, cfg, weights, 16) as layer:
        if product.hip.moe_kernel_family(*layer.device_handles(), 16) != 1:
            pytest.skip("batches of 16 tokens of this layer run the prefill kernels")
        for tokens in (5, 6, 7, 9, 13, 16):
            print(f"  tokens={tokens}", flush=True)
            _, y, ids, w = layer.forward(x[:tokens])
            assert_parity(y, ids, w, want[0][:tokens], want[1][:tokens], want[2][:tokens], label=f"decode T={tokens}")


# shapes the matrix-core prefill kernels cover (Q4_K or IQ2_XXS experts, widths in whole 256-blocks), more than 4 tokens
PREFILL = [
    (256, 16, 4, 256, 256, 5), (256, 16, 4, 256, 256, 33), (512, 8, 3, 256, 512, 70),
    (256, 16, 4, 512, 256, 400),          # about 100 rows per expert: several passes of 64 rows
    (768, 40, 5, 256, 256, 129),
]


@pytest.mark.parametrize("gtype", [abi.GGUF_Q4_K, abi.GGUF_IQ2_XXS])
@pytest.mark.parametrize("h,e,k,i,s,tokens", PREFILL)
def test_prefill_kernels_match_oracle_and_general_kernels(product, oracle, h, e, k, i, s, tokens, gtype):
    print(f"case prefill type={gtype} h={h} e={e} k={k} i={i} s={s} T={tokens}", flush=True)
    cfg = abi.moe_config(h, e, k, i, s)
    weights, x = make_layer_inputs(cfg, gtype, tokens, seed=h + e + tokens)
    want = forward_with(oracle, cfg, weights, x)
    with pf.MoeLayer(product, cfg, weights, tokens) as layer:
        _, y, ids, w = layer.forward(x)
        worst = assert_parity(y, ids, w, *want, label=f"prefill T={tokens}")
        print(f"  max abs err {worst:.2e}, serial-order reroutes {layer.serial_order_reroutes()}", flush=True)
        _, y2, ids2, _ = layer.forward(x)
        np.testing.assert_array_equal(y, y2, err_msg="prefill path is not deterministic")
        layer.force_general()
        _, y, ids, w = layer.forward(x)
        assert_parity(y, ids, w, *want, label="general kernels on a prefill shape")


def test_prefill_from_row_order_when_the_tile_ordered_copy_is_switched_off(product, oracle, monkeypatch):
    """PF_MOE_PREFILL_COPY=0 at create: the grouped product reads the GGUF row order, same results bit for bit.  A Q4_K
    layer keeps one copy of its experts either way: the tile-ordered one alone serves every kernel family."""
    cfg = abi.moe_config(512, 8, 3, 256, 512)
    weights, x = make_layer_inputs(cfg, abi.GGUF_Q4_K, 70, seed=590)
    want = forward_with(oracle, cfg, weights, x)
    with pf.MoeLayer(product, cfg, weights, 70) as layer:
        _, y_tiled, _, _ = layer.forward(x)
    monkeypatch.setenv("PF_MOE_PREFILL_COPY", "0")
    with pf.MoeLayer(product, cfg, weights, 70) as layer:
        bytes_without = product.hip.moe_bytes(layer.device_handles()[0])
        _, y, ids, w = layer.forward(x)
    monkeypatch.delenv("PF_MOE_PREFILL_COPY")
    with pf.MoeLayer(product, cfg, weights, 70) as layer:
        bytes_with = product.hip.moe_bytes(layer.device_handles()[0])
    assert_parity(y, ids, w, *want, label="prefill from the row order")
    np.testing.assert_array_equal(y, y_tiled, err_msg="the two weight orders give different results")
    assert bytes_with == bytes_without


def test_prefill_rows_of_very_different_magnitude(product, oracle):
    """Per-row power-of-two scaling: rows spanning 1e-6 .. 1e6 keep the relative accuracy."""
    cfg = abi.moe_config(256, 16, 4, 256, 256)
    weights, x = make_layer_inputs(cfg, abi.GGUF_Q4_K, 24, seed=77, normalise=False)
    scales = np.logspace(-6, 6, 24).astype(np.float32)
    x = (x / np.abs(x).max(axis=1, keepdims=True)) * scales[:, None]
    want = forward_with(oracle, cfg, weights, x)
    got = forward_with(product, cfg, weights, x)
    np.testing.assert_array_equal(got[1], want[1])
    rel = np.abs(got[0] - want[0]).max(axis=1) / np.maximum(np.abs(want[0]).max(axis=1), 1e-30)
    print("relative row errors", rel, flush=True)
    # fp16 operands: about 2^-11 per rounding, relative to the row's largest output, at every scale
    assert (rel < 4e-3).all() and rel.max() < 3 * rel.min() + 1e-3


def test_saturated_softmax_follows_the_reference_tie_rule(product, oracle):
    """Logits so far apart that exp() underflows: the reference picks the remaining experts by
    lowest id (equal zero probabilities), not by logit."""
    cfg = abi.moe_config(512, 32, 6, 256, 256)
    weights, x = make_layer_inputs(cfg, abi.GGUF_Q4_K, 4, seed=91)
    x = x * np.float32(3e4)
    want = forward_with(oracle, cfg, weights, x)
    assert (want[2] == 0).any(), "the case must contain underflowed probabilities"
    for tokens in (1, 4):
        got = forward_with(product, cfg, weights, x[:tokens])
        np.testing.assert_array_equal(got[1], want[1][:tokens])
        np.testing.assert_allclose(got[2], want[2][:tokens], atol=2e-6, rtol=2e-5)
        rel = np.abs(got[0] - want[0][:tokens]).max() / np.abs(want[0]).max()
        assert rel < 1e-4, rel


@pytest.mark.parametrize("gtype", [abi.GGUF_Q4_K, abi.GGUF_IQ2_XXS])
def test_full_size_prefill_rows_match_oracle(product, oracle, gtype):
    from picoforge_amd import workloads
    cfg = workloads.measured_config()
    weights, x = make_layer_inputs(cfg, gtype, 48, seed=5)
    print(f"full-size prefill, 48 tokens, type={gtype}", flush=True)
    want = forward_with(oracle, cfg, weights, x[:6])      # the CPU path costs 0.14 .. 0.26 s per token
    with pf.MoeLayer(product, cfg, weights, 48) as layer:
        _, y, ids, w = layer.forward(x)
        assert_parity(y[:6], ids[:6], w[:6], *want, label="full-size prefill")
        layer.force_general()
        _, yg, idsg, wg = layer.forward(x)
        assert_parity(y, ids, w, yg, idsg, wg, label="prefill against general kernels, all 48 rows")


LARGER_PREFILL = [
    # hidden, experts, top_k, inter, shared_inter, tokens, expert type: shapes where a workgroup walks several
    # work items, slabs are partial (768 = 256 + 512 rows ... ) and experts have many row tiles
    (1024, 128, 8, 768, 256, 777, abi.GGUF_Q4_K),
    (768, 24, 6, 1024, 512, 1500, abi.GGUF_Q4_K),
    (1024, 64, 4, 512, 768, 901, abi.GGUF_IQ2_XXS),
    (2048, 512, 10, 512, 512, 640, abi.GGUF_IQ2_XXS),
]


@pytest.mark.parametrize("h,e,k,i,s,tokens,gtype", LARGER_PREFILL)
def test_prefill_kernels_match_general_kernels_on_larger_shapes(product, h, e, k, i, s, tokens, gtype):
    """The matrix-core path against the FP32 dequantise-and-FMA kernels of the same library (written
    independently; each is checked against the oracle on smaller shapes)."""
    print(f"case larger prefill type={gtype} h={h} e={e} k={k} i={i} s={s} T={tokens}", flush=True)
    cfg = abi.moe_config(h, e, k, i, s)
    weights, x = make_layer_inputs(cfg, gtype, tokens, seed=h + e + tokens)
    with pf.MoeLayer(product, cfg, weights, tokens) as layer:
        _, y, ids, w = layer.forward(x)
        layer.force_general()
        _, yg, idsg, wg = layer.forward(x)
    worst = assert_parity(y, ids, w, yg, idsg, wg, label="prefill against general kernels")
    print(f"  max abs difference {worst:.2e} of the bound", flush=True)


@pytest.mark.parametrize("norm", [True, False])
def test_decode_unnormalised_weights_and_repeat_calls(product, oracle, norm):
    cfg = abi.moe_config(512, 64, 4, 256, 256, norm=norm)
    weights, x = make_layer_inputs(cfg, abi.GGUF_Q4_K, 3, seed=77)
    want = forward_with(oracle, cfg, weights, x)
    with pf.MoeLayer(product, cfg, weights, 4) as layer:
        for _ in range(3):                        # the workspace is reused call after call
            _, y, ids, w = layer.forward(x)
            assert_parity(y, ids, w, *want, label=f"norm={norm}")


@pytest.mark.parametrize("tokens", [1, 5, 16, 17])
def test_host_pointer_forward_with_padded_rows_and_without_routes(product, tokens):
    """Batches of up to 16 tokens pass through the workspace's pinned block (the output rows are written into it by the
    kernels, ids and weights arrive in one copy), longer ones through one copy per buffer: both must place rows at the
    caller's pitches, leave the padding alone and give the same rows with and without the routes asked for."""
    cfg = abi.moe_config(512, 64, 4, 256, 256)
    weights, x = make_layer_inputs(cfg, abi.GGUF_Q4_K, tokens, seed=31)
    h, k = cfg.hidden_size, cfg.top_k
    with pf.MoeLayer(product, cfg, weights, 32) as layer:
        _, y0, ids0, w0 = layer.forward(x)
        _, y1, _, _ = layer.forward(x, want_routes=False)
        assert np.array_equal(y0, y1)
        wide_x = np.full((tokens, h + 24), 7.0, dtype=np.float32)
        wide_x[:, :h] = x
        wide_y = np.full((tokens, h + 8), -5.0, dtype=np.float32)
        wide_ids = np.full((tokens, k + 3), 0xABCDEF01, dtype=np.uint32)
        wide_w = np.full((tokens, k + 1), -5.0, dtype=np.float32)
        routes = abi.Qwen4MoeRoutes(abi.u32_view(wide_ids, cols=k), abi.f32_view(wide_w, cols=k))
        st = product.forward(layer.handle, abi.f32_view(wide_x, cols=h), abi.f32_view(wide_y, cols=h), C.byref(routes),
                             layer.work, C.byref(layer.err))
        assert st == abi.QW4_OK, layer.err.detail
        assert np.array_equal(wide_y[:, :h], y0) and (wide_y[:, h:] == -5.0).all()
        assert np.array_equal(wide_ids[:, :k], ids0) and (wide_ids[:, k:] == 0xABCDEF01).all()
        assert np.array_equal(wide_w[:, :k], w0) and (wide_w[:, k:] == -5.0).all()


@pytest.mark.parametrize("tokens", [1, 4])
def test_host_pointer_forwards_in_turn_share_one_pinned_block(product, oracle, tokens):
    """Short batches stage their rows and results in one pinned block of the workspace: calls of different batch
    sizes, with and without routes, and on the general kernels, one after the other, must not see each other's rows."""
    cfg = abi.moe_config(512, 64, 4, 256, 256)
    weights, x = make_layer_inputs(cfg, abi.GGUF_Q4_K, 2 * tokens + 3, seed=41)
    xa, xb, xc = x[:tokens], x[tokens:2 * tokens], x[2 * tokens:]
    want_a, want_b = forward_with(oracle, cfg, weights, xa), forward_with(oracle, cfg, weights, xb)
    with pf.MoeLayer(product, cfg, weights, 8) as layer:
        _, ya, ids_a, w_a = layer.forward(xa)
        _, yb, _, _ = layer.forward(xb, want_routes=False)
        assert_parity(ya, ids_a, w_a, *want_a, label="first call")
        for turn in range(3):
            _, y, ids, w = layer.forward(xb)
            assert np.array_equal(y, yb), turn
            assert_parity(y, ids, w, *want_b, label=f"turn {turn}, second input")
            layer.forward(xc)                                       # another batch size in between
            _, y, ids, w = layer.forward(xa)
            assert np.array_equal(y, ya) and np.array_equal(ids, ids_a) and np.array_equal(w, w_a), turn
            _, y, _, _ = layer.forward(xa, want_routes=False)
            assert np.array_equal(y, ya), turn
            layer.force_general()
            _, yg, idsg, wg = layer.forward(xa)
            assert_parity(yg, idsg, wg, *want_a, label=f"general kernels, turn {turn}")
            layer.force_general(False)


def test_close_logits_are_rerouted_in_serial_order(product, oracle):
    """Two router rows that differ in the last place give logits closer than the guard's
    tolerance: the token must go through the reference-order path and still match the oracle."""
    cfg = abi.moe_config(512, 32, 6, 256, 256)
    weights, x = make_layer_inputs(cfg, abi.GGUF_Q4_K, 2, seed=5)
    router = weights.raw[0].view(np.float32).reshape(32, 512)
    z = x.astype(np.float64) @ router.astype(np.float64).T
    best = np.argsort(-z[0])[:3]
    router[best[1]] = router[best[0]]             # exact tie between the two best experts
    router[best[2]] = router[best[0]]
    router[best[2], 7] = np.nextafter(router[best[2], 7], np.float32(10))   # and a one-ulp neighbour
    want = forward_with(oracle, cfg, weights, x)
    for general in (False, True):
        with pf.MoeLayer(product, cfg, weights, 2) as layer:
            if general:
                layer.force_general()
            _, y, ids, w = layer.forward(x)
            assert_parity(y, ids, w, *want, label=f"tie general={general}")
            assert layer.serial_order_reroutes() >= 1


@pytest.mark.parametrize("norm", [True, False])
def test_many_near_ties_are_settled_by_the_doubtful_experts_alone(product, oracle, norm):
    """Router rows in pairs that differ by a few ulps in a few places: nearly every token has logits closer than the
    guard's tolerance among its best, some with equal probabilities (the lower id wins), some with probabilities a
    few ulps apart (all logits are then summed serially).  Ids must match the CPU path bit for bit on the decode
    kernels (1 and 16 tokens a call), the prefill kernels and the general ones."""
    cfg = abi.moe_config(512, 64, 6, 256, 256, norm=norm)
    tokens = 320
    weights, x = make_layer_inputs(cfg, abi.GGUF_Q4_K, tokens, seed=2024)
    router = weights.raw[0].view(np.float32).reshape(64, 512)
    rng = np.random.default_rng(7)
    for pair in range(32):
        twin = router[2 * pair].copy()
        for col in rng.choice(512, size=int(rng.integers(0, 4)), replace=False):   # 0 places: an exact twin
            for _ in range(int(rng.integers(1, 4))):
                twin[col] = np.nextafter(twin[col], np.float32(rng.choice([-10.0, 10.0])))
        router[2 * pair + 1] = twin
    want = forward_with(oracle, cfg, weights, x)
    with pf.MoeLayer(product, cfg, weights, tokens) as layer:
        for first in range(0, 24):                          # one token a call
            _, y, ids, w = layer.forward(x[first:first + 1])
            assert_parity(y, ids, w, want[0][first:first + 1], want[1][first:first + 1], want[2][first:first + 1],
                          label=f"near ties, token {first} alone")
        for first in range(0, tokens, 16):                  # short batches on the decode kernels
            _, y, ids, w = layer.forward(x[first:first + 16])
            assert_parity(y, ids, w, want[0][first:first + 16], want[1][first:first + 16], want[2][first:first + 16],
                          label=f"near ties, tokens {first}..{first + 15}")
        decode_reroutes, decode_full = layer.serial_order_reroutes(), layer.full_reroutes()
        _, y, ids, w = layer.forward(x)                      # one chunk on the prefill kernels
        assert_parity(y, ids, w, *want, label="near ties, prefill chunk")
        reroutes, full = layer.serial_order_reroutes() - decode_reroutes, layer.full_reroutes() - decode_full
        print(f"  decode calls: {decode_reroutes} re-routed, {decode_full} the long way; chunk: {reroutes} of {tokens} "
              f"re-routed, {full} the long way", flush=True)
        assert reroutes > tokens // 2, "the case must be full of near ties"
        assert full < reroutes, "the doubtful experts alone must settle some tokens"
        layer.force_general()
        _, y, ids, w = layer.forward(x)
        assert_parity(y, ids, w, *want, label="near ties, general kernels")


@pytest.mark.parametrize("clones", [24, 40, 80])
def test_crowds_of_near_equal_experts(product, oracle, clones):
    """Many router rows that are copies of one row up to a few ulps, and tokens that point along that row: the crowd
    fills the top of every token's logits, so the re-route sees 17..32, 33..64 or more than 64 doubtful experts (the
    last go the long way).  Decode, prefill and general kernels against the CPU path, ids bit for bit."""
    cfg = abi.moe_config(512, 128, 8, 256, 256)
    tokens = 48
    weights, x = make_layer_inputs(cfg, abi.GGUF_Q4_K, tokens, seed=77 + clones)
    router = weights.raw[0].view(np.float32).reshape(128, 512)
    rng = np.random.default_rng(clones)
    for e in range(1, clones):
        row = router[0].copy()
        for col in rng.choice(512, size=int(rng.integers(0, 3)), replace=False):   # 0 places: an exact copy
            row[col] = np.nextafter(row[col], np.float32(rng.choice([-10.0, 10.0])))
        router[e] = row
    x = (x * np.float32(0.3) + router[0][None, :] * np.float32(40.0)).astype(np.float32)   # the crowd's logit leads
    want = forward_with(oracle, cfg, weights, x)
    assert (want[1] < clones).all(), "every selected expert must come from the crowd"
    with pf.MoeLayer(product, cfg, weights, tokens) as layer:
        for first in range(0, 6):
            _, y, ids, w = layer.forward(x[first:first + 1])
            assert_parity(y, ids, w, want[0][first:first + 1], want[1][first:first + 1], want[2][first:first + 1],
                          label=f"crowd of {clones}, token {first} alone")
        _, y, ids, w = layer.forward(x[:16])
        assert_parity(y, ids, w, want[0][:16], want[1][:16], want[2][:16], label=f"crowd of {clones}, 16 tokens")
        _, y, ids, w = layer.forward(x)
        assert_parity(y, ids, w, *want, label=f"crowd of {clones}, chunk")
        reroutes, full = layer.serial_order_reroutes(), layer.full_reroutes()
        print(f"  crowd of {clones}: {reroutes} re-routed, {full} the long way", flush=True)
        assert reroutes >= tokens
        if clones > 64:
            assert full > 0, "more than 64 doubtful experts must go the long way"
        layer.force_general()
        _, y, ids, w = layer.forward(x)
        assert_parity(y, ids, w, *want, label=f"crowd of {clones}, general kernels")


def test_nonfinite_activation_is_reported_and_sticky_until_reset(product):
    cfg = abi.moe_config(512, 32, 6, 256, 256)
    weights, x = make_layer_inputs(cfg, abi.GGUF_Q4_K, 2, seed=6)
    big = weights.raw[1].copy()
    with pf.MoeLayer(product, cfg, weights, 2) as layer:
        bad = x.copy()
        bad[1, 3] = np.inf
        st, y, ids, w = layer.forward(bad, check=False)
        assert st == abi.QW4_NONFINITE and (y == -99).all()       # host preflight, outputs untouched
        st, y, ids, w = layer.forward(x, check=False)
        assert st == abi.QW4_OK                                   # a preflight failure does not poison the workspace
        huge = (x * np.float32(3e37)).astype(np.float32)          # finite input, overflow inside the block
        st, y, ids, w = layer.forward(huge, check=False)
        assert st == abi.QW4_NONFINITE and (y == -99).all()
        st, _, _, _ = layer.forward(x, check=False)
        assert st == abi.QW4_BAD_STATE                            # src/qwen4_moe.c:388,421
        assert layer.reset() == abi.QW4_OK
        st, _, _, _ = layer.forward(x, check=False)
        assert st == abi.QW4_OK
    del big


@pytest.mark.parametrize("gtype", [abi.GGUF_Q4_K, abi.GGUF_IQ2_XXS])
def test_full_size_decode_tokens_match_oracle(product, oracle, gtype):
    """The measured shape: hidden 2048, 512 experts, top-10, intermediate 512, one to four tokens."""
    print(f"case full-size type={gtype}", flush=True)
    cfg = abi.moe_config(2048, 512, 10, 512, 512)
    weights, x = make_layer_inputs(cfg, gtype, 4, seed=5)
    margins = top_margin(oracle, cfg, weights, x)
    want = forward_with(oracle, cfg, weights, x)
    with pf.MoeLayer(product, cfg, weights, 4) as layer:
        _, y, ids, w = layer.forward(x)
        worst = assert_parity(y, ids, w, *want, label=f"full type{gtype}")
        for tokens in (1, 2):
            _, y1, ids1, w1 = layer.forward(x[:tokens])
            assert_parity(y1, ids1, w1, want[0][:tokens], want[1][:tokens], want[2][:tokens], label=f"T={tokens}")
        layer.force_general()
        _, y, ids, w = layer.forward(x[:2])
        assert_parity(y, ids, w, want[0][:2], want[1][:2], want[2][:2], label="general kernels, full size")
    print(f"margins {margins}, max abs err {worst:.3e}", file=sys.stderr)
