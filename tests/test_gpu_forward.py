"""GPU parity of qwen4_moe_forward: the HIP path through the C-ABI against the CPU oracle."""
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


# shapes the specialised decode kernels cover (power-of-two widths), 1..4 tokens per call
DECODE = [
    (512, 32, 6, 256, 256, abi.GGUF_Q4_K), (512, 32, 6, 256, 256, abi.GGUF_IQ2_XXS),
    (1024, 96, 5, 512, 256, abi.GGUF_Q4_K), (1024, 96, 5, 256, 1024, abi.GGUF_IQ2_XXS),
    (2048, 64, 10, 1024, 512, abi.GGUF_Q4_K),
]


@pytest.mark.parametrize("h,e,k,i,s,gtype", DECODE)
def test_decode_kernels_match_oracle_and_general_kernels(product, oracle, h, e, k, i, s, gtype):
    print(f"case decode h={h} e={e} k={k} i={i} s={s} type={gtype}", flush=True)
    cfg = abi.moe_config(h, e, k, i, s)
    weights, x = make_layer_inputs(cfg, gtype, 4, seed=h + e + gtype)
    x[3] = x[2]                                   # two identical tokens share every expert
    want = forward_with(oracle, cfg, weights, x)
    with pf.MoeLayer(product, cfg, weights, 4) as layer:
        for tokens in (1, 2, 3, 4):
            print(f"  tokens={tokens}", flush=True)
            _, y, ids, w = layer.forward(x[:tokens])
            assert_parity(y, ids, w, want[0][:tokens], want[1][:tokens], want[2][:tokens], label=f"decode T={tokens}")
        layer.force_general()
        _, y, ids, w = layer.forward(x)
        assert_parity(y, ids, w, *want, label="general kernels on a decode shape")


@pytest.mark.parametrize("norm", [True, False])
def test_decode_unnormalised_weights_and_repeat_calls(product, oracle, norm):
    cfg = abi.moe_config(512, 64, 4, 256, 256, norm=norm)
    weights, x = make_layer_inputs(cfg, abi.GGUF_Q4_K, 3, seed=77)
    want = forward_with(oracle, cfg, weights, x)
    with pf.MoeLayer(product, cfg, weights, 4) as layer:
        for _ in range(3):                        # the workspace is reused call after call
            _, y, ids, w = layer.forward(x)
            assert_parity(y, ids, w, *want, label=f"norm={norm}")


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
