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


@pytest.mark.parametrize("gtype", [abi.GGUF_Q4_K, abi.GGUF_IQ2_XXS])
def test_full_size_decode_tokens_match_oracle(product, oracle, gtype):
    """The measured shape: hidden 2048, 512 experts, top-10, intermediate 512, one and four tokens."""
    print(f"case full-size type={gtype}", flush=True)
    cfg = abi.moe_config(2048, 512, 10, 512, 512)
    weights, x = make_layer_inputs(cfg, gtype, 4, seed=5)
    margins = top_margin(oracle, cfg, weights, x)
    want = forward_with(oracle, cfg, weights, x)
    with pf.MoeLayer(product, cfg, weights, 4) as layer:
        _, y, ids, w = layer.forward(x)
        worst = assert_parity(y, ids, w, *want, label=f"full type{gtype}")
        _, y1, ids1, w1 = layer.forward(x[:1])
        assert_parity(y1, ids1, w1, want[0][:1], want[1][:1], want[2][:1], label="single token")
    print(f"margins {margins}, max abs err {worst:.3e}", file=sys.stderr)
