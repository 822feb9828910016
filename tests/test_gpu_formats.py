"""GPU parity on the formats real checkpoints use beside Q4_K and IQ2_XXS: F16, BF16, Q8_0 (shared
expert), Q2_K and MXFP4 (routed down projections).  Operators in reference order are bit-exact; the MoE
block on the two checkpoint profiles (src/qwen4_config.c:197-216: IQ2_XXS gate/up + Q2_K down, Q4_K
gate/up + MXFP4 down, Q8_0 shared expert in both) is held to the path's bar against the CPU oracle."""
import struct

import numpy as np
import pytest

import picoforge_amd as pf
from picoforge_amd import abi

from helpers import assert_parity, call_decode, call_matmul, forward_with, make_layer_inputs, random_blocks

pytestmark = pytest.mark.gpu
ALL = sorted(abi.BLOCK)


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


@pytest.mark.parametrize("gtype", ALL)
def test_decode_and_product_bit_exact_on_every_format(product, oracle, gtype):
    print(f"case format {abi.FORMAT_NAME[gtype]}", flush=True)
    rng = np.random.default_rng(500 + gtype)
    rows, k = 9, 768
    raw = random_blocks(gtype, rows * k, rng, scale=1.0)
    for row in range(rows):
        st0, want = call_decode(oracle, raw, gtype, k, rows, row)
        st1, got = call_decode(product, raw, gtype, k, rows, row)
        assert st0 == st1 == abi.QW4_OK
        np.testing.assert_array_equal(bits(got), bits(want))
    x = rng.uniform(-1, 1, (5, 640)).astype(np.float32)
    for expert in range(3):   # logical K 640 of 768 stored: padding is never read
        st0, want = call_matmul(oracle, raw, gtype, k, 3, 3, expert, x, k_logical=640)
        st1, got = call_matmul(product, raw, gtype, k, 3, 3, expert, x, k_logical=640)
        assert st0 == st1 == abi.QW4_OK
        np.testing.assert_array_equal(bits(got), bits(want))


def test_closed_forms_of_the_reference_tests(product):
    """tests/test_qwen4_packed.py:224-237, :362-367 through the device decoders."""
    def decode(raw, gtype, columns=256, rows=1):
        raw = np.frombuffer(bytes(raw), dtype=np.uint8).copy()
        return np.stack([call_decode(product, raw, gtype, columns, rows, r)[1] for r in range(rows)])
    raw = bytes([0x23]) * 16 + bytes([0xe4]) * 64 + struct.pack("<ee", 1, 0.5)
    np.testing.assert_array_equal(decode(raw, abi.GGUF_Q2_K)[0], np.tile(np.repeat([-1, 2, 5, 8], 32), 2))
    codes = np.arange(-128, 128, dtype=np.int16)
    raw = b"".join(struct.pack("<e", 0.125) + codes[s:s + 32].astype("i1").tobytes() for s in range(0, 256, 32))
    np.testing.assert_array_equal(bits(decode(raw, abi.GGUF_Q8_0)[0]), bits(codes.astype(np.float32) * 0.125))
    nib = bytes(i | ((15 - i) << 4) for i in range(16))
    got = decode(b"".join(bytes([e]) + nib for e in (0, 127, 252)), abi.GGUF_MXFP4, 32, 3)
    table = np.array([0, .5, 1, 1.5, 2, 3, 4, 6, -0.0, -.5, -1, -1.5, -2, -3, -4, -6], dtype=np.float32)
    for row, e in enumerate((0, 127, 252)):
        want = np.concatenate([table, table[::-1]]) * np.float32(2.0 ** (e - 127))
        np.testing.assert_array_equal(bits(got[row]), bits(want))
    r = np.frombuffer(bytes([254]) + nib, dtype=np.uint8).copy()
    assert call_decode(product, r, abi.GGUF_MXFP4, 32, 1, 0)[0] == abi.QW4_NONFINITE


PROFILES = [
    # hidden, experts, top_k, inter, shared_inter, down_physical, profile, tokens
    (256, 8, 3, 256, 256, 256, "q2", 5),
    (512, 16, 4, 512, 256, 512, "q4", 3),
    (256, 8, 3, 160, 96, 256, "q2", 2),      # logical K 160 stored in 256 (the checkpoint's 640 in 768)
    (512, 32, 6, 256, 256, 256, "q4", 1),
    (512, 32, 6, 256, 256, 256, "q2", 40),   # chunks: the matrix-core kernels
    (512, 32, 6, 256, 256, 256, "q4", 37),
]


@pytest.mark.parametrize("h,e,k,i,s,dp,profile,tokens", PROFILES)
def test_checkpoint_profiles_match_oracle(product, oracle, h, e, k, i, s, dp, profile, tokens):
    print(f"case profile {profile} h={h} e={e} k={k} i={i} s={s} down_physical={dp} T={tokens}", flush=True)
    cfg = abi.moe_config(h, e, k, i, s, down_physical=dp)
    if profile == "q4" and dp != i:
        pytest.skip("MXFP4 down tensors are stored at the logical width")
    if s % 32 or (profile == "q2" and i % 32):
        pytest.skip("block multiple")
    weights, x = make_layer_inputs(cfg, profile, tokens, seed=700 + h + tokens)
    want = forward_with(oracle, cfg, weights, x)
    got = forward_with(product, cfg, weights, x)
    worst = assert_parity(*got, *want, label=f"profile {profile}")
    print(f"  max abs err {worst:.2e}", flush=True)


@pytest.mark.parametrize("gtype", [abi.GGUF_F16, abi.GGUF_BF16, abi.GGUF_Q8_0])
def test_uniform_layers_of_the_plain_formats(product, oracle, gtype):
    cfg = abi.moe_config(128, 8, 2, 64, 32)
    weights, x = make_layer_inputs(cfg, gtype, 6, seed=800 + gtype, std=0.1)
    want = forward_with(oracle, cfg, weights, x)
    got = forward_with(product, cfg, weights, x)
    assert_parity(*got, *want, label=abi.FORMAT_NAME[gtype])


# shapes the decode kernels cover, on the two checkpoint profiles, 1..4 tokens per call (to 16 on the tile order)
DECODE_PROFILES = [
    (512, 32, 6, 256, 256, "q2", None), (512, 32, 6, 256, 256, "q4", None),
    (1024, 96, 5, 512, 256, "q2", None), (1024, 96, 5, 256, 1024, "q4", None),   # a shared expert wider than the routed ones
    (2048, 64, 10, 512, 512, "q2", None), (2048, 64, 10, 512, 512, "q4", None),  # the measured widths
    # the checkpoints' own widths (tests/fixtures/qwen4/text/config.json: hidden 2560, intermediate 640, shared 640;
    # the Q2_K down projection stored 768 wide): rows of 40 and 10 segments, two passes on some lanes
    (2560, 64, 10, 640, 640, "q2", 768), (2560, 64, 10, 640, 640, "q4", None), (2560, 512, 10, 640, 640, "q2", 768),
    (1280, 48, 4, 320, 320, "q2", 512), (768, 24, 3, 384, 448, "q4", None),
    (512, 32, 14, 1536, 256, "q4", None), (512, 32, 14, 1536, 512, "q2", None),   # wide activation rows: more than 64 KB of LDS in the down kernel
]


@pytest.mark.parametrize("h,e,k,i,s,profile,down_physical", DECODE_PROFILES)
def test_decode_kernels_on_checkpoint_profiles(product, oracle, h, e, k, i, s, profile, down_physical):
    print(f"case decode profile {profile} h={h} e={e} k={k} i={i} s={s} down stored {down_physical or i} wide", flush=True)
    cfg = abi.moe_config(h, e, k, i, s, down_physical=down_physical)
    weights, x = make_layer_inputs(cfg, profile, 16, seed=h + e + len(profile))
    x[3] = x[2]                                   # two identical tokens share every expert
    want = forward_with(oracle, cfg, weights, x)
    with pf.MoeLayer(product, cfg, weights, 16) as layer:
        moe, work = layer.device_handles()
        assert product.hip.moe_kernel_family(moe, work, 1) == 1, "the decode kernels do not cover this layer"
        # layers whose tile-ordered copies are kept take short batches of up to 16 tokens on the decode kernels too
        short = product.hip.moe_kernel_family(moe, work, 16) == 1
        assert short or h not in (2048, 2560), "the measured widths must be covered up to 16 tokens"
        for tokens in (1, 2, 3, 4) + ((7, 16) if short else ()):
            print(f"  tokens={tokens}", flush=True)
            _, y, ids, w = layer.forward(x[:tokens])
            worst = assert_parity(y, ids, w, want[0][:tokens], want[1][:tokens], want[2][:tokens],
                                  label=f"decode {profile} T={tokens}")
        print(f"  max abs err {worst:.2e}", flush=True)
        if (k * cfg.down_physical + s) * 4 <= 64 * 1024:   # the general kernels stage a token's activation rows in LDS
            layer.force_general()
            _, y, ids, w = layer.forward(x)
            assert_parity(y, ids, w, *want, label="general kernels on the same layer")


# chunks on the checkpoint profiles: the ring kernel for the routed gate/up tensors, the plain grouped
# product for the Q8_0 shared expert and the Q2_K / MXFP4 down tensors
PREFILL_PROFILES = [
    (256, 16, 4, 256, 256, 5), (256, 16, 4, 256, 256, 33), (512, 8, 3, 256, 512, 70),
    (256, 16, 4, 512, 256, 400),          # about 100 rows per expert: several row tiles
    (768, 40, 5, 256, 256, 129),
]


@pytest.mark.parametrize("profile", ["q2", "q4"])
@pytest.mark.parametrize("h,e,k,i,s,tokens", PREFILL_PROFILES)
def test_prefill_kernels_on_checkpoint_profiles(product, oracle, h, e, k, i, s, tokens, profile):
    print(f"case prefill profile {profile} h={h} e={e} k={k} i={i} s={s} T={tokens}", flush=True)
    cfg = abi.moe_config(h, e, k, i, s)
    weights, x = make_layer_inputs(cfg, profile, tokens, seed=h + e + tokens)
    want = forward_with(oracle, cfg, weights, x)
    with pf.MoeLayer(product, cfg, weights, tokens) as layer:
        moe, work = layer.device_handles()
        assert product.hip.moe_kernel_family(moe, work, tokens) == 2, "the prefill kernels do not cover this layer"
        _, y, ids, w = layer.forward(x)
        worst = assert_parity(y, ids, w, *want, label=f"prefill {profile} T={tokens}")
        print(f"  max abs err {worst:.2e}", flush=True)
        _, y2, _, _ = layer.forward(x)
        np.testing.assert_array_equal(y, y2, err_msg="not deterministic")
        if (k * cfg.down_physical + s) * 4 <= 64 * 1024:   # the general kernels stage a token's activation rows in LDS
            layer.force_general()
            _, y, ids, w = layer.forward(x)
            assert_parity(y, ids, w, *want, label="general kernels on the same layer")


# chunks at widths that are not whole 256-blocks: the checkpoints' own (hidden 2560, intermediate and shared 640, the
# Q2_K down projection stored 768 wide) and two smaller ones; (h, e, k, i, s, tokens)
PREFILL_ODD_WIDTHS = [(2560, 32, 4, 640, 640, 70), (512, 16, 3, 384, 128, 40), (768, 24, 5, 128, 896, 300)]


@pytest.mark.parametrize("profile", ["q2", "q4"])
@pytest.mark.parametrize("h,e,k,i,s,tokens", PREFILL_ODD_WIDTHS)
def test_prefill_kernels_at_checkpoint_widths(product, oracle, h, e, k, i, s, tokens, profile):
    print(f"case prefill profile {profile} h={h} e={e} k={k} i={i} s={s} T={tokens}", flush=True)
    cfg = abi.moe_config(h, e, k, i, s, down_physical=(i + 255) // 256 * 256 if profile == "q2" else i)
    weights, x = make_layer_inputs(cfg, profile, tokens, seed=h + i + tokens)
    want = forward_with(oracle, cfg, weights, x)
    with pf.MoeLayer(product, cfg, weights, tokens) as layer:
        moe, work = layer.device_handles()
        assert product.hip.moe_kernel_family(moe, work, tokens) == 2, "the prefill kernels do not cover this layer"
        _, y, ids, w = layer.forward(x)
        worst = assert_parity(y, ids, w, *want, label=f"prefill {profile} T={tokens}")
        print(f"  max abs err {worst:.2e}", flush=True)
        if (k * cfg.down_physical + s) * 4 <= 64 * 1024:   # the general kernels stage a token's activation rows in LDS
            layer.force_general()
            _, y, ids, w = layer.forward(x)
            assert_parity(y, ids, w, *want, label="general kernels on the same layer")


@pytest.mark.parametrize("profile", ["q2", "q4"])
def test_full_size_profile_layers(product, oracle, profile):
    """The measured shape (hidden 2048, 512 experts, top-10, intermediate 512, shared 512) in the checkpoint
    profiles: one to four decode tokens and the first rows of a 640-token chunk against the oracle, the whole
    chunk against the general kernels of the same library."""
    print(f"case full-size profile {profile}", flush=True)
    cfg = abi.moe_config(2048, 512, 10, 512, 512)
    weights, x = make_layer_inputs(cfg, profile, 640, seed=9)
    want = forward_with(oracle, cfg, weights, x[:6])
    with pf.MoeLayer(product, cfg, weights, 640) as layer:
        moe, work = layer.device_handles()
        assert product.hip.moe_kernel_family(moe, work, 4) == 1 and product.hip.moe_kernel_family(moe, work, 640) == 2
        for tokens in (1, 4):
            _, y, ids, w = layer.forward(x[:tokens])
            assert_parity(y, ids, w, want[0][:tokens], want[1][:tokens], want[2][:tokens], label=f"decode T={tokens}")
        _, y, ids, w = layer.forward(x)
        worst = assert_parity(y[:6], ids[:6], w[:6], *want, label="chunk, first rows against the oracle")
        layer.force_general()
        _, yg, idsg, wg = layer.forward(x)
        assert_parity(y, ids, w, yg, idsg, wg, label="chunk against the general kernels")
    print(f"  max abs err {worst:.2e}", flush=True)
