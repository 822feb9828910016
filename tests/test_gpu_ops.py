"""GPU parity of the stand-alone operators: route, group, packed decode and product.

Integer and index results are compared bit for bit; the reference-order kernels
(packed product, decode, route on given logits) are compared bit for bit too.
"""
import struct

import numpy as np
import pytest

from picoforge_amd import abi

from helpers import call_decode, call_group, call_matmul, call_route

pytestmark = pytest.mark.gpu


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


# ---- route ----------------------------------------------------------------------
def test_route_known_answers(product):
    # ties go to the lower id; reference's unit vectors (tests/test_qwen4_moe.c:52-63)
    cfg = abi.moe_config(8, 4, 2, 5, 3)
    z = np.array([[0, 1e-9, 0, -1e-9], [0, 2, 2, -1000]], dtype=np.float32)
    st, p, ids, w, _ = call_route(product, cfg, z, pitch_pad=3)
    assert st == abi.QW4_OK
    np.testing.assert_array_equal(ids[:, :2], [[0, 1], [1, 2]])
    np.testing.assert_array_equal(w[:, :2], [[0.5, 0.5], [0.5, 0.5]])
    assert p[0, 0] == 0.25 and p[1, 3] == 0.0
    assert (p[:, 4:] == -99).all() and (w[:, 2:] == -99).all() and (ids[:, 2:] == 0xFFFFFFFF).all()
    cfg.norm_topk_prob = False
    st, p, ids, w, _ = call_route(product, cfg, z)
    assert w[0, 0] == 0.25
    cfg.norm_topk_prob = True
    z = np.array([[-3e38, 3e38, 0, -1e-9]], dtype=np.float32)
    st, p, ids, w, _ = call_route(product, cfg, z)
    np.testing.assert_array_equal(ids[0], [1, 0])
    np.testing.assert_array_equal(w[0], [1.0, 0.0])


def test_route_nonfinite_leaves_outputs_untouched(product):
    cfg = abi.moe_config(8, 4, 2, 5, 3)
    for bad in (np.nan, np.inf):
        z = np.zeros((3, 4), dtype=np.float32)
        z[2, 1] = bad
        st, p, ids, w, err = call_route(product, cfg, z)
        assert st == abi.QW4_NONFINITE and err.row == 2
        assert (p == -99).all() and (w == -99).all() and (ids == 0xFFFFFFFF).all()


@pytest.mark.parametrize("experts,k,tokens", [(512, 10, 64), (4, 2, 5), (100, 7, 9), (2048, 8, 3)])
def test_route_matches_oracle(product, oracle, experts, k, tokens):
    rng = np.random.default_rng(experts + k)
    cfg = abi.moe_config(8, experts, k, 5, 3)
    z = rng.normal(0, 1.5, (tokens, experts)).astype(np.float32)
    z[0] = 0                                   # all tied: ids 0..k-1
    if tokens > 2:
        z[1, ::3] = z[1, 0]                    # many exact ties
        z[2] = np.round(z[2] * 4) / 4          # quantised logits: ties across experts
    st0, p0, i0, w0, _ = call_route(oracle, cfg, z)
    st1, p1, i1, w1, _ = call_route(product, cfg, z)
    assert st0 == st1 == abi.QW4_OK
    np.testing.assert_array_equal(i1, i0)
    # probabilities and weights follow the reference's evaluation order and the kernels evaluate the
    # C library's expf algorithm step by step: every bit matches
    np.testing.assert_array_equal(p1.view(np.uint32), p0.view(np.uint32))
    np.testing.assert_array_equal(w1.view(np.uint32), w0.view(np.uint32))


# ---- group ----------------------------------------------------------------------
def test_group_known_answer_and_errors(product):
    cfg = abi.moe_config(8, 4, 2, 5, 3)
    ids = np.array([[2, 0], [1, 2], [2, 0]], dtype=np.uint32)   # tests/test_qwen4_moe.c:140,173-176
    st, off, cur, p2r, r2p = call_group(product, cfg, ids)
    assert st == abi.QW4_OK
    np.testing.assert_array_equal(off[:5], [0, 2, 3, 6, 6])
    np.testing.assert_array_equal(r2p[:6], [1, 5, 2, 0, 3, 4])
    np.testing.assert_array_equal(p2r[r2p[:6].astype(np.int64)], np.arange(6))
    np.testing.assert_array_equal(cur[:4], off[1:5])
    fill = np.iinfo(np.uint64).max
    assert off[5] == fill and cur[4] == fill and p2r[6] == fill and r2p[6] == fill
    for bad, status in (([[2, 0], [1, 2], [4, 0]], abi.QW4_RANGE), ([[2, 0], [1, 2], [2, 2]], abi.QW4_INVALID_ARGUMENT)):
        st, off, cur, p2r, r2p = call_group(product, cfg, np.array(bad, dtype=np.uint32))
        assert st == status
        assert (off == fill).all() and (cur == fill).all() and (p2r == fill).all() and (r2p == fill).all()


@pytest.mark.parametrize("tokens,experts,k", [(1, 512, 10), (4, 512, 10), (1024, 512, 10), (65, 7, 3), (0, 4, 2)])
def test_group_matches_stable_argsort(product, oracle, tokens, experts, k):
    rng = np.random.default_rng(tokens + experts)
    ids = np.stack([rng.permutation(experts)[:k] for _ in range(tokens)]).astype(np.uint32) if tokens else \
        np.zeros((0, k), dtype=np.uint32)
    cfg = abi.moe_config(8, experts, k, 5, 3)
    st, off, cur, p2r, r2p = call_group(product, cfg, ids)
    assert st == abi.QW4_OK
    flat = ids.reshape(-1).astype(np.int64)
    order = np.argsort(flat, kind="stable")
    np.testing.assert_array_equal(off[:experts + 1], np.concatenate([[0], np.cumsum(np.bincount(flat, minlength=experts))]))
    np.testing.assert_array_equal(r2p[:tokens * k], order)
    if tokens:
        st0, off0, cur0, p2r0, r2p0 = call_group(oracle, cfg, ids)
        np.testing.assert_array_equal(p2r, p2r0)
        np.testing.assert_array_equal(cur[:experts], cur0[:experts])


# ---- packed decode and product ----------------------------------------------------
def test_decode_all_half_patterns_through_q4k_and_iq2(product, oracle):
    # every finite binary16 value as d of a block whose decoded value equals d * small integer
    halves = np.arange(65536, dtype=np.uint32)
    halves = halves[(halves & 0x7C00) != 0x7C00]
    rng = np.random.default_rng(1)
    pick = np.concatenate([halves[:2048], halves[31744 - 64:31744], halves[32768:32768 + 2048],
                           rng.choice(halves, 512)]).astype(np.uint16)
    blocks = np.zeros((len(pick), 66), dtype=np.uint8)
    blocks[:, 0:2] = pick.view(np.uint8).reshape(-1, 2)
    raw = blocks.reshape(-1)
    for row in range(0, len(pick), 97):
        st0, want = call_decode(oracle, raw, abi.GGUF_IQ2_XXS, 256, len(pick), row)
        st1, got = call_decode(product, raw, abi.GGUF_IQ2_XXS, 256, len(pick), row)
        assert st0 == st1 == abi.QW4_OK
        np.testing.assert_array_equal(bits(got), bits(want))


@pytest.mark.parametrize("gtype,size", [(abi.GGUF_Q4_K, 144), (abi.GGUF_IQ2_XXS, 66)])
def test_decode_and_product_random_blocks_bit_exact(product, oracle, gtype, size):
    rng = np.random.default_rng(7 + gtype)
    rows, k = 9, 768
    blocks = rng.integers(0, 256, (rows * k // 256, size), dtype=np.uint8)
    scale = rng.uniform(-1, 1, (len(blocks), 1)).astype(np.float16).view(np.uint8)
    blocks[:, 0:2] = scale
    if gtype == abi.GGUF_Q4_K:
        blocks[:, 2:4] = rng.uniform(0, 1, (len(blocks), 1)).astype(np.float16).view(np.uint8)
    raw = blocks.reshape(-1)
    for row in range(rows):
        st0, want = call_decode(oracle, raw, gtype, k, rows, row)
        st1, got = call_decode(product, raw, gtype, k, rows, row)
        assert st0 == st1 == abi.QW4_OK
        np.testing.assert_array_equal(bits(got), bits(want))
    x = rng.uniform(-1, 1, (5, 640)).astype(np.float32)
    # three experts of three rows each; logical K 640 of 768 stored: padding is never read
    for expert in range(3):
        st0, want = call_matmul(oracle, raw, gtype, k, 3, 3, expert, x, k_logical=640)
        st1, got = call_matmul(product, raw, gtype, k, 3, 3, expert, x, k_logical=640)
        assert st0 == st1 == abi.QW4_OK
        np.testing.assert_array_equal(bits(got), bits(want))


def test_product_f32_overflow_and_empty(product):
    raw = np.array([2.0 ** 127, 2.0 ** 127], dtype=np.float32).view(np.uint8)
    st, y = call_matmul(product, raw, abi.GGUF_F32, 2, 1, 1, 0, np.ones((1, 2), dtype=np.float32))
    assert st == abi.QW4_NONFINITE and (y == -99).all()      # sum overflows (tests/test_qwen4_packed.c:111-118)
    st, y = call_matmul(product, np.array([np.nan], dtype=np.float32).view(np.uint8), abi.GGUF_F32, 1, 1, 1, 0,
                        np.zeros((0, 1), dtype=np.float32))
    assert st == abi.QW4_OK                                   # zero rows never look at the weights
    ones = np.ones(640, dtype=np.float32).view(np.uint8)
    st, y = call_matmul(product, ones, abi.GGUF_F32, 640, 1, 1, 0, np.ones((3, 640), dtype=np.float32))
    assert st == abi.QW4_OK and (y == 640).all()
