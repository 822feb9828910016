"""Shared helpers of the parity tests."""
import ctypes as C

import numpy as np

import picoforge_amd as pf
from picoforge_amd import abi

# Parity bar of the path: expert ids bit-exact; outputs within 1e-3 absolute plus
# 1e-4 relative of the CPU path on the same inputs (FP32 activations).
ATOL, RTOL = 1e-3, 1e-4


def make_layer_inputs(cfg, expert_type, tokens, seed, std=0.02, normalise=True, shared_type=None):
    synth = pf.Synth()
    weights = pf.LayerWeights.synthetic(cfg, expert_type, seed, std=std, shared_type=shared_type)
    x = synth.normal((tokens, cfg.hidden_size), 1000 + seed)
    if normalise and tokens:
        x = pf.rms_normalise(x)
    return weights, x


def forward_with(api, cfg, weights, x, cap=None):
    with pf.MoeLayer(api, cfg, weights, x.shape[0] if cap is None else cap) as layer:
        _, y, ids, w = layer.forward(x)
    return y, ids, w


def top_margin(api_oracle, cfg, weights, x):
    """Smallest gap between adjacent entries of the sorted top-(k+1) router logits, per token,
    from float64 logits (used to state how well separated a test's routing is)."""
    router = weights.raw[0].view(np.float32).reshape(cfg.experts, cfg.hidden_size).astype(np.float64)
    z = x.astype(np.float64) @ router.T
    k = min(cfg.top_k + 1, cfg.experts)
    top = -np.sort(-z, axis=1)[:, :k]
    return (top[:, :-1] - top[:, 1:]).min(axis=1) if k > 1 else np.full(len(x), np.inf)


def assert_parity(y, ids, w, y_ref, ids_ref, w_ref, label=""):
    np.testing.assert_array_equal(ids, ids_ref, err_msg=f"{label}: expert ids differ")
    np.testing.assert_allclose(w, w_ref, atol=2e-6, rtol=2e-5, err_msg=f"{label}: route weights")
    assert np.isfinite(y).all(), f"{label}: nonfinite output"
    err = np.abs(y.astype(np.float64) - y_ref.astype(np.float64))
    bound = ATOL + RTOL * np.abs(y_ref)
    worst = float((err / bound).max()) if err.size else 0.0
    assert worst <= 1.0, f"{label}: max abs err {err.max():.3e}, {worst:.2f}x the bound"
    return float(err.max()) if err.size else 0.0


def call_route(api, cfg, logits, pitch_pad=0):
    """qwen4_moe_route on dense or padded views; returns (status, probs, ids, weights, err)."""
    t, e = logits.shape
    k = cfg.top_k
    z = np.full((t, e + pitch_pad), -7.0, dtype=np.float32)
    z[:, :e] = logits
    p = np.full((t, e + pitch_pad), -99.0, dtype=np.float32)
    w = np.full((t, k + pitch_pad), -99.0, dtype=np.float32)
    ids = np.full((t, k + pitch_pad), 0xFFFFFFFF, dtype=np.uint32)
    routes = abi.Qwen4MoeRoutes(abi.u32_view(ids, cols=k), abi.f32_view(w, cols=k))
    err = abi.Qwen4Error()
    st = api.route(C.byref(cfg), abi.f32_view(z, cols=e), routes, abi.f32_view(p, cols=e), C.byref(err))
    return st, p, ids, w, err


def call_group(api, cfg, ids):
    t, k = ids.shape
    e = cfg.experts
    ids = np.ascontiguousarray(ids, dtype=np.uint32)
    fill = np.iinfo(np.uint64).max
    off = np.full(e + 2, fill, dtype=np.uint64)
    cur = np.full(e + 1, fill, dtype=np.uint64)
    p2r = np.full(t * k + 1, fill, dtype=np.uint64)
    r2p = np.full(t * k + 1, fill, dtype=np.uint64)
    g = abi.QW4MoeGrouping(off.ctypes.data, (e + 1) * 8, cur.ctypes.data, e * 8, p2r.ctypes.data, r2p.ctypes.data,
                           t * k * 8, t * k * 8)
    err = abi.Qwen4Error()
    st = api.group_pairs(C.byref(cfg), abi.u32_view(ids), g, C.byref(err))
    return st, off, cur, p2r, r2p


def call_matmul(api, raw, gtype, k_storage, n_out, experts, expert, x, k_logical=None):
    view = abi.packed_view(raw, gtype, k_storage, n_out, experts, k_logical)
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.full((x.shape[0], n_out), -99.0, dtype=np.float32)
    err = abi.Qwen4Error()
    st = api.matmul(C.byref(view), expert, abi.f32_view(x), abi.f32_view(y), C.byref(err))
    return st, y


def call_decode(api, raw, gtype, k_storage, rows, row, experts=1, expert=0):
    view = abi.packed_view(raw, gtype, k_storage, rows, experts)
    out = np.full(k_storage, -99.0, dtype=np.float32)
    err = abi.Qwen4Error()
    st = api.decode_row(C.byref(view), expert, row, out.ctypes.data, k_storage, C.byref(err))
    return st, out


def random_blocks(gtype, elements, rng, scale=0.125):
    """Random packed bytes of `elements` values in a format, every decoded value finite: block scales are
    halves drawn from +-scale (Q8_0, Q2_K, Q4_K, IQ2_XXS), exponents 110..140 (MXFP4), finite patterns
    (F16, BF16), N(0, 1) (F32)."""
    block, size = abi.BLOCK[gtype]
    assert elements % block == 0
    n = elements // block
    if gtype == abi.GGUF_F32:
        return rng.normal(0, 1, elements).astype(np.float32).view(np.uint8)
    if gtype in (abi.GGUF_F16, abi.GGUF_BF16):
        v = rng.normal(0, 1, elements).astype(np.float32)
        if gtype == abi.GGUF_F16:
            return v.astype(np.float16).view(np.uint8)
        return (v.view(np.uint32) >> 16).astype(np.uint16).view(np.uint8)
    raw = rng.integers(0, 256, (n, size), dtype=np.uint8)
    half = lambda: rng.uniform(-scale, scale, (n, 1)).astype(np.float16).view(np.uint8)  # noqa: E731
    if gtype == abi.GGUF_Q2_K:
        raw[:, 80:82] = half()
        raw[:, 82:84] = half()
    elif gtype == abi.GGUF_MXFP4:
        raw[:, 0] = rng.integers(110, 141, n, dtype=np.uint8)
    else:
        raw[:, 0:2] = half()
        if gtype == abi.GGUF_Q4_K:
            raw[:, 2:4] = half()
    return raw.reshape(-1)
