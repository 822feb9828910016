"""GPU parity on the benchmark configurations themselves, at their full shape
(hidden 2048, 512 experts, top-10, intermediate 512, shared 512): Q4_K chunks of 1024, 1777 and 2048 tokens
under a Zipf(1.1) router, the 4-token verify batches with about half of the experts shared between
neighbours, and a stack of independent layers."""
import ctypes as C

import numpy as np
import pytest

import picoforge_amd as pf
from picoforge_amd import abi, workloads

from helpers import ATOL, RTOL, assert_parity, call_matmul, call_route, forward_with, make_layer_inputs

pytestmark = pytest.mark.gpu


def oracle_routes(oracle, cfg, weights, x):
    """Router logits in the reference's serial order (the F32 packed product) and its routing, for every token."""
    st, logits = call_matmul(oracle, weights.raw[0], abi.GGUF_F32, cfg.hidden_size, cfg.experts, 1, 0, x)
    assert st == abi.QW4_OK
    st, _, ids, w, _ = call_route(oracle, cfg, logits)
    assert st == abi.QW4_OK
    return ids, w


def pick_chunk_rows(ids0, load, tokens):
    """Rows of the busiest experts (first, middle and last of their row lists), of the least loaded ones, and the
    chunk's first, middle and last rows."""
    picked = []
    for e in np.argsort(-load)[:6]:
        rows = np.nonzero((ids0 == e).any(axis=1))[0]
        picked += [rows[0], rows[len(rows) // 2], rows[-1]]
    for e in np.argsort(load)[:10]:                       # the least loaded experts (a few rows each)
        if load[e]:
            picked.append(np.nonzero((ids0 == e).any(axis=1))[0][0])
    picked += [0, tokens // 2 - 1, tokens - 1]
    return np.unique(np.array(picked))


def check_zipf_chunk(product, oracle, cfg, weights, layer, x, label, extra_rows=()):
    """One chunk through a resident layer: every token's expert ids and route weights against the oracle's routing,
    the outputs of picked rows against the oracle's forward (the oracle works token by token, so a subset of rows
    is a valid check).  Returns the row-tile count of the chunk's grouped products."""
    tokens = len(x)
    print(f"{label}: device forward of {tokens} tokens", flush=True)
    _, y, ids, w = layer.forward(x)
    reroutes = layer.serial_order_reroutes()
    print(f"{label}: oracle routes of all {tokens} tokens", flush=True)
    ids0, w0 = oracle_routes(oracle, cfg, weights, x)
    np.testing.assert_array_equal(ids, ids0, err_msg=f"expert ids of the {tokens}-token chunk")
    np.testing.assert_allclose(w, w0, atol=2e-6, rtol=2e-5)
    load = np.bincount(ids0.reshape(-1), minlength=cfg.experts)
    tiles = int(((load + 31) // 32).sum()) + (tokens + 31) // 32       # the experts' 32-row tiles and the shared expert's
    picked = np.unique(np.concatenate([pick_chunk_rows(ids0, load, tokens), np.array(extra_rows, dtype=np.int64)]))
    assert len(picked) >= 24
    print(f"{label}: oracle forward of {len(picked)} rows; max load {load.max()}, idle experts {(load == 0).sum()}, "
          f"{tiles} row tiles, serial-order reroutes {reroutes}", flush=True)
    with pf.MoeLayer(oracle, cfg, weights, len(picked)) as cpu:
        _, y0, ids1, w1 = cpu.forward(x[picked])
    np.testing.assert_array_equal(ids1, ids0[picked])       # the oracle's forward routes like its route call
    worst = assert_parity(y[picked], ids[picked], w[picked], y0, ids1, w1, label=f"{label} rows")
    print(f"{label}: max abs err {worst:.3e} on {len(picked)} rows", flush=True)
    return tiles, load


@pytest.mark.parametrize("tokens", [1024, 1777, 2048])
def test_q4k_zipf_chunk_at_full_shape(product, oracle, tokens):
    """The prefill chunk of the benchmark (1024 tokens), the stack's chunk (2048 tokens) and a ragged length
    between them, Q4_K experts under the Zipf(1.1) router."""
    cfg = workloads.measured_config()
    weights = pf.LayerWeights.synthetic(cfg, abi.GGUF_Q4_K, seed=1)
    workloads.zipf_router(weights, seed=1, temperature=0.18)
    x = workloads.prefill_chunk(weights, tokens, seed=tokens // 1024)
    with pf.MoeLayer(product, cfg, weights, tokens) as layer:
        assert product.hip.moe_kernel_family(*layer.device_handles(), tokens) == 2, "the prefill kernels do not cover this layer"
        tiles, load = check_zipf_chunk(product, oracle, cfg, weights, layer, x, f"zipf chunk {tokens}",
                                       extra_rows=(31, 32, tokens - 33, tokens - 32))
    assert load.max() > 96 and (load == 0).sum() < 64, (load.max(), (load == 0).sum())   # several 32-row tiles; most experts active
    if tokens != 1024:
        # the grouped products deal their row tiles to the XCDs in groups of 64: a count that is no multiple of 64
        # has a last, partly filled group
        assert tiles % 64 != 0, tiles


def test_q4k_verify_batches_share_experts(product, oracle):
    cfg = workloads.measured_config()
    weights = pf.LayerWeights.synthetic(cfg, abi.GGUF_Q4_K, seed=1)
    xs, info = workloads.verify_batches(weights, 4, seed=3)
    print(f"verify batches: {info}", flush=True)
    assert 0.3 <= info["mean_adjacent_overlap"] <= 0.7 and info["mean_unique_experts"] < 36
    with pf.MoeLayer(product, cfg, weights, 4) as gpu, pf.MoeLayer(oracle, cfg, weights, 4) as cpu:
        assert product.hip.moe_kernel_family(*gpu.device_handles(), 4) == 1
        for b, x in enumerate(xs):
            _, y, ids, w = gpu.forward(x)
            _, y0, ids0, w0 = cpu.forward(x)
            shared = len(set(ids0[0]) & set(ids0[1]))
            worst = assert_parity(y, ids, w, y0, ids0, w0, label=f"verify batch {b}")
            print(f"  batch {b}: {len(set(ids0.reshape(-1)))} unique experts, tokens 0/1 share {shared}, max abs err {worst:.2e}", flush=True)


def test_stack_of_independent_layers(product, oracle):
    """Four resident Q4_K layers driven like the 48-layer benchmark: one captured sequence of forwards,
    forward i through layer i % 4 with its own seeded input; every layer's last output against the oracle."""
    from bench import Tools
    tools, hip = Tools(), product.hip
    cfg = workloads.measured_config()
    n_layers, rounds = 4, 2
    layers, all_weights = [], []
    for l in range(n_layers):
        weights = pf.LayerWeights.synthetic(cfg, abi.GGUF_Q4_K, seed=1000 + l)
        workloads.zipf_router(weights, seed=1000 + l, temperature=0.18)
        layers.append(pf.MoeLayer(product, cfg, weights, 4))
        all_weights.append(weights)
    h = cfg.hidden_size
    x = pf.rms_normalise(pf.Synth().normal((rounds * n_layers, h), 79))
    x[:, 0] = 1.0                                             # the Zipf bias input
    moes = [l.device_handles()[0] for l in layers]
    works = [l.device_handles()[1] for l in layers]
    d_x = hip.to_device(x)
    d_y = hip.to_device(np.full((n_layers, h), -99.0, dtype=np.float32))
    plan = tools.plan_moe(moes, works, d_x, len(x), d_y, n_layers, 1, rounds * n_layers, h)
    tools.run(plan, 2)
    tools.destroy(plan)
    y = hip.from_device(d_y, (n_layers, h), np.float32)
    for l in (0, n_layers - 1):                               # forward i = layer i % 4; the last round's input stays
        token = x[(rounds - 1) * n_layers + l][None, :]
        ids = hip.from_device(hip.work_ids(works[l]), (1, cfg.top_k), np.uint32)
        w = hip.from_device(hip.work_route_weights(works[l]), (1, cfg.top_k), np.float32)
        assert int(hip.from_device(hip.work_error_word(works[l]), (1,), np.uint32)[0]) == 0
        with pf.MoeLayer(oracle, cfg, all_weights[l], 1) as cpu:
            _, y0, ids0, w0 = cpu.forward(token)
        worst = assert_parity(y[l][None, :], ids, w, y0, ids0, w0, label=f"stack layer {l}")
        print(f"  layer {l}: max abs err {worst:.2e}", flush=True)
    hip.free(d_x)
    hip.free(d_y)
    # the stack's other leg: a 2048-token chunk through the first and the last layer, each under its own router
    for l in (0, n_layers - 1):
        chunk = workloads.prefill_chunk(all_weights[l], 2048, seed=50 + l)
        with pf.MoeLayer(product, cfg, all_weights[l], 2048) as wide:
            assert product.hip.moe_kernel_family(*wide.device_handles(), 2048) == 2
            check_zipf_chunk(product, oracle, cfg, all_weights[l], wide, chunk, f"stack layer {l}, chunk")
    for l in layers:
        l.close()


def test_views_over_released_weight_bytes(product, oracle):
    """qwen4_moe_forward refuses views that overlap the bytes the layer was created from (the
    reference's rule); after pf_moe_forget_host_weights the addresses are free for reuse."""
    cfg = abi.moe_config(512, 32, 6, 256, 256)
    weights = pf.LayerWeights.synthetic(cfg, abi.GGUF_Q4_K, seed=8)
    x = pf.rms_normalise(pf.Synth().normal((2, 512), 12))
    with pf.MoeLayer(oracle, cfg, weights, 2) as cpu:
        _, y0, ids0, w0 = cpu.forward(x)
    with pf.MoeLayer(product, cfg, weights, 2) as layer:
        router = weights.raw[0].view(np.float32)                     # the layer's own router bytes, 64 KB
        inside = router[:2 * 512].reshape(2, 512)
        y = np.full((2, 512), -99.0, dtype=np.float32)
        err = abi.Qwen4Error()
        st = product.forward(layer.handle, abi.f32_view(inside), abi.f32_view(y), None, layer.work, C.byref(err))
        assert st == abi.QW4_INVALID_ARGUMENT and (y == -99).all()
        product.forget_host_weights(layer.handle)
        inside[:] = x                                                # the bytes now belong to the caller again
        st = product.forward(layer.handle, abi.f32_view(inside), abi.f32_view(y), None, layer.work, C.byref(err))
        assert st == abi.QW4_OK, err.detail
        err_abs = np.abs(y - y0)
        assert (err_abs <= ATOL + RTOL * np.abs(y0)).all()


@pytest.mark.parametrize("gtype", [abi.GGUF_Q4_K, abi.GGUF_IQ2_XXS])
@pytest.mark.parametrize("tokens", [8, 13, 16, 17, 32])
def test_batches_between_decode_and_prefill_match_oracle(product, oracle, gtype, tokens):
    """5 to 32 rows at the measured shape (a long verify batch, a short prompt): more rows than the decode kernels
    take, few enough that nearly every routed expert sees one row.  Every row against the CPU path."""
    cfg = workloads.measured_config()
    weights, x = make_layer_inputs(cfg, gtype, tokens, seed=40 + tokens)
    print(f"full shape, {tokens} rows, type={gtype}", flush=True)
    want = forward_with(oracle, cfg, weights, x)
    y, ids, w = forward_with(product, cfg, weights, x)
    assert_parity(y, ids, w, *want, label=f"{tokens} rows")
