"""The forward's observer (src/qwen4_moe.c:305-382, stages of src/qwen4_moe_internal.h:9-12): with an
observer set the shipped library runs the block as the reference's sequence of operators, so every
stage it reports — which stage, expert and microbatch, and the rows going in and out — must equal the
CPU path's bit for bit, and so must the block's output."""
import numpy as np
import pytest

import picoforge_amd as pf
from picoforge_amd import abi
from helpers import make_layer_inputs

pytestmark = pytest.mark.gpu


def traces(api, cfg, weights, x, cap):
    seen = []
    with pf.MoeLayer(api, cfg, weights, cap) as layer:
        layer.observe(seen)
        _, y, ids, w = layer.forward(x)
        layer.observe(None)
        _, y_fast, ids_fast, _ = layer.forward(x)
    return seen, y, ids, w, y_fast, ids_fast


@pytest.mark.parametrize("gtype,tokens,cap", [(abi.GGUF_Q4_K, 5, 5), (abi.GGUF_IQ2_XXS, 3, 8), (abi.GGUF_Q8_0, 37, 40)])
def test_every_stage_matches_the_cpu_path(product, oracle, gtype, tokens, cap):
    cfg = abi.moe_config(256, 12, 3, 256, 256)
    weights, x = make_layer_inputs(cfg, gtype, tokens, seed=31)
    got, y, ids, w, y_fast, ids_fast = traces(product, cfg, weights, x, cap)
    want, y_ref, ids_ref, w_ref, _, _ = traces(oracle, cfg, weights, x, cap)
    assert [(s, e, t, a.shape, b.shape) for s, e, t, a, b in got] == [(s, e, t, a.shape, b.shape) for s, e, t, a, b in want]
    stages = {s for s, *_ in got}
    assert stages == set(range(13))
    if tokens > 32:   # two microbatches, the second starting at token 32
        assert {t for _, _, t, _, _ in got} == {0, 32}
    for (s, e, t, a, b), (_, _, _, a_ref, b_ref) in zip(got, want):
        assert np.array_equal(a, a_ref), f"stage {s} expert {e} microbatch {t}: input rows differ"
        assert np.array_equal(b, b_ref), f"stage {s} expert {e} microbatch {t}: output rows differ"
    assert np.array_equal(y, y_ref) and np.array_equal(ids, ids_ref) and np.array_equal(w, w_ref)
    # the unobserved forward of the same layer: the throughput kernels, within the path's tolerance
    assert np.array_equal(ids_fast, ids_ref)
    np.testing.assert_allclose(y_fast, y_ref, atol=1e-3, rtol=1e-4)


def test_observer_needs_the_host_weight_bytes(product):
    cfg = abi.moe_config(256, 8, 2, 256, 256)
    weights, x = make_layer_inputs(cfg, abi.GGUF_Q4_K, 2, seed=5)
    with pf.MoeLayer(product, cfg, weights, 2) as layer:
        product.forget_host_weights(layer.handle)
        layer.observe([])
        st, *_ = layer.forward(x, check=False)
        assert st == abi.QW4_BAD_STATE


def test_route_log_records_every_forward_of_every_layer(product, tmp_path, monkeypatch):
    """PF_ROUTE_LOG (the per-layer part of the reference's QW4_ROUTE_LOG, src/qwen4_forward_gpu.m:62-65,894-900):
    records of uint32 pos, count, layers = 1, top_k and the ids, in one new file per layer."""
    prefix = tmp_path / "route"
    monkeypatch.setenv("PF_ROUTE_LOG", str(prefix))
    cfg = abi.moe_config(256, 16, 4, 256, 256)
    expected = {}
    for n, (gtype, seed) in enumerate([(abi.GGUF_Q4_K, 3), (abi.GGUF_IQ2_XXS, 4)]):
        weights, x = make_layer_inputs(cfg, gtype, 7, seed=seed)
        with pf.MoeLayer(product, cfg, weights, 8) as layer:
            _, _, ids_a, _ = layer.forward(x[:1])
            _, _, ids_b, _ = layer.forward(x[1:5], want_routes=False)   # logged although the caller asked for no routes
            _, _, ids_c, _ = layer.forward(x[1:5])
            _, _, ids_d, _ = layer.forward(x[5:])
            assert (ids_b == 0xFFFFFFFF).all()
            expected[n] = [(0, ids_a), (1, ids_c), (5, ids_c), (9, ids_d)]
    monkeypatch.delenv("PF_ROUTE_LOG")
    files = sorted(tmp_path.iterdir())
    assert len(files) == 2
    for path, n in zip(files, sorted(expected)):
        data = np.fromfile(path, dtype="<u4")
        at = 0
        for pos, ids in expected[n]:
            head = data[at:at + 4]
            assert list(head) == [pos, ids.shape[0], 1, cfg.top_k]
            at += 4
            assert np.array_equal(data[at:at + ids.size].reshape(ids.shape), ids)
            at += ids.size
        assert at == data.size
    # the file must be new: a layer created under a prefix whose next file exists is refused
    suffix = int(files[-1].suffix[1:]) + 1
    (tmp_path / f"route.{suffix}").write_bytes(b"")
    monkeypatch.setenv("PF_ROUTE_LOG", str(prefix))
    weights, _ = make_layer_inputs(cfg, abi.GGUF_Q4_K, 1, seed=3)
    with pytest.raises(pf.MoeError) as refused:
        pf.MoeLayer(product, cfg, weights, 1)
    assert refused.value.status == abi.QW4_IO
