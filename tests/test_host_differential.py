"""Property-based differential test of the preflight checks: randomly malformed views of the
hyper-connection operators and of qwen4_moe_route go to the CPU oracle, to the reference's compiled C
path (where it was built) and to the shipped library's host side.  All three must agree on what is
refused and with which status; what passes the checks reaches the kernels, which this test does not need
(without a device the shipped library then reports QW4_GPU_ERROR, with one it computes)."""
import ctypes as C

import numpy as np
from hypothesis import HealthCheck, event, given, settings
from hypothesis import strategies as st

from picoforge_amd import abi

PASSED = "passed the checks"
ARENA = np.zeros(1 << 16, dtype=np.float32)      # every generated view points into this buffer
ARENA[:] = np.linspace(-1.0, 1.0, ARENA.size, dtype=np.float32)


def outcome(status):
    return PASSED if status in (abi.QW4_OK, abi.QW4_NONFINITE, abi.QW4_GPU_ERROR) else abi.status_name(status)


@st.composite
def views(draw, rank_choices=(1, 2, 3, 4), base_dims=None):
    """A view descriptor that is right in most fields and wrong in a few."""
    rank = draw(st.sampled_from(rank_choices))
    dims = list(base_dims) if base_dims and draw(st.integers(0, 9)) else \
        [draw(st.sampled_from([0, 1, 2, 3, 5, 8, 2 ** 32 + 1])) for _ in range(4)]
    dims = (dims + [1, 1, 1, 1])[:4]
    strides = [0, 0, 0, 0]
    span = 4
    for axis in range(min(rank, 4) - 1, -1, -1):      # dense strides, then a few perturbed
        strides[axis] = span
        span *= max(dims[axis], 1) if dims[axis] < 2 ** 20 else 1
    for axis in range(4):
        kind = draw(st.integers(0, 19))
        if kind == 0:
            strides[axis] += draw(st.sampled_from([4, 8, 64]))      # pitched
        elif kind == 1:
            strides[axis] = draw(st.sampled_from([0, 2, 3, 4, 6]))  # overlapping or misaligned
    v = abi.Qwen4F32()
    offset = draw(st.sampled_from([0, 0, 0, 4, 64, 2, 4096]))
    v.data = None if draw(st.integers(0, 15)) == 0 else ARENA.ctypes.data + offset
    v.rank = rank
    v.dim[:] = dims
    v.stride_bytes[:] = strides
    v.capacity_bytes = draw(st.sampled_from([ARENA.nbytes - 65536] * 8 + [0, 4, 64, 1 << 14]))
    return v


def clone(v):
    c = abi.Qwen4F32()
    C.memmove(C.byref(c), C.byref(v), C.sizeof(v))
    return c


def mostly(value, *others, weight=8):
    return st.sampled_from([value] * weight + list(others))


shapes = st.builds(lambda s, h, r, eps: abi.Qwen4HcShape(s, h, r, eps), mostly(2, 0, 1, 3, 2 ** 32), mostly(5, 0, 1, 8),
                   mostly(1, 0, 5), mostly(1e-6, 0.0, -1.0, float("nan"), float("inf")))
CUBE, MATRIX = (3, 3, 3, 3, 3, 3, 1, 2, 4), (2, 2, 2, 2, 2, 2, 1, 3)


def apis(oracle, reference, product_host):
    return [a for a in (oracle, reference, product_host) if a is not None]


@settings(max_examples=400, deadline=None, suppress_health_check=[HealthCheck.function_scoped_fixture])
@given(shape=shapes, normed=views(CUBE, (2, 2, 5)), logits=views(CUBE, (2, 2, 5)), mixed=views(MATRIX, (2, 5)),
       null_shape=st.integers(0, 30))
def test_hc_read_preflight_agrees(oracle, reference, product_host, shape, normed, logits, mixed, null_shape):
    logits, mixed = clone(logits), clone(mixed)
    if logits.data and logits.data % 4096:      # most inputs in regions of their own; some share one
        logits.data += 16384
    if mixed.data:
        mixed.data += 32768 if mixed.data % 4096 == 0 else 0
    results = []
    for api in apis(oracle, reference, product_host):
        err = abi.Qwen4Error()
        st_ = api.hc.read(None if null_shape == 0 else C.byref(shape), clone(normed), clone(logits), clone(mixed), C.byref(err))
        results.append(outcome(st_))
    event(results[0])
    assert len(set(results)) == 1, results


@settings(max_examples=400, deadline=None, suppress_health_check=[HealthCheck.function_scoped_fixture])
@given(shape=shapes, residual=views(CUBE, (2, 2, 5)), block=views(MATRIX, (2, 5)), inject=views(MATRIX, (2, 2)))
def test_hc_add_preflight_agrees(oracle, reference, product_host, shape, residual, block, inject):
    block, inject = clone(block), clone(inject)
    if block.data and block.data % 4096 == 0:
        block.data += 16384
    if inject.data and inject.data % 4096 == 0:
        inject.data += 32768
    results = []
    saved = ARENA.copy()
    for api in apis(oracle, reference, product_host):
        err = abi.Qwen4Error()
        st_ = api.hc.add(C.byref(shape), clone(residual), clone(block), clone(inject), C.byref(err))
        results.append(outcome(st_))
        ARENA[:] = saved                      # the operator works in place when it passes the checks
    event(results[0])
    assert len(set(results)) == 1, results


@settings(max_examples=300, deadline=None, suppress_health_check=[HealthCheck.function_scoped_fixture])
@given(logits=views(MATRIX, (3, 8)), probs=views(MATRIX, (3, 8)), weights=views(MATRIX, (3, 2)), top_k=mostly(2, 0, 1, 8, 9),
       experts=mostly(8, 0, 1), ids_rows=mostly(3, 2), ids_cols=mostly(2, 3), ids_pitch=mostly(8, 12, 7, 4))
def test_route_preflight_agrees(oracle, reference, product_host, logits, probs, weights, top_k, experts, ids_rows, ids_cols,
                                ids_pitch):
    # separate regions of the arena, so that aliasing is only what the strategy puts in
    logits, probs, weights = clone(logits), clone(probs), clone(weights)
    if probs.data:
        probs.data += 16384
    if weights.data:
        weights.data += 32768
    ids = np.zeros(64, dtype=np.uint32)
    results = []
    saved = ARENA.copy()
    for api in apis(oracle, reference, product_host):
        cfg = abi.moe_config(8, experts, top_k, 5, 3)
        idv = abi.Qwen4U32Mut(ids.ctypes.data, ids.nbytes, ids_rows, ids_cols, ids_pitch)
        err = abi.Qwen4Error()
        st_ = api.route(C.byref(cfg), clone(logits), abi.Qwen4MoeRoutes(idv, clone(weights)), clone(probs), C.byref(err))
        results.append(outcome(st_))
        ARENA[:] = saved
    event(results[0])
    assert len(set(results)) == 1, results
