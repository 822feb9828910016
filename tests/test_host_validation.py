"""Host logic of the shipped library without a GPU: every check that the reference makes before
it touches data (tests/test_qwen4_moe.c:64-86,146-171,234-287; tests/test_qwen4_packed.c) must give
the reference's code, leave the outputs untouched and never need a device.  Checks that read the
data itself (nonfinite logits, ids out of range) run on the device and are covered by the GPU tests."""
import ctypes as C

import numpy as np

import picoforge_amd as pf
import pytest
from picoforge_amd import abi

from hc_cases import call_add, call_read, error_cases, hc_shape, random_case, run_error_case


def _f32(buf, rows, cols, pitch):
    v = abi.Qwen4F32(buf.ctypes.data, buf.nbytes, 2)
    v.dim[:] = (rows, cols, 1, 1)
    v.stride_bytes[:] = (pitch, 4, 0, 0)
    return v


def test_route_argument_errors_match_the_oracle(product_host, oracle):
    product = product_host
    for case in (0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 12, 13):
        codes = []
        for api in (oracle, product):
            z = np.zeros(64, dtype=np.float32)
            p = np.full(64, -99, dtype=np.float32)
            w = np.full(64, -99, dtype=np.float32)
            ids = np.full(64, 0xFFFFFFFF, dtype=np.uint32)
            cfg = abi.moe_config(8, 4, 2, 5, 3)
            logits, probs, weights = _f32(z, 2, 4, 28), _f32(p, 2, 4, 32), _f32(w, 2, 2, 16)
            idv = abi.Qwen4U32Mut(ids.ctypes.data, ids.nbytes, 2, 2, 20)
            if case == 0: logits.data = None
            if case == 1: logits.rank = 1
            if case == 2: probs.stride_bytes[1] = 8
            if case == 3: weights.capacity_bytes = 23
            if case == 4: idv.row_stride_bytes = 7
            if case == 5: cfg.top_k = 5
            if case == 6: idv.cols = 3
            if case == 7: probs.capacity_bytes = 47
            if case == 8: probs.data = z.ctypes.data + 4
            if case == 9: weights.data = p.ctypes.data
            if case == 12: logits.dim[0] = 2 ** 64 - 1
            if case == 13: probs.data = z.ctypes.data
            err = abi.Qwen4Error()
            st = api.route(C.byref(cfg), logits, abi.Qwen4MoeRoutes(idv, weights), probs, C.byref(err))
            assert st == err.code != abi.QW4_OK, case
            assert (p == -99).all() and (w == -99).all() and (ids == 0xFFFFFFFF).all(), case
            codes.append((st, bytes(err.subject)))
        assert codes[0] == codes[1], (case, codes)


def test_group_argument_errors_match_the_oracle(product_host, oracle):
    product = product_host
    fill = np.iinfo(np.uint64).max
    for case in (2, 3, 4, 5, 6, 7, 8):
        codes = []
        for api in (oracle, product):
            buf = np.zeros(16, dtype=np.uint64)
            ids = buf.view(np.uint32)[:9]
            ids[:] = [2, 0, 99, 1, 2, 99, 2, 0, 99]
            off, cur = np.full(6, fill, dtype=np.uint64), np.full(5, fill, dtype=np.uint64)
            p2r, r2p = np.full(7, fill, dtype=np.uint64), np.full(7, fill, dtype=np.uint64)
            cfg = abi.moe_config(8, 4, 2, 5, 3)
            v = abi.Qwen4U32Mut(ids.ctypes.data, 36, 3, 2, 12)
            g = abi.QW4MoeGrouping(off.ctypes.data, 48, cur.ctypes.data, 40, p2r.ctypes.data, r2p.ctypes.data, 56, 56)
            if case == 2: g.row_to_pair_capacity_bytes = 6 * 8 - 1
            if case == 3: g.pair_to_row = g.row_to_pair
            if case == 4: g.offsets = None
            if case == 5: v.row_stride_bytes = 7
            if case == 6: v.rows = 2 ** 64 - 1
            if case == 7: v.cols = 1
            if case == 8: g.offsets = ids.ctypes.data
            err = abi.Qwen4Error()
            st = api.group_pairs(C.byref(cfg), v, g, C.byref(err))
            assert st == err.code != abi.QW4_OK, case
            assert (off == fill).all() and (cur == fill).all() and (p2r == fill).all() and (r2p == fill).all(), case
            codes.append(st)
        assert codes[0] == codes[1], (case, codes)


def test_create_validation_precedes_the_device(product_host, oracle):
    """Shape, capacity and format errors of the eight tensors come from the host checks, in the
    reference's order; only a valid layer reaches the device (and fails there without one)."""
    product = product_host
    cfg = abi.moe_config(8, 4, 2, 5, 3)
    raw = np.zeros(512, dtype=np.float32).view(np.uint8)
    for api in (oracle, product):
        err = abi.Qwen4Error()
        handle = C.c_void_p()
        bad = pf.LayerWeights(cfg, [raw] * 8, [abi.GGUF_F32] * 8)
        bad.struct.down.layout.k_logical = 4
        assert api.create(C.byref(cfg), C.byref(bad.struct), C.byref(handle), C.byref(err)) == abi.QW4_SHAPE
        assert not handle
        bad.struct.down.layout.k_logical = 5
        bad.struct.up.span.bytes = bad.struct.up.layout.tensor_bytes - 1
        assert api.create(C.byref(cfg), C.byref(bad.struct), C.byref(handle), C.byref(err)) == abi.QW4_CAPACITY
        bad.struct.up.span.bytes = raw.size
        bad.struct.gate.layout.row_bytes += 1
        assert api.create(C.byref(cfg), C.byref(bad.struct), C.byref(handle), C.byref(err)) == abi.QW4_FORMAT
        assert api.create(None, C.byref(bad.struct), C.byref(handle), C.byref(err)) == abi.QW4_INVALID_ARGUMENT
        assert api.create(C.byref(cfg), C.byref(bad.struct), None, C.byref(err)) == abi.QW4_INVALID_ARGUMENT
    good = pf.LayerWeights(cfg, [raw] * 8, [abi.GGUF_F32] * 8)
    err = abi.Qwen4Error()
    handle = C.c_void_p()
    st = product.create(C.byref(cfg), C.byref(good.struct), C.byref(handle), C.byref(err))
    if product.hip.device_count() < 1:
        assert st == abi.QW4_GPU_ERROR and not handle       # no silent CPU path
    else:
        assert st == abi.QW4_OK
        product.destroy(handle)


def test_null_handles_give_the_oracle_codes(product_host, oracle):
    seen = []
    for api in (oracle, product_host):
        err = abi.Qwen4Error()
        size = C.c_size_t(7)
        work = C.c_void_p()
        codes = [api.work_size(None, 4, C.byref(size), C.byref(err)),
                 api.work_create(None, 4, 1 << 20, C.byref(work), C.byref(err)),
                 api.work_reset(None, C.byref(err))]
        assert all(c != abi.QW4_OK for c in codes) and not work
        api.work_destroy(None)
        api.destroy(None)
        seen.append(codes)
    assert seen[0] == seen[1]


# ---- hyper-connection read and add: every check made before the data is read ---------------------
HC_PREFLIGHT = [c for c in error_cases() if c[2] != abi.QW4_NONFINITE or "eps" in c[0]]


@pytest.mark.parametrize("op", ["read", "add"])
@pytest.mark.parametrize("case", HC_PREFLIGHT, ids=lambda c: c[0])
def test_hc_argument_errors_match_the_oracle(product_host, oracle, op, case):
    _, mutate, status = case
    st_o, out_o, err_o = run_error_case(oracle, op, mutate)
    st_p, out_p, err_p = run_error_case(product_host, op, mutate)
    assert st_p == st_o == status
    assert (bytes(err_p.subject), bytes(err_p.detail)) == (bytes(err_o.subject), bytes(err_o.detail))
    np.testing.assert_array_equal(out_p.view(np.uint32), out_o.view(np.uint32))   # untouched


def test_hc_alias_and_empty_batches_need_no_device(product_host, oracle):
    for api in (oracle, product_host):
        normed, logits, block, inject = random_case(2, 4, 64, 21)
        err = abi.Qwen4Error()
        inside = normed[:, 0, :]
        st = api.hc.read(C.byref(hc_shape(4, 64)), abi.f32_cube(normed), abi.f32_cube(logits),
                         abi.f32_view(inside, pitch_bytes=normed.strides[0], capacity=normed.nbytes), C.byref(err))
        assert st == abi.QW4_INVALID_ARGUMENT and b"alias" in err.detail
        st = api.hc.add(C.byref(hc_shape(4, 64)), abi.f32_cube(normed),
                        abi.f32_view(normed[:, 1, :], pitch_bytes=normed.strides[0], capacity=normed.nbytes),
                        abi.f32_view(inject), C.byref(err))
        assert st == abi.QW4_INVALID_ARGUMENT and b"alias" in err.detail
        assert api.hc.read(None, abi.f32_cube(normed), abi.f32_cube(logits), abi.f32_view(block), None) == \
            abi.QW4_INVALID_ARGUMENT
        empty3 = np.zeros((0, 4, 64), dtype=np.float32)
        empty2 = np.zeros((0, 64), dtype=np.float32)
        assert call_read(api, empty3, empty3, empty2)[0] == abi.QW4_OK
        assert call_add(api, empty3, empty2, np.zeros((0, 4), dtype=np.float32))[0] == abi.QW4_OK
