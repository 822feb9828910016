"""Pins of the CPU oracle's hyper-connection read and add (oracle/orc_hc.c).

Independent of the oracle's own formulas: the known-answer vectors of the
reference's C test (tests/test_qwen4_recurrent.c:107-121), closed forms
(zero and saturated gates, zero and unit injection), a float32 numpy evaluation
that rounds once per operation, the tolerance of the reference's own Python test
against a float64 evaluation (tests/test_qwen4_recurrent.py:648-649: 2e-5
absolute) and, where it was built, the reference's compiled C path bit for bit,
statuses and partial results included.
"""
import ctypes as C

import numpy as np
import pytest

from picoforge_amd import abi

from hc_cases import SHAPES, call_add, call_read, error_cases, hc_shape, pitched, random_case, run_error_case


def test_known_answers_of_the_reference_c_test(oracle):
    normed = np.array([[[1, 2, 3], [10, 20, 30]]], dtype=np.float32)
    logits = np.zeros_like(normed)
    st, mixed, _ = call_read(oracle, normed, logits)
    assert st == abi.QW4_OK
    np.testing.assert_array_equal(mixed, [[2.75, 5.5, 8.25]])
    st, _ = call_add(oracle, normed, np.array([[3, -2, 1]], dtype=np.float32), np.ones((1, 2), dtype=np.float32))
    assert st == abi.QW4_OK
    np.testing.assert_array_equal(normed.ravel(), [4, 0, 4, 13, 18, 31])


@pytest.mark.parametrize("t,h,w", SHAPES)
def test_read_closed_forms(oracle, t, h, w):
    normed, _, _, _ = random_case(t, h, w, 11)
    # gate 0 -> every weight exactly 0.5; gate +40 -> exactly 1 (1 + e^-40 rounds to 1); gate -110 -> exactly 0
    for gate, weight in ((0.0, np.float32(0.5)), (40.0, np.float32(1.0)), (-110.0, np.float32(0.0))):
        st, mixed, _ = call_read(oracle, normed, np.full_like(normed, gate))
        assert st == abi.QW4_OK
        expect = np.zeros((t, w), dtype=np.float32)
        for s in range(h):   # float32 numpy: one rounding per product and per sum, streams ascending
            expect = expect + normed[:, s, :] * weight
        np.testing.assert_array_equal(mixed, expect / np.float32(h))


@pytest.mark.parametrize("t,h,w", SHAPES)
def test_read_within_the_reference_tests_tolerance_of_float64(oracle, t, h, w):
    normed, logits, _, _ = random_case(t, h, w, 12, scale=4.0)
    st, mixed, _ = call_read(oracle, normed, logits)
    assert st == abi.QW4_OK
    gate = 1.0 / (1.0 + np.exp(-logits.astype(np.float64)))
    expect = (normed.astype(np.float64) * gate).sum(axis=1) / h
    np.testing.assert_allclose(mixed, expect, atol=2e-5, rtol=0)
    # and a float32 evaluation with the sigmoid rounded from float64: expf is within an ulp of that,
    # so each term is within a few ulps
    term = normed * gate.astype(np.float32)
    acc = np.zeros((t, w), dtype=np.float32)
    for s in range(h):
        acc = acc + term[:, s, :]
    np.testing.assert_allclose(mixed, acc / np.float32(h), atol=4e-7 * h * max(1.0, float(np.abs(normed).max(initial=0))), rtol=0)


@pytest.mark.parametrize("t,h,w", SHAPES)
def test_add_is_one_rounded_product_and_one_rounded_sum(oracle, t, h, w):
    normed, _, block, inject = random_case(t, h, w, 13)
    residual = normed.copy()
    st, _ = call_add(oracle, residual, block, inject)
    assert st == abi.QW4_OK
    product = inject[:, :, None] * block[:, None, :]     # float32, rounded
    np.testing.assert_array_equal(residual, normed + product)
    # zero injection leaves the residual alone; unit injection of a zero block too
    residual = normed.copy()
    assert call_add(oracle, residual, block, np.zeros_like(inject))[0] == abi.QW4_OK
    np.testing.assert_array_equal(residual, normed)


@pytest.mark.parametrize("t,h,w", [(3, 4, 64), (7, 3, 33)])
def test_pitched_views_touch_only_their_elements(oracle, t, h, w):
    normed, logits, block, inject = random_case(t, h, w, 14)
    _, want, _ = call_read(oracle, normed, logits)
    big_n, view_n = pitched(normed, 1, 3)
    big_g, view_g = pitched(logits, 2, 5)
    mixed = np.full((t, w + 9), -99.0, dtype=np.float32)
    st, _, _ = call_read(oracle, normed, logits, mixed,
                         views=(abi.f32_cube(view_n), abi.f32_cube(view_g), abi.f32_view(mixed, cols=w)))
    assert st == abi.QW4_OK
    np.testing.assert_array_equal(mixed[:, :w], want)
    assert (mixed[:, w:] == -99.0).all()
    dense = normed.copy()
    call_add(oracle, dense, block, inject)
    big_r, view_r = pitched(normed, 2, 7)
    st, _ = call_add(oracle, view_r, block, inject, views=(abi.f32_cube(view_r), abi.f32_view(block), abi.f32_view(inject)))
    assert st == abi.QW4_OK
    np.testing.assert_array_equal(view_r, dense)
    assert (big_r[:, h:, :] == -77.0).all() and (big_r[:, :, w:] == -77.0).all()


@pytest.mark.parametrize("op", ["read", "add"])
@pytest.mark.parametrize("case", error_cases(), ids=lambda c: c[0])
def test_preflight_errors_leave_the_output_alone(oracle, reference, op, case):
    _, mutate, status = case
    st, out, err = run_error_case(oracle, op, mutate)
    assert st == status and err.code == status, (abi.status_name(st), err.detail)
    if op == "read":
        assert (out == -99.0).all()
    if reference is not None:
        st_ref, out_ref, err_ref = run_error_case(reference, op, mutate)
        assert st_ref == st and err_ref.detail == err.detail
        np.testing.assert_array_equal(out.view(np.uint32), out_ref.view(np.uint32))


@pytest.mark.parametrize("op", ["read", "add"])
def test_aliases_and_null_shape_are_refused(oracle, reference, op):
    for api in filter(None, (oracle, reference)):
        normed, logits, block, inject = random_case(2, 4, 64, 16)
        err = abi.Qwen4Error()
        if op == "read":
            inside = normed[:, 0, :]            # the output inside an input
            st = api.hc.read(C.byref(hc_shape(4, 64)), abi.f32_cube(normed), abi.f32_cube(logits),
                             abi.f32_view(inside, pitch_bytes=normed.strides[0], capacity=normed.nbytes), C.byref(err))
            assert st == abi.QW4_INVALID_ARGUMENT and b"alias" in err.detail
            assert api.hc.read(None, abi.f32_cube(normed), abi.f32_cube(logits), abi.f32_view(block), None) == \
                abi.QW4_INVALID_ARGUMENT
        else:
            inside = normed[:, 1, :]
            st = api.hc.add(C.byref(hc_shape(4, 64)), abi.f32_cube(normed),
                            abi.f32_view(inside, pitch_bytes=normed.strides[0], capacity=normed.nbytes),
                            abi.f32_view(inject), C.byref(err))
            assert st == abi.QW4_INVALID_ARGUMENT and b"alias" in err.detail
            assert api.hc.add(None, abi.f32_cube(normed), abi.f32_view(block), abi.f32_view(inject), None) == \
                abi.QW4_INVALID_ARGUMENT


def test_overflow_stops_the_call_where_the_reference_stops(oracle, reference):
    big = np.float32(3e38)
    for api in filter(None, (oracle, reference)):
        normed = np.full((2, 4, 8), 1.0, dtype=np.float32)
        normed[1, :, 3] = big                       # the sum of four overflows at token 1, column 3
        st, mixed, err = call_read(api, normed, np.full_like(normed, 40.0))
        assert st == abi.QW4_NONFINITE and b"HC read overflow" in err.detail
        assert (mixed[0] == 1.0).all() and (mixed[1, :3] == 1.0).all() and (mixed[1, 3:] == -99.0).all()
        residual = np.full((2, 4, 8), 1.0, dtype=np.float32)
        residual[1, 2, 5] = big
        block = np.full((2, 8), big, dtype=np.float32)
        block[0] = 1.0
        st, err = call_add(api, residual, block, np.ones((2, 4), dtype=np.float32))
        assert st == abi.QW4_NONFINITE and b"HC residual overflow" in err.detail
        assert (residual[0] == 2.0).all() and (residual[1, :2] == big).all() and (residual[1, 2, :5] == big).all()
        assert residual[1, 2, 5] == big and (residual[1, 2, 6:] == 1.0).all() and (residual[1, 3] == 1.0).all()


@pytest.mark.parametrize("t,h,w", SHAPES)
@pytest.mark.parametrize("scale", [1.0, 30.0])
def test_bit_identical_to_the_compiled_reference(oracle, reference, t, h, w, scale):
    if reference is None:
        pytest.skip("oracle/_ref was not built (reference tree not mounted at build time)")
    normed, logits, block, inject = random_case(t, h, w, 17, scale=scale)
    if t:
        logits.ravel()[:4] = (0.0, -0.0, 89.0, -104.0)   # the exp branches (tests/test_qwen4_fast_kernels.py:2742)
    st_o, mixed_o, _ = call_read(oracle, normed, logits)
    st_r, mixed_r, _ = call_read(reference, normed, logits)
    assert st_o == st_r == abi.QW4_OK
    np.testing.assert_array_equal(mixed_o.view(np.uint32), mixed_r.view(np.uint32))
    res_o, res_r = normed.copy(), normed.copy()
    assert call_add(oracle, res_o, block, inject)[0] == call_add(reference, res_r, block, inject)[0] == abi.QW4_OK
    np.testing.assert_array_equal(res_o.view(np.uint32), res_r.view(np.uint32))
