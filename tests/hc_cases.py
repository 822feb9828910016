"""Inputs, call wrappers and preflight error cases shared by the tests of the hyper-connection
read and add: the same cases run against the CPU oracle, a build of the reference and the
shipped library."""
import ctypes as C

import numpy as np

from picoforge_amd import abi

# token, stream and hidden counts the reference tests (tests/test_qwen4_fast_kernels.py:2716,
# tests/test_qwen4_recurrent.py:638) plus a pitched case
SHAPES = [(1, 4, 2560), (3, 4, 2560), (7, 3, 33), (2, 1, 5), (5, 3, 7), (0, 4, 64)]


def hc_shape(streams, hidden, low_rank=5, eps=1e-6):
    return abi.Qwen4HcShape(streams, hidden, low_rank, eps)


def call_read(api, normed, logits, mixed=None, shape=None, views=None):
    t, h, w = normed.shape
    if mixed is None:
        mixed = np.full((t, w), -99.0, dtype=np.float32)
    shape = hc_shape(h, w) if shape is None else shape
    err = abi.Qwen4Error()
    n, g, m = views if views else (abi.f32_cube(normed), abi.f32_cube(logits), abi.f32_view(mixed))
    st = api.hc.read(C.byref(shape), n, g, m, C.byref(err))
    return st, mixed, err


def call_add(api, residual, block, inject, shape=None, views=None):
    t, h, w = residual.shape
    shape = hc_shape(h, w) if shape is None else shape
    err = abi.Qwen4Error()
    r, b, i = views if views else (abi.f32_cube(residual), abi.f32_view(block), abi.f32_view(inject))
    st = api.hc.add(C.byref(shape), r, b, i, C.byref(err))
    return st, err


def random_case(t, h, w, seed, scale=1.0):
    rng = np.random.default_rng(seed)
    normed = rng.standard_normal((t, h, w)).astype(np.float32)
    logits = (rng.standard_normal((t, h, w)) * scale).astype(np.float32)
    block = rng.standard_normal((t, w)).astype(np.float32)
    inject = rng.uniform(0.0, 2.0 / h, (t, h)).astype(np.float32)
    return normed, logits, block, inject


def pitched(array, pad_rows, pad_cols, fill=-77.0):
    """The same values as a slice of a larger array: token and stream axes pitched."""
    t, h, w = array.shape
    big = np.full((t, h + pad_rows, w + pad_cols), fill, dtype=np.float32)
    big[:, :h, :w] = array
    return big, big[:, :h, :w]


def error_cases():
    """(name, mutate(views, arrays, shape) -> None, expected status) for both operators."""
    def nan_at(which, index):
        def m(v, a, s):
            a[which][index] = np.nan
        return m

    def set_dim(which, axis, value):
        def m(v, a, s):
            v[which].dim[axis] = value
        return m

    def set_stride(which, axis, value):
        def m(v, a, s):
            v[which].stride_bytes[axis] = value
        return m

    def set_field(which, name, value):
        def m(v, a, s):
            setattr(v[which], name, value)
        return m

    def set_shape(name, value):
        def m(v, a, s):
            setattr(s, name, value)
        return m

    def as_matrix(v, a, s):
        v[0].rank = 2
        v[0].dim[:] = (8, 64, 1, 1)
        v[0].stride_bytes[:] = (256, 4, 0, 0)
    return [
        ("first input NaN", nan_at(0, (1, 2, 3)), abi.QW4_NONFINITE),
        ("second input Inf", lambda v, a, s: a[1].__setitem__((0,) * a[1].ndim, np.inf), abi.QW4_NONFINITE),
        ("wrong stream count", set_dim(0, 1, 3), abi.QW4_SHAPE),
        ("rank 2 over cube strides", set_field(0, "rank", 2), abi.QW4_STRIDE),
        ("valid view of the wrong rank", as_matrix, abi.QW4_SHAPE),
        ("feature stride", set_stride(0, 2, 8), abi.QW4_STRIDE),
        ("overlapping axes", set_stride(0, 0, 4), abi.QW4_STRIDE),
        ("capacity short", set_field(0, "capacity_bytes", 16), abi.QW4_CAPACITY),
        ("null data", set_field(0, "data", None), abi.QW4_INVALID_ARGUMENT),
        ("zero low rank", set_shape("low_rank", 0), abi.QW4_SHAPE),
        ("streams beyond uint32", set_shape("streams", 2 ** 32), abi.QW4_RANGE),
        ("eps zero", set_shape("rms_eps", 0.0), abi.QW4_RANGE),
        ("eps NaN", set_shape("rms_eps", float("nan")), abi.QW4_NONFINITE),
    ]


def run_error_case(api, op, mutate):
    normed, logits, block, inject = random_case(2, 4, 64, 15)
    shape = hc_shape(4, 64)
    if op == "read":
        mixed = np.full((2, 64), -99.0, dtype=np.float32)
        arrays = [normed, logits, mixed]
        views = [abi.f32_cube(normed), abi.f32_cube(logits), abi.f32_view(mixed)]
        mutate(views, arrays, shape)
        st, _, err = call_read(api, normed, logits, mixed, shape=shape, views=views)
        return st, mixed, err
    residual = normed.copy()
    arrays = [residual, block, inject]
    views = [abi.f32_cube(residual), abi.f32_view(block), abi.f32_view(inject)]
    mutate(views, arrays, shape)
    st, err = call_add(api, residual, block, inject, shape=shape, views=views)
    return st, residual, err
