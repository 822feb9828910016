"""ctypes mirror of the C boundary (include/qwen4_types.h, qwen4_packed.h, qwen4_moe.h, qwen4_hc.h).

The same structures serve the shipped library, the CPU oracle and a build of the
reference, since all three use the reference's layouts (src/qwen4_types.h,
src/qwen4_packed.h:6-11, src/qwen4_moe.h:7-11).
"""
import ctypes as C

import numpy as np

STATUS = ["OK", "INVALID_ARGUMENT", "MISSING", "TYPE", "RANGE", "SHAPE", "STRIDE", "FORMAT",
          "UNSUPPORTED", "OVERFLOW", "CAPACITY", "OOM", "OWNER", "BUSY", "STALE", "BAD_STATE",
          "NONFINITE", "IO", "EOF", "CANCELLED", "GPU_ERROR"]
globals().update({"QW4_" + name: value for value, name in enumerate(STATUS)})

GGUF_F32, GGUF_F16, GGUF_Q8_0, GGUF_Q2_K, GGUF_Q4_K, GGUF_IQ2_XXS, GGUF_BF16, GGUF_MXFP4 = 0, 1, 8, 10, 12, 16, 30, 39
# (elements per block, bytes per block), src/gguf.c:12-16
BLOCK = {GGUF_F32: (1, 4), GGUF_F16: (1, 2), GGUF_Q8_0: (32, 34), GGUF_Q2_K: (256, 84), GGUF_Q4_K: (256, 144),
         GGUF_IQ2_XXS: (256, 66), GGUF_BF16: (1, 2), GGUF_MXFP4: (32, 17)}
FORMAT_NAME = {0: "F32", 1: "F16", 8: "Q8_0", 10: "Q2_K", 12: "Q4_K", 16: "IQ2_XXS", 30: "BF16", 39: "MXFP4"}


class Qwen4Error(C.Structure):
    _fields_ = [("code", C.c_int), ("os_errno", C.c_int), ("file_offset", C.c_uint64),
                ("row", C.c_uint64), ("requested_bytes", C.c_size_t),
                ("completed_bytes", C.c_size_t), ("subject", C.c_char * 128),
                ("detail", C.c_char * 256)]


class Qwen4CpuSpan(C.Structure):
    _fields_ = [("data", C.c_void_p), ("bytes", C.c_size_t)]


class Qwen4F32(C.Structure):
    _fields_ = [("data", C.c_void_p), ("capacity_bytes", C.c_size_t), ("rank", C.c_size_t),
                ("dim", C.c_size_t * 4), ("stride_bytes", C.c_size_t * 4)]


Qwen4F32Mut = Qwen4F32  # identical layout; constness is not visible through the ABI


class Qwen4U32Mut(C.Structure):
    _fields_ = [("data", C.c_void_p), ("capacity_bytes", C.c_size_t), ("rows", C.c_size_t),
                ("cols", C.c_size_t), ("row_stride_bytes", C.c_size_t)]


class Qwen4MoeConfig(C.Structure):
    _fields_ = [("hidden_size", C.c_uint32), ("experts", C.c_uint32), ("top_k", C.c_uint32),
                ("intermediate", C.c_uint32), ("shared_intermediate", C.c_uint32),
                ("down_physical", C.c_uint32), ("norm_topk_prob", C.c_bool),
                ("trunk_type", C.c_uint32 * 3)]


class Qwen4HcShape(C.Structure):   # src/qwen4_types.h:69
    _fields_ = [("streams", C.c_size_t), ("hidden_size", C.c_size_t), ("low_rank", C.c_size_t),
                ("rms_eps", C.c_float)]


class GgufTensor(C.Structure):
    _fields_ = [("name", C.c_char * 128), ("type", C.c_uint32), ("rank", C.c_uint32),
                ("shape", C.c_size_t * 4), ("file_offset", C.c_size_t), ("bytes", C.c_size_t)]


class QW4PackedLayout(C.Structure):
    _fields_ = [("gguf_type", C.c_uint32), ("k_storage", C.c_size_t), ("k_logical", C.c_size_t),
                ("n_out", C.c_size_t), ("n_experts", C.c_size_t), ("row_bytes", C.c_size_t),
                ("expert_bytes", C.c_size_t), ("tensor_bytes", C.c_size_t)]


class QW4PackedCpuView(C.Structure):
    _fields_ = [("span", Qwen4CpuSpan), ("layout", QW4PackedLayout)]


class Qwen4MoeWeights(C.Structure):
    _fields_ = [(name, QW4PackedCpuView) for name in
                ("router", "gate", "up", "down", "shared_gate", "shared_up", "shared_down",
                 "shared_router")]


class Qwen4MoeRoutes(C.Structure):
    _fields_ = [("ids", Qwen4U32Mut), ("weights", Qwen4F32Mut)]


class QW4MoeGrouping(C.Structure):
    _fields_ = [("offsets", C.c_void_p), ("offsets_capacity_bytes", C.c_size_t),
                ("cursors", C.c_void_p), ("cursors_capacity_bytes", C.c_size_t),
                ("pair_to_row", C.c_void_p), ("row_to_pair", C.c_void_p),
                ("pair_to_row_capacity_bytes", C.c_size_t),
                ("row_to_pair_capacity_bytes", C.c_size_t)]


class QW4ExpertLayer(C.Structure):   # include/qwen4_expert_pool.h
    _fields_ = [("offset", C.c_uint64 * 3)]


class QW4PoolStats(C.Structure):
    _fields_ = [("hits", C.c_uint64), ("misses", C.c_uint64), ("evictions", C.c_uint64), ("bytes_read", C.c_uint64),
                ("acquire_ns", C.c_uint64)]


OBSERVER = C.CFUNCTYPE(None, C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, Qwen4F32, Qwen4F32)


def moe_config(hidden, experts, top_k, inter, shared_inter, down_physical=None, norm=True,
               trunk=(0, 0, 0)):
    c = Qwen4MoeConfig(hidden, experts, top_k, inter, shared_inter,
                       inter if down_physical is None else down_physical, bool(norm))
    c.trunk_type[:] = trunk
    return c


def f32_view(array, rows=None, cols=None, pitch_bytes=None, capacity=None):
    """View of a 2-D float32 numpy array (the array may be wider than cols: padding)."""
    assert array.dtype == np.float32 and array.ndim == 2 and (array.size == 0 or array.strides[1] == 4)
    v = Qwen4F32()
    v.data = array.ctypes.data if array.size else None
    rows = array.shape[0] if rows is None else rows
    cols = array.shape[1] if cols is None else cols
    v.rank = 2
    v.dim[:] = (rows, cols, 1, 1)
    pitch = array.strides[0] if pitch_bytes is None else pitch_bytes
    if array.shape[0] == 0 or pitch == 0:
        pitch = array.shape[1] * 4
    v.stride_bytes[:] = (pitch, 4, 0, 0)
    v.capacity_bytes = (array.shape[0] * pitch) if capacity is None else capacity
    return v


def f32_cube(array, dims=None):
    """View of a 3-D float32 numpy array [tokens, streams, hidden]; token and stream axes may be
    pitched (a slice of a larger array), the last axis is contiguous.  dims overrides the
    dimensions the view declares."""
    assert array.dtype == np.float32 and array.ndim == 3 and (array.size == 0 or array.strides[2] == 4)
    v = Qwen4F32()
    v.data = array.ctypes.data if array.size else None
    v.rank = 3
    d = tuple(array.shape) if dims is None else tuple(dims)
    v.dim[:] = d + (1,)
    s1 = array.strides[1] if array.shape[1] > 1 and array.size else d[2] * 4
    s0 = array.strides[0] if array.shape[0] > 1 and array.size else max(d[1], 1) * s1
    v.stride_bytes[:] = (s0, s1, 4, 0)
    v.capacity_bytes = 0 if not array.size else (array.shape[0] - 1) * s0 + (array.shape[1] - 1) * s1 + \
        array.shape[2] * 4
    return v


def u32_view(array, rows=None, cols=None):
    assert array.dtype == np.uint32 and array.ndim == 2 and (array.size == 0 or array.strides[1] == 4)
    v = Qwen4U32Mut()
    v.data = array.ctypes.data if array.size else None
    v.rows = array.shape[0] if rows is None else rows
    v.cols = array.shape[1] if cols is None else cols
    pitch = array.strides[0] if array.shape[0] and array.strides[0] else array.shape[1] * 4
    v.row_stride_bytes = pitch
    v.capacity_bytes = array.shape[0] * pitch
    return v


def packed_layout(gguf_type, k_storage, n_out, n_experts, k_logical=None):
    """Layout arithmetic of qw4_packed_layout_init (src/qwen4_packed.c:8-33), host-side."""
    block, size = BLOCK[gguf_type]
    assert k_storage % block == 0
    l = QW4PackedLayout()
    l.gguf_type = gguf_type
    l.k_storage = k_storage
    l.k_logical = k_storage if k_logical is None else k_logical
    l.n_out = n_out
    l.n_experts = n_experts
    l.row_bytes = k_storage // block * size
    l.expert_bytes = l.row_bytes * n_out
    l.tensor_bytes = l.expert_bytes * n_experts
    return l


def packed_view(raw, gguf_type, k_storage, n_out, n_experts, k_logical=None):
    """QW4PackedCpuView over a uint8 numpy buffer holding the whole tensor."""
    assert raw.dtype == np.uint8 and raw.flags["C_CONTIGUOUS"]
    v = QW4PackedCpuView()
    v.layout = packed_layout(gguf_type, k_storage, n_out, n_experts, k_logical)
    assert raw.size >= v.layout.tensor_bytes, (raw.size, v.layout.tensor_bytes)
    v.span.data = raw.ctypes.data
    v.span.bytes = raw.size
    return v


def status_name(code):
    return STATUS[code] if 0 <= code < len(STATUS) else "status %d" % code
