"""GGUF checkpoints as the source of a layer's MoE weights (include/pf_gguf.h).

`GgufFile` wraps the library's reader: what gguf_open, the MoE part of
qwen4_config_load and the MoE rows of the weight catalog do in the reference
(src/gguf.c:31-105, src/qwen4_config.c:152-216, src/qwen4_weights.c:91-99).  The
parsing runs in the library's C code; this file only declares the entry points.

    with GgufFile(api, path) as f:
        model = f.moe_model()
        with f.moe_layer(3, token_cap=4) as layer:       # uploads layer 3's eight tensors
            status, y, ids, weights = layer.forward(x)
"""
import ctypes as C
import os

import numpy as np

from . import abi
from .layer import ROLE, MoeError, MoeLayer


class PfGgufMoeModel(C.Structure):
    _fields_ = [("blocks", C.c_uint32), ("trunk_blocks", C.c_uint32), ("mtp_blocks", C.c_uint32),
                ("moe", abi.Qwen4MoeConfig), ("hc", abi.Qwen4HcShape), ("semantic_profile", C.c_char_p)]


class GgufApi:
    """The pf_gguf_* entry points of one library."""

    def __init__(self, lib):
        vp, E, P = C.c_void_p, abi.Qwen4Error, C.POINTER

        def bind(name, restype, *argtypes):
            fn = getattr(lib, "pf_gguf_" + name)
            fn.restype, fn.argtypes = restype, list(argtypes)
            return fn
        self.open = bind("open", C.c_int, C.c_char_p, P(vp), P(E))
        self.close = bind("close", None, vp)
        self.tensor_count = bind("tensor_count", C.c_size_t, vp)
        self.tensor = bind("tensor", P(abi.GgufTensor), vp, C.c_size_t)
        self.find = bind("find", P(abi.GgufTensor), vp, C.c_char_p)
        self.data_offset = bind("data_offset", C.c_size_t, vp)
        self.file_size = bind("file_size", C.c_size_t, vp)
        self.tensor_bytes = bind("tensor_bytes", vp, vp, P(abi.GgufTensor))
        self.moe_model = bind("moe_model", C.c_int, vp, P(PfGgufMoeModel), P(E))
        self.moe_layer_config = bind("moe_layer_config", C.c_int, P(PfGgufMoeModel), C.c_uint32,
                                     P(abi.Qwen4MoeConfig), P(E))
        self.moe_weights = bind("moe_weights", C.c_int, vp, P(PfGgufMoeModel), C.c_uint32,
                                P(abi.Qwen4MoeWeights), P(E))
        self.moe_create = bind("moe_create", C.c_int, vp, P(PfGgufMoeModel), C.c_uint32, P(vp), P(E))


class GgufError(MoeError):
    def __init__(self, status, err):
        super().__init__(status, f"{err.subject.decode(errors='replace')}: {err.detail.decode(errors='replace')}")
        self.subject, self.detail = err.subject.decode(errors="replace"), err.detail.decode(errors="replace")


class FileLayerWeights:
    """One layer's eight views into an open file; the shape MoeLayer expects of its weights argument."""

    def __init__(self, cfg, struct, owner):
        self.cfg, self.struct, self.owner = cfg, struct, owner   # owner: keeps the mapping alive

    @property
    def nbytes(self):
        return sum(getattr(self.struct, name).span.bytes for name, _ in self.struct._fields_)

    @property
    def types(self):
        return [getattr(self.struct, role).layout.gguf_type for role in ROLE]

    @property
    def raw(self):
        """The tensors' bytes as read-only arrays over the mapping, in Qwen4MoeWeights order (no copy)."""
        out = []
        for role in ROLE:
            span = getattr(self.struct, role).span
            array = np.ctypeslib.as_array((C.c_uint8 * span.bytes).from_address(span.data))
            array.flags.writeable = False
            out.append(array)
        return out


class GgufFile:
    def __init__(self, api, path):
        self.moe_api = api
        self.api = GgufApi(api.lib)
        self.handle, self.err = C.c_void_p(), abi.Qwen4Error()
        st = self.api.open(os.fsencode(path), C.byref(self.handle), C.byref(self.err))
        if st != abi.QW4_OK:
            raise GgufError(st, self.err)
        self._model = None

    def close(self):
        if self.handle:
            self.api.close(self.handle)
            self.handle = C.c_void_p()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()
        return False

    def __len__(self):
        return self.api.tensor_count(self.handle)

    @property
    def data_offset(self):
        return self.api.data_offset(self.handle)

    def tensors(self):
        """Descriptors in file order as dicts."""
        out = []
        for i in range(len(self)):
            t = self.api.tensor(self.handle, i).contents
            out.append(dict(name=t.name.decode(), type=t.type, shape=list(t.shape[:t.rank]),
                            file_offset=t.file_offset, bytes=t.bytes))
        return out

    def moe_model(self):
        if self._model is None:
            model = PfGgufMoeModel()
            st = self.api.moe_model(self.handle, C.byref(model), C.byref(self.err))
            if st != abi.QW4_OK:
                raise GgufError(st, self.err)
            self._model = model
        return self._model

    def layer_config(self, layer):
        cfg = abi.Qwen4MoeConfig()
        st = self.api.moe_layer_config(C.byref(self.moe_model()), layer, C.byref(cfg), C.byref(self.err))
        if st != abi.QW4_OK:
            raise GgufError(st, self.err)
        return cfg

    def moe_weights(self, layer):
        w = abi.Qwen4MoeWeights()
        st = self.api.moe_weights(self.handle, C.byref(self.moe_model()), layer, C.byref(w), C.byref(self.err))
        if st != abi.QW4_OK:
            raise GgufError(st, self.err)
        return FileLayerWeights(self.layer_config(layer), w, self)

    def moe_layer(self, layer, token_cap, api=None):
        """A MoeLayer on the file's tensors: created by pf_gguf_moe_create in the library that reads the
        file, or, with `api`, by another library's qwen4_moe_create from the same views."""
        weights = self.moe_weights(layer)
        if api is not None:
            return MoeLayer(api, weights.cfg, weights, token_cap)
        handle = C.c_void_p()
        st = self.api.moe_create(self.handle, C.byref(self.moe_model()), layer, C.byref(handle), C.byref(self.err))
        if st != abi.QW4_OK:
            raise GgufError(st, self.err)
        return MoeLayer(self.moe_api, weights.cfg, weights, token_cap, handle=handle)
