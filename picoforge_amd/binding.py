"""Loading and typing of the C-ABI libraries.

`load_product()` opens picoforge_amd/libpicoforge_moe.so, the shipped library:
the C11 host side with the entry points of the reference's src/qwen4_moe.h plus
the HIP shim of include/pf_moe_hip.h.  It raises if the library is missing; no
part of this package computes anything on the CPU in its place.

`MoeApi` types the eight entry points (and the two tested private helpers) of a
library that follows the reference's boundary; the prefixes are parameters so
that test code can type other libraries with the same boundary the same way.
"""
import ctypes as C
from pathlib import Path

import numpy as np

from . import abi

PACKAGE_DIR = Path(__file__).resolve().parent
REPO_DIR = PACKAGE_DIR.parent
PRODUCT_LIB = PACKAGE_DIR / "libpicoforge_moe.so"
SYNTH_LIB = PACKAGE_DIR / "libpf_synth.so"


class LibraryMissing(RuntimeError):
    pass


def _open(path):
    if not Path(path).exists():
        raise LibraryMissing(f"{path} is not built: run python -c 'import __graft_entry__ as g; g.build()' "
                             "or make -C picoforge_amd/csrc")
    return C.CDLL(str(path), mode=C.RTLD_LOCAL)


class MoeApi:
    """Typed view of one library exporting the reference's MoE boundary."""

    def __init__(self, lib, moe_prefix="qwen4_moe_", private_prefix="qw4_moe_", packed_prefix="qw4_packed_"):
        self.lib = lib
        P, E = C.POINTER, abi.Qwen4Error
        vp, sz = C.c_void_p, C.c_size_t

        def bind(name, restype, *argtypes):
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = list(argtypes)
            return fn

        m = moe_prefix
        self.create = bind(m + "create", C.c_int, P(abi.Qwen4MoeConfig), P(abi.Qwen4MoeWeights), P(vp), P(E))
        self.destroy = bind(m + "destroy", None, vp)
        self.work_size = bind(m + "work_size", C.c_int, vp, sz, P(sz), P(E))
        self.work_create = bind(m + "work_create", C.c_int, vp, sz, sz, P(vp), P(E))
        self.work_reset = bind(m + "work_reset", C.c_int, vp, P(E))
        self.work_destroy = bind(m + "work_destroy", None, vp)
        self.route = bind(m + "route", C.c_int, P(abi.Qwen4MoeConfig), abi.Qwen4F32, abi.Qwen4MoeRoutes,
                          abi.Qwen4F32Mut, P(E))
        self.forward = bind(m + "forward", C.c_int, vp, abi.Qwen4F32, abi.Qwen4F32Mut, P(abi.Qwen4MoeRoutes), vp,
                            P(E))
        self.group_pairs = bind(private_prefix + "group_pairs", C.c_int, P(abi.Qwen4MoeConfig), abi.Qwen4U32Mut,
                                abi.QW4MoeGrouping, P(E))
        self.observe = bind(private_prefix + "observe", None, vp, abi.OBSERVER, vp)
        if hasattr(lib, "pf_moe_forget_host_weights"):
            self.forget_host_weights = bind("pf_moe_forget_host_weights", None, vp)
        if hasattr(lib, "pf_moe_device_layer"):
            self.device_layer = bind("pf_moe_device_layer", vp, vp)
            self.device_work = bind("pf_moe_device_work", vp, vp)
        if hasattr(lib, "pf_moe_create_streamed"):   # expert streaming (include/qwen4_expert_pool.h, include/qwen4_moe.h)
            u32 = C.c_uint32
            self.create_streamed = bind("pf_moe_create_streamed", C.c_int, P(abi.Qwen4MoeConfig), P(abi.Qwen4MoeWeights),
                                        P(vp), P(E))
            self.forward_streamed = bind("pf_moe_forward_streamed", C.c_int, vp, vp, u32, abi.Qwen4F32, abi.Qwen4F32Mut,
                                         P(abi.Qwen4MoeRoutes), vp, P(E))
            self.pool_create = bind("qw4_pool_create", vp, C.c_int, P(abi.QW4ExpertLayer), u32, u32, P(sz), u32)
            self.pool_destroy = bind("qw4_pool_destroy", None, vp)
            self.pool_acquire = bind("qw4_pool_acquire", C.c_int, vp, u32, P(u32), sz, P(u32))
            self.pool_release = bind("qw4_pool_release", None, vp, P(u32), sz)
            self.pool_set_readers = bind("qw4_pool_set_readers", None, vp, u32)
            self.pool_region = bind("qw4_pool_region", vp, vp, C.c_int, P(sz))
            self.pool_stats = bind("qw4_pool_stats", abi.QW4PoolStats, vp)
            self.pool_set_formats = bind("pf_pool_set_formats", C.c_int, vp, P(u32), P(sz), P(sz))
            self.pool_slots = bind("pf_pool_slots", u32, vp)
            self.pool_format = bind("pf_pool_format", u32, vp, C.c_int)
        self.layout_init = bind(packed_prefix + "layout_init", C.c_int, P(abi.GgufTensor), sz,
                                P(abi.QW4PackedLayout), P(E))
        self.decode_row = bind(packed_prefix + "decode_row", C.c_int, P(abi.QW4PackedCpuView), sz, sz, vp, sz, P(E))
        self.matmul = bind(packed_prefix + "matmul", C.c_int, P(abi.QW4PackedCpuView), sz, abi.Qwen4F32,
                           abi.Qwen4F32Mut, P(E))


class HcApi:
    """The hyper-connection read and add either side of the block (include/qwen4_hc.h,
    src/qwen4_ops.h:43-48) and, where the library has it, the chained read -> MoE -> add."""

    def __init__(self, lib, prefix="qwen4_hc_"):
        P, E, vp = C.POINTER, abi.Qwen4Error, C.c_void_p
        S, V = P(abi.Qwen4HcShape), abi.Qwen4F32
        self.read = getattr(lib, prefix + "read")
        self.read.restype, self.read.argtypes = C.c_int, [S, V, V, V, P(E)]
        self.add = getattr(lib, prefix + "add")
        self.add.restype, self.add.argtypes = C.c_int, [S, V, V, V, P(E)]
        if hasattr(lib, "pf_moe_forward_hc"):
            self.forward_hc = lib.pf_moe_forward_hc
            self.forward_hc.restype = C.c_int
            self.forward_hc.argtypes = [vp, S, V, V, V, V, P(abi.Qwen4MoeRoutes), vp, P(E)]


def load_product():
    lib = _open(PRODUCT_LIB)
    api = MoeApi(lib)
    api.hip = HipShim(lib)
    api.hc = HcApi(lib)
    return api


class HipShim:
    """include/pf_moe_hip.h"""

    def __init__(self, lib):
        P, vp, sz, u32p = C.POINTER, C.c_void_p, C.c_size_t, C.POINTER(C.c_uint32)

        def bind(name, restype, *argtypes):
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = list(argtypes)
            setattr(self, name.replace("pf_hip_", ""), fn)

        bind("pf_hip_device_count", C.c_int)
        bind("pf_hip_last_error", C.c_char_p)
        bind("pf_hip_moe_create", C.c_int, P(PfHipMoeDesc), P(vp), P(sz), P(vp))
        bind("pf_hip_moe_destroy", None, vp)
        bind("pf_hip_moe_bytes", sz, vp)
        bind("pf_hip_work_bytes", sz, P(PfHipMoeDesc), sz)
        bind("pf_hip_work_create", C.c_int, vp, sz, P(vp))
        bind("pf_hip_work_destroy", None, vp)
        bind("pf_hip_moe_forward_device", C.c_int, vp, vp, vp, sz, vp, sz, sz, vp)
        bind("pf_hip_moe_forward_static", C.c_int, vp, vp, sz, vp, sz, vp, vp, vp, sz, vp)
        bind("pf_hip_work_ids", vp, vp)
        bind("pf_hip_work_route_weights", vp, vp)
        bind("pf_hip_work_logits", vp, vp)
        bind("pf_hip_work_error_word", vp, vp)
        bind("pf_hip_work_exact_rows", C.c_int, vp, u32p)
        bind("pf_hip_work_full_reroutes", C.c_int, vp, u32p)
        bind("pf_hip_work_clear_status", C.c_int, vp)
        bind("pf_hip_work_force_general", None, vp, C.c_int)
        bind("pf_hip_work_limit_kernels", None, vp, C.c_int)
        bind("pf_hip_work_check_guards", C.c_int, vp, P(C.c_int), P(C.c_int))
        bind("pf_hip_moe_forward_host", C.c_int, vp, vp, vp, sz, vp, sz, vp, sz, vp, sz, sz, u32p)
        bind("pf_hip_route_host", C.c_int, vp, sz, sz, sz, C.c_int, vp, vp, vp, u32p, P(C.c_uint64))
        bind("pf_hip_group_pairs_host", C.c_int, vp, sz, sz, sz, vp, vp, vp, u32p, P(C.c_int))
        bind("pf_hip_packed_matmul_host", C.c_int, C.c_uint32, vp, sz, sz, sz, vp, sz, vp, u32p)
        bind("pf_hip_packed_decode_row_host", C.c_int, C.c_uint32, vp, sz, sz, vp, u32p)
        bind("pf_hip_malloc", C.c_int, P(vp), sz)
        bind("pf_hip_free", None, vp)
        bind("pf_hip_memcpy_h2d", C.c_int, vp, vp, sz)
        bind("pf_hip_memcpy_d2h", C.c_int, vp, vp, sz)
        bind("pf_hip_synchronize", C.c_int)
        bind("pf_hip_moe_kernel_family", C.c_int, vp, vp, sz)
        bind("pf_hip_moe_decode_launches", C.c_int, vp, vp, sz)
        bind("pf_hip_hc_read_device", C.c_int, vp, sz, sz, vp, sz, sz, vp, sz, sz, sz, sz, vp, vp)
        bind("pf_hip_hc_add_device", C.c_int, vp, sz, sz, vp, sz, vp, sz, sz, sz, sz, vp, vp)
        bind("pf_hip_moe_forward_hc_device", C.c_int, vp, vp, vp, sz, sz, vp, sz, sz, vp, sz, sz, vp, sz, sz, vp)
        bind("pf_hip_hc_read_host", C.c_int, vp, sz, sz, vp, sz, sz, vp, sz, sz, sz, sz, u32p)
        bind("pf_hip_hc_add_host", C.c_int, vp, sz, sz, vp, sz, vp, sz, sz, sz, sz, u32p)

    def check(self, rc, what):
        if rc != 0:
            raise RuntimeError(f"{what}: shim status {rc}: {self.last_error().decode()}")

    def to_device(self, array):
        array = np.ascontiguousarray(array)
        ptr = C.c_void_p()
        self.check(self.malloc(C.byref(ptr), array.nbytes), "malloc")
        if array.nbytes:
            self.check(self.memcpy_h2d(ptr, array.ctypes.data, array.nbytes), "h2d")
        return ptr

    def from_device(self, ptr, shape, dtype):
        out = np.empty(shape, dtype=dtype)
        if out.nbytes:
            self.check(self.memcpy_d2h(out.ctypes.data, ptr, out.nbytes), "d2h")
        return out


class PfHipMoeDesc(C.Structure):
    _fields_ = [("hidden", C.c_uint32), ("experts", C.c_uint32), ("top_k", C.c_uint32), ("inter", C.c_uint32),
                ("shared_inter", C.c_uint32), ("down_physical", C.c_uint32), ("norm_topk", C.c_uint32),
                ("type", C.c_uint32 * 8)]


class Synth:
    """picoforge_amd/csrc/pf_synth.c"""

    def __init__(self):
        lib = _open(SYNTH_LIB)
        vp, sz = C.c_void_p, C.c_size_t
        lib.pf_synth_normal_f32.argtypes = [vp, sz, C.c_uint64, C.c_float, C.c_float]
        lib.pf_synth_q4k_quantize.argtypes = [vp, sz, vp]
        lib.pf_synth_q4k_normal.argtypes = [vp, sz, C.c_uint64, C.c_float]
        lib.pf_synth_iq2xxs_uniform.argtypes = [vp, sz, C.c_uint64, C.c_float]
        for name in ("pf_synth_q8_0_normal", "pf_synth_q2k_normal", "pf_synth_mxfp4_normal"):
            getattr(lib, name).argtypes = [vp, sz, C.c_uint64, C.c_float]
        for fn in (lib.pf_synth_normal_f32, lib.pf_synth_q4k_quantize, lib.pf_synth_q4k_normal,
                   lib.pf_synth_iq2xxs_uniform, lib.pf_synth_q8_0_normal, lib.pf_synth_q2k_normal,
                   lib.pf_synth_mxfp4_normal):
            fn.restype = None
        self.lib = lib

    def normal(self, shape, seed, std=1.0, mean=0.0):
        out = np.empty(shape, dtype=np.float32)
        self.lib.pf_synth_normal_f32(out.ctypes.data, out.size, seed, mean, std)
        return out

    def q4k_normal(self, blocks, seed, std):
        out = np.empty(blocks * 144, dtype=np.uint8)
        self.lib.pf_synth_q4k_normal(out.ctypes.data, blocks, seed, std)
        return out

    def q4k_quantize(self, values):
        values = np.ascontiguousarray(values, dtype=np.float32)
        assert values.size % 256 == 0
        out = np.empty(values.size // 256 * 144, dtype=np.uint8)
        self.lib.pf_synth_q4k_quantize(values.ctypes.data, values.size // 256, out.ctypes.data)
        return out

    def quantised_normal(self, gtype, elements, seed, std):
        """N(0, std) weights quantised to Q8_0, Q2_K or MXFP4 blocks."""
        name, (block, size) = {abi.GGUF_Q8_0: "q8_0", abi.GGUF_Q2_K: "q2k", abi.GGUF_MXFP4: "mxfp4"}[gtype], abi.BLOCK[gtype]
        assert elements % block == 0
        out = np.empty(elements // block * size, dtype=np.uint8)
        getattr(self.lib, f"pf_synth_{name}_normal")(out.ctypes.data, elements // block, seed, std)
        return out

    def iq2xxs_uniform(self, blocks, seed, d_base=2.0 ** -12):
        out = np.empty(blocks * 66, dtype=np.uint8)
        self.lib.pf_synth_iq2xxs_uniform(out.ctypes.data, blocks, seed, d_base)
        return out
