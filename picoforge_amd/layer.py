"""Host-side mirror of how the reference's forward loop uses the MoE block.

`LayerWeights` holds the eight tensors of one layer as GGUF bytes and the views
over them (the job of the reference's create_moe binds, src/qwen4_forward.c:174-187);
`MoeLayer` owns a Qwen4Moe handle and a workspace of one library and runs
qwen4_moe_forward like layer_cpu does (src/qwen4_forward.c:365).  The class is
agnostic of which library it drives: the shipped HIP one, the CPU oracle or a
build of the reference.
"""
import ctypes as C

import numpy as np

from . import abi
from .binding import Synth

ROLE = ("router", "gate", "up", "down", "shared_gate", "shared_up", "shared_down", "shared_router")


def shapes(cfg):
    """(k_storage, k_logical, n_out, experts) per tensor, in Qwen4MoeWeights order (src/qwen4_moe.c:56-57)."""
    h, i, s, e = cfg.hidden_size, cfg.intermediate, cfg.shared_intermediate, cfg.experts
    return [(h, h, e, 1), (h, h, i, e), (h, h, i, e), (cfg.down_physical, i, h, e),
            (h, h, s, 1), (h, h, s, 1), (s, s, h, 1), (h, h, 1, 1)]


class LayerWeights:
    def __init__(self, cfg, raw, types):
        self.cfg, self.raw, self.types = cfg, list(raw), list(types)
        self.struct = abi.Qwen4MoeWeights()
        for role, buf, gtype, (ks, kl, n, e) in zip(ROLE, self.raw, self.types, shapes(cfg)):
            setattr(self.struct, role, abi.packed_view(buf, gtype, ks, n, e, kl))

    @property
    def nbytes(self):
        return sum(b.size for b in self.raw)

    def without_routed_bytes(self):
        """The same views with the routed tensors' bytes withheld: what pf_moe_create_streamed takes for a layer whose
        routed experts stay in a file."""
        struct = abi.Qwen4MoeWeights()
        C.memmove(C.byref(struct), C.byref(self.struct), C.sizeof(struct))
        for role in ("gate", "up", "down"):
            view = getattr(struct, role)
            view.span.data, view.span.bytes = None, 0
        return struct

    # the two profiles of real checkpoints (src/qwen4_config.c:197-216, src/qwen4_weights.c:91-99):
    # routed gate/up, routed down, shared expert
    PROFILE = {"q2": (abi.GGUF_IQ2_XXS, abi.GGUF_Q2_K, abi.GGUF_Q8_0), "q4": (abi.GGUF_Q4_K, abi.GGUF_MXFP4, abi.GGUF_Q8_0)}

    @classmethod
    def synthetic(cls, cfg, expert_type, seed, std=0.02, shared_type=None, router_std=None, iq2_d=2.0 ** -12,
                  down_type=None):
        """Seeded weights: routers F32 N(0, router_std or std); expert tensors N(0, std) quantised to
        Q4_K, Q8_0, Q2_K or MXFP4, IQ2_XXS blocks drawn uniformly, or plain F32 / F16 / BF16.
        expert_type may name a checkpoint profile, "q2" or "q4"."""
        synth = Synth()
        if expert_type in cls.PROFILE:
            expert_type, down_type, shared_type = cls.PROFILE[expert_type]
        shared_type = expert_type if shared_type is None else shared_type
        down_type = expert_type if down_type is None else down_type
        types = [abi.GGUF_F32, expert_type, expert_type, down_type, shared_type, shared_type, shared_type,
                 abi.GGUF_F32]
        raw = []
        for j, (gtype, (ks, kl, n, e)) in enumerate(zip(types, shapes(cfg))):
            stream = seed * 16 + j + 1
            count = ks * n * e
            if gtype == abi.GGUF_F32:
                sd = (router_std or std) if j in (0, 7) else std
                raw.append(synth.normal((count,), stream, sd).view(np.uint8))
            elif gtype == abi.GGUF_Q4_K:
                raw.append(synth.q4k_normal(count // 256, stream, std))
            elif gtype == abi.GGUF_IQ2_XXS:
                raw.append(synth.iq2xxs_uniform(count // 256, stream, iq2_d))
            elif gtype in (abi.GGUF_Q8_0, abi.GGUF_Q2_K, abi.GGUF_MXFP4):
                raw.append(synth.quantised_normal(gtype, count, stream, std))
            elif gtype == abi.GGUF_F16:
                raw.append(synth.normal((count,), stream, std).astype(np.float16).view(np.uint8))
            elif gtype == abi.GGUF_BF16:
                raw.append((synth.normal((count,), stream, std).view(np.uint32) >> 16).astype(np.uint16).view(np.uint8))
            else:
                raise ValueError(gtype)
        return cls(cfg, raw, types)


class MoeError(RuntimeError):
    def __init__(self, status, detail):
        super().__init__(f"{abi.status_name(status)}: {detail}")
        self.status = status


class MoeLayer:
    def __init__(self, api, cfg, weights, token_cap, handle=None):
        """handle: a Qwen4Moe the library already created from these weights (the layer then owns it)."""
        self.api, self.cfg, self.weights, self.cap = api, cfg, weights, token_cap
        self.err = abi.Qwen4Error()
        self.handle, self.work = handle or C.c_void_p(), C.c_void_p()
        if handle is None:
            st = api.create(C.byref(cfg), C.byref(weights.struct), C.byref(self.handle), C.byref(self.err))
            self._raise(st)
        size = C.c_size_t()
        self._raise(api.work_size(self.handle, token_cap, C.byref(size), C.byref(self.err)))
        self.work_bytes = size.value
        self._raise(api.work_create(self.handle, token_cap, size.value, C.byref(self.work), C.byref(self.err)))

    def _raise(self, st):
        if st != abi.QW4_OK:
            raise MoeError(st, self.err.detail.decode(errors="replace"))

    def forward(self, x, want_routes=True, check=True):
        """x [T, H] float32 -> (status, y, ids, weights)."""
        x = np.ascontiguousarray(x, dtype=np.float32)
        t, k = x.shape[0], self.cfg.top_k
        y = np.full((t, self.cfg.hidden_size), -99.0, dtype=np.float32)
        ids = np.full((t, k), 0xFFFFFFFF, dtype=np.uint32)
        w = np.full((t, k), -99.0, dtype=np.float32)
        routes = abi.Qwen4MoeRoutes(abi.u32_view(ids), abi.f32_view(w))
        st = self.api.forward(self.handle, abi.f32_view(x), abi.f32_view(y),
                              C.byref(routes) if want_routes else None, self.work, C.byref(self.err))
        if check:
            self._raise(st)
        return st, y, ids, w

    def forward_hc(self, normed, logits, residual, inject, fused=None, check=True, low_rank=1, eps=1e-6):
        """The block between its two hyper-connection steps, as layer_cpu runs them
        (src/qwen4_forward.c:362-367): read [T, S, H] -> MoE -> add into residual [T, S, H] in place.
        fused=None uses the library's single call where it has one (the shipped library), the three
        calls otherwise (the CPU oracle, a build of the reference).  Returns (status, ids, weights)."""
        t, s, h = normed.shape
        k = self.cfg.top_k
        shape = abi.Qwen4HcShape(s, h, low_rank, eps)
        ids = np.full((t, k), 0xFFFFFFFF, dtype=np.uint32)
        w = np.full((t, k), -99.0, dtype=np.float32)
        routes = abi.Qwen4MoeRoutes(abi.u32_view(ids), abi.f32_view(w))
        hc = self.api.hc
        if fused is None:
            fused = hasattr(hc, "forward_hc")
        if fused:
            st = hc.forward_hc(self.handle, C.byref(shape), abi.f32_cube(normed), abi.f32_cube(logits),
                               abi.f32_cube(residual), abi.f32_view(inject), C.byref(routes), self.work,
                               C.byref(self.err))
        else:
            mixed = np.full((t, h), -99.0, dtype=np.float32)
            block = np.full((t, h), -99.0, dtype=np.float32)
            st = hc.read(C.byref(shape), abi.f32_cube(normed), abi.f32_cube(logits), abi.f32_view(mixed),
                         C.byref(self.err))
            if st == abi.QW4_OK:
                st = self.api.forward(self.handle, abi.f32_view(mixed), abi.f32_view(block), C.byref(routes),
                                      self.work, C.byref(self.err))
            if st == abi.QW4_OK:
                st = hc.add(C.byref(shape), abi.f32_cube(residual), abi.f32_view(block), abi.f32_view(inject),
                            C.byref(self.err))
        if check:
            self._raise(st)
        return st, ids, w

    def observe(self, record=None):
        """Set (record: a list to append to) or clear the forward's observer.  Each entry is
        (stage, expert, token, input rows, output rows) with the rows copied out during the callback;
        expert is -1 where the library reports SIZE_MAX."""
        def view(v):
            rows, cols, pitch = v.dim[0], v.dim[1], v.stride_bytes[0] // 4
            if not rows or not cols:
                return np.zeros((rows, cols), np.float32)
            flat = np.frombuffer((C.c_float * ((rows - 1) * pitch + cols)).from_address(v.data), dtype=np.float32)
            return np.stack([flat[r * pitch:r * pitch + cols].copy() for r in range(rows)])

        def callback(_ctx, stage, expert, token, a, b):
            record.append((stage, -1 if expert == C.c_size_t(-1).value else expert, token, view(a), view(b)))

        self._observer = abi.OBSERVER(callback) if record is not None else C.cast(None, abi.OBSERVER)
        self.api.observe(self.work, self._observer, None)

    def device_handles(self):
        """(PfHipMoe*, PfHipWork*) behind this layer: shipped library only."""
        return self.api.device_layer(self.handle), self.api.device_work(self.work)

    def force_general(self, on=True):
        """Route every batch size through the general kernels (tests of both kernel families)."""
        self.api.hip.work_force_general(self.api.device_work(self.work), 1 if on else 0)

    def serial_order_reroutes(self):
        count = C.c_uint32()
        self.api.hip.work_exact_rows(self.api.device_work(self.work), C.byref(count))
        return count.value

    def full_reroutes(self):
        """Of the re-routed tokens, those whose every logit was summed serially (see pf_hip_work_full_reroutes)."""
        count = C.c_uint32()
        self.api.hip.work_full_reroutes(self.api.device_work(self.work), C.byref(count))
        return count.value

    def reset(self):
        return self.api.work_reset(self.work, C.byref(self.err))

    def close(self):
        if self.work:
            self.api.work_destroy(self.work)
            self.work = C.c_void_p()
        if self.handle:
            self.api.destroy(self.handle)
            self.handle = C.c_void_p()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


def rms_normalise(x, eps=0.0):
    x = np.asarray(x, dtype=np.float32)
    scale = np.sqrt(np.mean(x.astype(np.float64) ** 2, axis=-1, keepdims=True) + eps)
    return (x / scale).astype(np.float32)
