"""Expert streaming (include/qwen4_expert_pool.h, pf_moe_create_streamed / pf_moe_forward_streamed): the pool's
bookkeeping against a model of the reference's (src/qwen4_expert_pool.c: least recently used unpinned slot, slot 0
first, two-pass acquire, failure leaves nothing pinned), the bytes that arrive in the device regions, and a layer
whose routed experts stay in a file against the CPU path on the full weights."""
import ctypes as C
import os

import numpy as np
import pytest

import picoforge_amd as pf
from picoforge_amd import abi
from helpers import assert_parity, forward_with, make_layer_inputs

pytestmark = pytest.mark.gpu


class ModelPool:
    """The reference's bookkeeping in a few lines: recency list, pins, owner table."""

    def __init__(self, slots):
        self.order = list(range(slots))          # victims first: slot 0 is the first to go
        self.pins = [0] * slots
        self.owner = [None] * slots
        self.where = {}
        self.hits = self.misses = self.evictions = 0

    def acquire(self, layer, experts, n_experts):
        taken, new = [], []
        for e in experts:
            key = (layer, e)
            s = self.where.get(key) if e < n_experts else None
            if e >= n_experts or (s is None and all(self.pins[c] for c in self.order)):
                for t in taken:
                    self.pins[t] -= 1
                for t in new:
                    del self.where[self.owner[t]]
                    self.owner[t] = None
                return None
            if s is not None:
                self.hits += 1
            else:
                s = next(c for c in self.order if not self.pins[c])
                if self.owner[s] is not None:
                    del self.where[self.owner[s]]
                    self.evictions += 1
                self.owner[s] = key
                self.where[key] = s
                self.misses += 1
                new.append(s)
            self.pins[s] += 1
            self.order.remove(s)
            self.order.append(s)
            taken.append(s)
        return taken

    def release(self, slots):
        for s in slots:
            if self.pins[s]:
                self.pins[s] -= 1


def u32(values):
    return (C.c_uint32 * len(values))(*values)


def test_pool_bookkeeping_and_contents(product, tmp_path):
    rng = np.random.default_rng(5)
    layers, experts, slots, sizes = 2, 6, 4, (96, 64, 160)
    blob = rng.integers(0, 256, 4096 + layers * experts * sum(sizes), dtype=np.uint8)
    offsets, at = [], 4096
    for _ in range(layers):
        row = []
        for b in sizes:
            row.append(at)
            at += experts * b
        offsets.append(row)
    path = tmp_path / "experts.bin"
    blob.tofile(path)
    fd = os.open(path, os.O_RDONLY)
    table = (abi.QW4ExpertLayer * layers)(*[abi.QW4ExpertLayer((C.c_uint64 * 3)(*row)) for row in offsets])
    pool = product.pool_create(fd, table, layers, experts, (C.c_size_t * 3)(*sizes), slots)
    assert pool
    model = ModelPool(slots)
    script = [("acquire", 0, [1, 2]), ("release", None, None), ("acquire", 1, [1, 5, 1]), ("acquire", 0, [2, 3]),
              ("acquire", 0, [0]),               # every slot pinned: refused, nothing changes
              ("release", None, None), ("release", None, None),
              ("acquire", 0, [4, 9]),            # id out of range: refused after one slot was taken
              ("acquire", 1, [0, 1, 2, 3]), ("release", None, None), ("acquire", 0, [5, 4, 3, 2]), ("release", None, None)]
    held = []
    for step, layer, ids in script:
        if step == "release":
            got = held.pop(0)
            product.pool_release(pool, u32(got), len(got))
            model.release(got)
            continue
        out = u32([0xFFFFFFFF] * len(ids))
        rc = product.pool_acquire(pool, layer, u32(ids), len(ids), out)
        want = model.acquire(layer, ids, experts)
        assert (rc == 0) == (want is not None), (step, layer, ids)
        if want is None:
            continue
        assert list(out) == want, (layer, ids)
        held.append(want)
        for e, s in zip(ids, want):               # the slot holds the expert's three slices as the file stores them
            for m, b in enumerate(sizes):
                size = C.c_size_t()
                region = product.pool_region(pool, m, C.byref(size))
                assert size.value == slots * b
                got = product.hip.from_device(C.c_void_p(region + s * b), (b,), np.uint8)
                start = offsets[layer][m] + e * b
                assert np.array_equal(got, blob[start:start + b]), (layer, e, m)
    stats = product.pool_stats(pool)
    assert (stats.hits, stats.misses, stats.evictions) == (model.hits, model.misses, model.evictions)
    assert stats.bytes_read == model.misses * sum(sizes) and stats.acquire_ns > 0
    assert model.evictions > 0 and model.hits > 0
    product.pool_destroy(pool)
    os.close(fd)


def streamed_weights(weights):
    """The same views with the routed tensors' bytes withheld."""
    return weights.without_routed_bytes()


@pytest.mark.parametrize("gtype,formatted", [(abi.GGUF_Q4_K, False), (abi.GGUF_F16, False), (abi.GGUF_Q4_K, True),
                                             (abi.GGUF_IQ2_XXS, True), ("q2", True), ("q4", True)])
def test_streamed_layer_matches_the_cpu_path(product, oracle, tmp_path, gtype, formatted):
    """formatted: the pool is told the matrices' formats and keeps its slots in the device layout (needed where that
    differs from the file's: IQ2_XXS, Q8_0, MXFP4 -- both checkpoint profiles, "q2" and "q4")."""
    cfg = abi.moe_config(256, 16, 4, 256, 256)
    weights, x = make_layer_inputs(cfg, gtype, 9, seed=61)
    # the model file: two layers' worth of tensors, this layer second, at page-aligned offsets
    sizes = [weights.raw[j].size // cfg.experts for j in (1, 2, 3)]
    filler = np.zeros(8192, np.uint8)
    pieces, offsets, at = [filler], [], filler.size
    for layer in range(2):
        row = []
        for j in (1, 2, 3):
            data = weights.raw[j] if layer == 1 else np.full_like(weights.raw[j], 0x5A)
            row.append(at)
            pieces.append(data)
            at += data.size
        offsets.append(row)
    path = tmp_path / "model.bin"
    np.concatenate(pieces).tofile(path)
    fd = os.open(path, os.O_RDONLY)
    table = (abi.QW4ExpertLayer * 2)(*[abi.QW4ExpertLayer((C.c_uint64 * 3)(*row)) for row in offsets])
    pool = product.pool_create(fd, table, 2, cfg.experts, (C.c_size_t * 3)(*sizes), 12)   # 12 slots for 16 experts
    assert pool
    product.pool_set_readers(pool, 3)
    def tell_formats(which):
        h, i = cfg.hidden_size, cfg.intermediate
        assert product.pool_set_formats(which, (C.c_uint32 * 3)(*weights.types[1:4]), (C.c_size_t * 3)(h, h, cfg.down_physical),
                                        (C.c_size_t * 3)(i, i, h)) == 0

    if formatted:
        tell_formats(pool)
        assert product.pool_format(pool, 2) == weights.types[3] and product.pool_slots(pool) == 12
    err, handle = abi.Qwen4Error(), C.c_void_p()
    struct = streamed_weights(weights)
    assert product.create_streamed(C.byref(cfg), C.byref(struct), C.byref(handle), C.byref(err)) == abi.QW4_OK, err.detail
    want = forward_with(oracle, cfg, weights, x)
    with pf.MoeLayer(product, cfg, weights, 4, handle=handle) as layer:
        # the plain forward has no experts to read
        st, *_ = layer.forward(x[:1], check=False)
        assert st == abi.QW4_BAD_STATE
        for first, count in ((0, 3), (3, 3), (6, 2), (8, 1), (0, 3)):
            rows = np.ascontiguousarray(x[first:first + count])
            y = np.full((count, cfg.hidden_size), -99.0, np.float32)
            ids = np.full((count, cfg.top_k), 0xFFFFFFFF, np.uint32)
            w = np.full((count, cfg.top_k), -99.0, np.float32)
            routes = abi.Qwen4MoeRoutes(abi.u32_view(ids), abi.f32_view(w))
            st = product.forward_streamed(layer.handle, pool, 1, abi.f32_view(rows), abi.f32_view(y), C.byref(routes),
                                          layer.work, C.byref(layer.err))
            assert st == abi.QW4_OK, layer.err.detail
            assert_parity(y, ids, w, want[0][first:first + count], want[1][first:first + count],
                          want[2][first:first + count], label=f"streamed rows {first}..{first + count}")
        stats = product.pool_stats(pool)
        assert stats.misses >= 12 and stats.evictions > 0 and stats.hits > 0
        assert stats.bytes_read == stats.misses * sum(sizes)
        # a pool with fewer slots than one token routes to cannot make the batch resident
        tiny = product.pool_create(fd, table, 2, cfg.experts, (C.c_size_t * 3)(*sizes), cfg.top_k - 1)
        if formatted:
            tell_formats(tiny)
        rows = np.ascontiguousarray(x[:2])
        y = np.full((2, cfg.hidden_size), -99.0, np.float32)
        st = product.forward_streamed(layer.handle, tiny, 1, abi.f32_view(rows), abi.f32_view(y), None, layer.work,
                                      C.byref(layer.err))
        assert st == abi.QW4_IO and (y == -99.0).all()
        product.pool_destroy(tiny)
        assert product.work_reset(layer.work, C.byref(layer.err)) == abi.QW4_OK
        # the layer and the larger pool go on working
        y = np.full((3, cfg.hidden_size), -99.0, np.float32)
        rows = np.ascontiguousarray(x[3:6])
        st = product.forward_streamed(layer.handle, pool, 1, abi.f32_view(rows), abi.f32_view(y), None, layer.work,
                                      C.byref(layer.err))
        assert st == abi.QW4_OK
        np.testing.assert_allclose(y, want[0][3:6], atol=1e-3, rtol=1e-4)
    product.pool_destroy(pool)
    os.close(fd)


@pytest.mark.parametrize("expert_type", [abi.GGUF_Q4_K, "q4", abi.GGUF_IQ2_XXS, "q2"])
def test_streamed_layer_on_the_decode_kernels(product, oracle, tmp_path, expert_type):
    """A layer of a shape the decode kernels cover -- Q4_K throughout, IQ2_XXS throughout, or in a checkpoint profile (Q4_K
    gate and up with an MXFP4 down tensor, IQ2_XXS gate and up with a Q2_K one; the shared expert Q8_0) -- streamed
    through a pool that was told its formats: the Q4_K and IQ2_XXS slots are kept in the tile order and batches of up to
    16 tokens run the decode kernels on them (the router kernel and the routing in the first device call, the expert
    kernels on the pairs' slots in the second); longer batches run the general kernels on the same slots.  56 slots for
    64 experts: evictions on the way."""
    cfg = abi.moe_config(512, 64, 4, 256, 256)
    tokens = 40
    weights, x = make_layer_inputs(cfg, expert_type, tokens, seed=67)
    x[5] = x[4]                                              # two tokens of a batch share every expert
    sizes = [weights.raw[j].size // cfg.experts for j in (1, 2, 3)]
    filler = np.zeros(4096, np.uint8)
    pieces, offsets, at = [filler], [], filler.size
    for j in (1, 2, 3):
        offsets.append(at)
        pieces.append(weights.raw[j])
        at += weights.raw[j].size
    path = tmp_path / "model.bin"
    np.concatenate(pieces).tofile(path)
    fd = os.open(path, os.O_RDONLY)
    table = (abi.QW4ExpertLayer * 1)(abi.QW4ExpertLayer((C.c_uint64 * 3)(*offsets)))
    pool = product.pool_create(fd, table, 1, cfg.experts, (C.c_size_t * 3)(*sizes), 56)
    assert pool
    h, i = cfg.hidden_size, cfg.intermediate
    assert product.pool_set_formats(pool, (C.c_uint32 * 3)(*weights.types[1:4]), (C.c_size_t * 3)(h, h, cfg.down_physical),
                                    (C.c_size_t * 3)(i, i, h)) == 0
    err, handle = abi.Qwen4Error(), C.c_void_p()
    struct = streamed_weights(weights)
    assert product.create_streamed(C.byref(cfg), C.byref(struct), C.byref(handle), C.byref(err)) == abi.QW4_OK, err.detail
    want = forward_with(oracle, cfg, weights, x)
    with pf.MoeLayer(product, cfg, weights, tokens, handle=handle) as layer:
        moe, work = layer.device_handles()
        assert product.hip.moe_kernel_family(moe, work, 1) == 1 and product.hip.moe_kernel_family(moe, work, 16) == 1
        assert product.hip.moe_kernel_family(moe, work, 17) == 0
        for first, count in ((0, 1), (1, 1), (2, 4), (6, 16), (22, 3), (0, 16), (20, 18), (25, 15)):
            print(f"  streamed rows {first}..{first + count}", flush=True)
            rows = np.ascontiguousarray(x[first:first + count])
            y = np.full((count, cfg.hidden_size), -99.0, np.float32)
            ids = np.full((count, cfg.top_k), 0xFFFFFFFF, np.uint32)
            w = np.full((count, cfg.top_k), -99.0, np.float32)
            routes = abi.Qwen4MoeRoutes(abi.u32_view(ids), abi.f32_view(w))
            st = product.forward_streamed(layer.handle, pool, 0, abi.f32_view(rows), abi.f32_view(y), C.byref(routes),
                                          layer.work, C.byref(layer.err))
            assert st == abi.QW4_OK, layer.err.detail
            assert_parity(y, ids, w, want[0][first:first + count], want[1][first:first + count],
                          want[2][first:first + count], label=f"streamed rows {first}..{first + count}")
        stats = product.pool_stats(pool)
        assert stats.evictions > 0 and stats.hits > 0
    product.pool_destroy(pool)
    os.close(fd)


def test_streaming_refuses_what_it_cannot_hold(product, tmp_path):
    cfg = abi.moe_config(256, 16, 4, 256, 256)
    weights, x = make_layer_inputs(cfg, abi.GGUF_IQ2_XXS, 1, seed=3)   # stored split on the device
    err, handle = abi.Qwen4Error(), C.c_void_p()
    # routed bytes handed to a streamed layer
    assert product.create_streamed(C.byref(cfg), C.byref(weights.struct), C.byref(handle), C.byref(err)) == abi.QW4_INVALID_ARGUMENT
    assert not handle
    # a pool of file bytes under a layer whose kernels read another layout; a pool told another format
    sizes = [weights.raw[j].size // cfg.experts for j in (1, 2, 3)]
    path = tmp_path / "model.bin"
    np.concatenate([weights.raw[j] for j in (1, 2, 3)]).tofile(path)
    fd = os.open(path, os.O_RDONLY)
    table = (abi.QW4ExpertLayer * 1)(abi.QW4ExpertLayer((C.c_uint64 * 3)(0, weights.raw[1].size, weights.raw[1].size + weights.raw[2].size)))
    struct = streamed_weights(weights)
    assert product.create_streamed(C.byref(cfg), C.byref(struct), C.byref(handle), C.byref(err)) == abi.QW4_OK
    with pf.MoeLayer(product, cfg, weights, 1, handle=handle) as layer:
        y = np.full((1, cfg.hidden_size), -99.0, np.float32)
        plain = product.pool_create(fd, table, 1, cfg.experts, (C.c_size_t * 3)(*sizes), 8)
        st = product.forward_streamed(layer.handle, plain, 0, abi.f32_view(x), abi.f32_view(y), None, layer.work, C.byref(layer.err))
        assert st == abi.QW4_SHAPE and (y == -99.0).all()
        h, i = cfg.hidden_size, cfg.intermediate
        # the formats cannot change once the pool was used, and must match the slices' sizes
        wrong = (C.c_uint32 * 3)(abi.GGUF_Q4_K, abi.GGUF_Q4_K, abi.GGUF_Q4_K)
        assert product.pool_set_formats(plain, wrong, (C.c_size_t * 3)(h, h, i), (C.c_size_t * 3)(i, i, h)) == -1
        product.pool_destroy(plain)
    os.close(fd)
