"""Pins of the loader's CPU oracle (oracle/orc_gguf.py) and, against it, the shipped loader's
host logic (pf_gguf_* of the library; no device involved).

The oracle is pinned by (1) the layout the file writer knows by construction (tests/gguf_files.py puts
every tensor itself), (2) the reference's compiled reader, config loader and weight catalog where
oracle/_ref was built: gguf_open, qwen4_config_load, qwen4_weights_describe / qwen4_weights_get, and
(3) the malformed files of the reference's own reader tests (tests/test_gguf.py:40-94), which the
reference answers by ending the process: checked in a child process.
"""
import ctypes as C
import struct
import subprocess
import sys
import textwrap

import numpy as np
import pytest

import picoforge_amd as pf
from picoforge_amd import abi
from picoforge_amd.gguf import GgufFile, GgufError

import gguf_files as gf
from oracle import orc_gguf

ROLE_ORDER = """TOKEN_EMBD LM_HEAD OUTPUT_HC_NORM OUTPUT_HC_DOWN OUTPUT_HC_UP PLE_TABLE HC_ATTN_NORM HC_ATTN_DOWN HC_ATTN_UP
HC_ATTN_INJECT HC_FFN_NORM HC_FFN_DOWN HC_FFN_UP HC_FFN_INJECT GDN_QKV GDN_GATE GDN_ALPHA GDN_BETA GDN_A GDN_DT GDN_CONV
GDN_NORM GDN_OUT ATTN_QG ATTN_K ATTN_V ATTN_OUT ATTN_Q_NORM ATTN_K_NORM INDEX_Q INDEX_K INDEX_Q_NORM INDEX_K_NORM MOE_ROUTER
MOE_GATE MOE_UP MOE_DOWN SHARED_GATE SHARED_UP SHARED_DOWN SHARED_ROUTER""".split()    # src/qwen4.h:38-53
ROLE_OF = dict(router="MOE_ROUTER", gate="MOE_GATE", up="MOE_UP", down="MOE_DOWN", shared_gate="SHARED_GATE",
               shared_up="SHARED_UP", shared_down="SHARED_DOWN", shared_router="SHARED_ROUTER")


class RefGguf(C.Structure):             # src/gguf.h:27-34
    _fields_ = [("fd", C.c_int), ("header", C.c_void_p), ("header_size", C.c_size_t), ("file_size", C.c_size_t),
                ("data_offset", C.c_size_t), ("tensor_count", C.c_size_t), ("metadata_count", C.c_size_t),
                ("tensors", C.POINTER(abi.GgufTensor)), ("metadata", C.c_void_p)]


class RefGdnShape(C.Structure):         # src/qwen4_types.h:62-68
    _fields_ = [("key_heads", C.c_size_t), ("value_heads", C.c_size_t), ("key_dim", C.c_size_t), ("value_dim", C.c_size_t),
                ("rms_eps", C.c_float), ("l2_eps", C.c_float), ("silu_gate", C.c_bool)]


class RefAttention(C.Structure):        # src/qwen4_types.h:70-74
    _fields_ = [(n, C.c_uint32) for n in ("heads", "kv_heads", "head_dim", "index_heads", "index_kv_heads", "index_dim",
                                          "ratio", "token_budget", "rotary_dim")] + [("rms_eps", C.c_float), ("rope_theta", C.c_float)]


class RefConfigView(C.Structure):       # src/qwen4.h:14-22
    _fields_ = [(n, C.c_uint32) for n in ("hidden_size", "vocab_size", "blocks", "trunk_blocks", "mtp_blocks",
                                          "max_positions", "gdn_conv_kernel")] + \
               [("gdn", RefGdnShape), ("hc", abi.Qwen4HcShape), ("attention", RefAttention), ("moe", abi.Qwen4MoeConfig),
                ("semantic_profile", C.c_char_p)]


class RefTensor(C.Structure):           # src/qwen4.h:29-35
    _fields_ = [("storage", abi.GgufTensor), ("logical_shape", C.c_uint64 * 4), ("block_elems", C.c_uint64),
                ("block_bytes", C.c_uint64), ("row_bytes", C.c_uint64), ("plane_bytes", C.c_uint64),
                ("domain", C.c_int), ("layout", C.c_int), ("gpu", C.c_void_p)]


class RefModel:
    """The reference's reader, config and catalog on one file."""

    def __init__(self, lib, path):
        self.lib, self.g, self.err = lib, RefGguf(), abi.Qwen4Error()
        lib.gguf_open.argtypes = [C.c_char_p, C.POINTER(RefGguf)]
        lib.gguf_open.restype = None
        lib.gguf_open(str(path).encode(), C.byref(self.g))
        self.config, self.weights = C.c_void_p(), C.c_void_p()
        lib.qwen4_config_load.argtypes = [C.POINTER(RefGguf), C.POINTER(C.c_void_p), C.POINTER(abi.Qwen4Error)]
        lib.qwen4_config_view.restype = C.POINTER(RefConfigView)
        lib.qwen4_config_view.argtypes = [C.c_void_p]
        lib.qwen4_weights_describe.argtypes = [C.POINTER(RefGguf), C.c_void_p, C.POINTER(C.c_void_p), C.POINTER(abi.Qwen4Error)]
        lib.qwen4_weights_get.argtypes = [C.c_void_p, C.c_uint32, C.c_int, C.POINTER(C.POINTER(RefTensor)), C.POINTER(abi.Qwen4Error)]

    def load_config(self):
        st = self.lib.qwen4_config_load(C.byref(self.g), C.byref(self.config), C.byref(self.err))
        return st, (self.lib.qwen4_config_view(self.config).contents if st == abi.QW4_OK else None)

    def describe(self):
        return self.lib.qwen4_weights_describe(C.byref(self.g), self.config, C.byref(self.weights), C.byref(self.err))

    def get(self, layer, role):
        out = C.POINTER(RefTensor)()
        st = self.lib.qwen4_weights_get(self.weights, layer, ROLE_ORDER.index(role), C.byref(out), C.byref(self.err))
        return st, (out.contents if st == abi.QW4_OK else None)

    def tensors(self):
        return [self.g.tensors[i] for i in range(self.g.tensor_count)]

    def close(self):
        self.lib.qwen4_weights_free.argtypes = [C.c_void_p]
        self.lib.qwen4_config_free.argtypes = [C.c_void_p]
        self.lib.qwen4_weights_free(self.weights)
        self.lib.qwen4_config_free(self.config)
        self.lib.gguf_close.argtypes = [C.POINTER(RefGguf)]
        self.lib.gguf_close(C.byref(self.g))


MODELS = [dict(profile="q2", kinds=("gdn", 4), mtp=1), dict(profile="q4", kinds=("gdn", 4), mtp=1),
          dict(profile="q2", kinds=(4, "gdn", "gdn", 8), mtp=0, alignment=4096),
          dict(profile="q4", kinds=("gdn",), mtp=2, dims=dict(inter=96, shared=64, experts=6, top_k=3))]


def oracle_status(fn, *args):
    try:
        return "OK", fn(*args)
    except orc_gguf.Refused as r:
        return r.status, r


def product_open(api, path):
    try:
        return "OK", GgufFile(api, path)
    except GgufError as e:
        return abi.STATUS[e.status], e


# ---------------------------------------------------------------- the reader

@pytest.mark.parametrize("model", MODELS, ids=lambda m: f"{m['profile']}-{len(m['kinds'])}+{m['mtp']}")
def test_reader_reports_the_layout_the_writer_made(tmp_path, product_host, reference, model):
    mf = gf.ModelFile(**model)
    expected = mf.write(tmp_path / "m.gguf")
    data = open(mf.path, "rb").read()
    parsed = orc_gguf.parse(data)
    assert parsed["data_offset"] == mf.data_offset
    got = {t["name"]: dict(type=t["type"], shape=t["shape"], file_offset=t["file_offset"], bytes=t["bytes"]) for t in parsed["tensors"]}
    assert got == expected
    assert [t["file_offset"] for t in parsed["tensors"]] == sorted(t["file_offset"] for t in parsed["tensors"])
    with GgufFile(product_host, mf.path) as f:
        assert f.data_offset == mf.data_offset
        assert f.tensors() == [dict(name=t["name"], type=t["type"], shape=t["shape"], file_offset=t["file_offset"],
                                    bytes=t["bytes"]) for t in parsed["tensors"]]
    if reference is not None:
        ref = RefModel(reference.lib, mf.path)
        assert ref.g.data_offset == mf.data_offset and ref.g.tensor_count == len(expected)
        for t, mine in zip(ref.tensors(), parsed["tensors"]):
            assert (t.name.decode(), t.type, list(t.shape[:t.rank]), t.file_offset, t.bytes) == \
                (mine["name"], mine["type"], mine["shape"], mine["file_offset"], mine["bytes"])
        ref.close()


def test_every_format_and_the_padded_down_projection(tmp_path, product_host):
    # tests/test_gguf.py:35-39 and the byte counts of tests/test_qwen4_inventory.py:36-47
    sizes = {(16, 256): 66, (12, 256): 144, (8, 32): 34, (39, 32): 17, (30, 32): 64, (0, 32): 128, (1, 32): 64, (10, 768): 252}
    for (kind, width), nbytes in sizes.items():
        data = gf.one_tensor(kind=kind, dims=(width,))
        assert orc_gguf.parse(data)["tensors"][0]["bytes"] == nbytes
        path = tmp_path / f"t{kind}.gguf"
        path.write_bytes(data)
        with GgufFile(product_host, path) as f:
            assert f.tensors()[0]["bytes"] == nbytes
    t = orc_gguf.parse(gf.one_tensor())["tensors"][0]
    assert (t["shape"], t["bytes"]) == ([768, 2], 2 * 3 * 84)


MALFORMED = [dict(dims=(640,)), dict(dims=(0,)), dict(dims=()), dict(dims=(1, 1, 1, 1, 1)), dict(kind=999), dict(offset=1),
             dict(offset=2 ** 64 - 32), dict(duplicate=True), dict(dims=(2 ** 63, 2 ** 63)), dict(architecture="qwen3"),
             dict(magic=b"FGUG"), dict(version=2), dict(name="down weight"), dict(name="d" * 128), dict(payload=503),
             dict(extra_meta=[gf.kv_str("general.architecture", "qwen4exp")]),
             dict(extra_meta=[gf.kv("general.alignment", 10, struct.pack("<Q", 32))]),
             dict(extra_meta=[gf.kv_u32("general.alignment", 3)]),
             dict(extra_meta=[gf.kv("bad", 7, b"\x02")]),
             dict(extra_meta=[gf.kv("bad", 9, struct.pack("<IQ", 9, 1))]),
             dict(extra_meta=[gf.kv("bad", 9, struct.pack("<IQ", 4, 2000001))]),
             dict(extra_meta=[gf.kv("bad", 13, b"")]),
             dict(extra_meta=[gf.kv("bad", 8, struct.pack("<Q", (16 << 20) + 1))])]


def malformed_id(case):
    return ",".join(f"{k}={str(v)[:24]}" for k, v in case.items())


@pytest.mark.parametrize("case", MALFORMED, ids=malformed_id)
def test_malformed_files_are_refused_with_the_same_reason(tmp_path, product_host, case):
    data = gf.one_tensor(**case)
    st, refusal = oracle_status(orc_gguf.parse, data)
    assert st != "OK", case
    path = tmp_path / "bad.gguf"
    path.write_bytes(data)
    st_p, e = product_open(product_host, path)
    assert (st_p, e.detail) == (st, refusal.detail)


def test_every_header_truncation_is_refused(tmp_path, product_host):
    data = gf.one_tensor(extra_meta=[gf.kv_u64s("some.array", [1, 2, 3]), gf.kv_str("some.text", "abc")])
    end = orc_gguf.parse(data)["data_offset"]
    path = tmp_path / "cut.gguf"
    for size in list(range(end)) + [len(data) - 1]:
        st, refusal = oracle_status(orc_gguf.parse, data[:size])
        assert st in ("FORMAT", "IO"), size
        path.write_bytes(data[:size])
        st_p, e = product_open(product_host, path)
        assert (st_p, e.detail) == (st, refusal.detail), size


def test_the_reference_ends_the_process_on_the_same_files(tmp_path, reference):
    """The reference's reader calls exit(1) after printing its reason (src/util.c:13-21); the oracle's detail must be
    that reason.  One child process reads all the files, one fork per file."""
    if reference is None:
        pytest.skip("oracle/_ref was not built (reference tree not mounted at build time)")
    cases = MALFORMED + [dict()]
    for i, case in enumerate(cases):
        (tmp_path / f"{i}.gguf").write_bytes(gf.one_tensor(**case))
    child = textwrap.dedent(f"""
        import ctypes, os, sys
        lib = ctypes.CDLL({str(pf.binding.REPO_DIR / 'oracle' / '_ref' / 'libqwen4_ref.so')!r})
        for i in range({len(cases)}):
            pid = os.fork()
            if pid == 0:
                buf = ctypes.create_string_buffer(256)
                lib.gguf_open(os.path.join({str(tmp_path)!r}, f"{{i}}.gguf").encode(), buf)
                os._exit(0)
            print(i, os.waitstatus_to_exitcode(os.waitpid(pid, 0)[1]), flush=True)
    """)
    run = subprocess.run([sys.executable, "-c", child], capture_output=True, text=True, timeout=120)
    codes = dict(tuple(map(int, line.split())) for line in run.stdout.splitlines())
    reasons = [line[len("picoforge: "):] for line in run.stderr.splitlines() if line.startswith("picoforge: ")]
    assert codes[len(cases) - 1] == 0 and all(codes[i] == 1 for i in range(len(cases) - 1)), (codes, run.stderr)
    ours = [oracle_status(orc_gguf.parse, gf.one_tensor(**case))[1].detail for case in MALFORMED]
    assert len(reasons) == len(ours) and all(r.startswith(d) for r, d in zip(reasons, ours)), list(zip(reasons, ours))


# ---------------------------------------------------------------- config and catalog

SUFFIX = dict(router="ffn_gate_inp.weight", gate="ffn_gate_exps.weight", up="ffn_up_exps.weight", down="ffn_down_exps.weight",
              shared_gate="ffn_gate_shexp.weight", shared_up="ffn_up_shexp.weight", shared_down="ffn_down_shexp.weight",
              shared_router="ffn_gate_inp_shexp.weight")


def as_dict(cfg):
    return dict(hidden_size=cfg.hidden_size, experts=cfg.experts, top_k=cfg.top_k, intermediate=cfg.intermediate,
                shared_intermediate=cfg.shared_intermediate, down_physical=cfg.down_physical,
                norm_topk_prob=bool(cfg.norm_topk_prob), trunk_type=list(cfg.trunk_type))


@pytest.mark.parametrize("model", MODELS, ids=lambda m: f"{m['profile']}-{len(m['kinds'])}+{m['mtp']}")
def test_model_and_catalog_agree_with_the_reference(tmp_path, product_host, reference, model):
    mf = gf.ModelFile(**model)
    expected = mf.write(tmp_path / "m.gguf")
    parsed = orc_gguf.parse(open(mf.path, "rb").read())
    m = orc_gguf.moe_model(parsed)
    d = mf.d
    assert (m["hidden_size"], m["experts"], m["top_k"], m["intermediate"], m["shared_intermediate"], m["down_physical"]) == \
        (d["hidden"], d["experts"], d["top_k"], d["inter"], d["shared"], mf.down_physical)
    assert (m["blocks"], m["mtp_blocks"], m["streams"], m["low_rank"], m["trunk_type"]) == \
        (len(mf.kinds), mf.mtp, d["streams"], d["low_rank"], list(mf.trunk))
    ref = RefModel(reference.lib, mf.path) if reference is not None else None
    if ref:
        st, view = ref.load_config()
        assert st == abi.QW4_OK, ref.err.detail
        assert as_dict(view.moe) == {k: m[k] for k in as_dict(view.moe)}
        assert (view.blocks, view.trunk_blocks, view.mtp_blocks, view.semantic_profile.decode()) == \
            (m["blocks"], m["trunk_blocks"], m["mtp_blocks"], m["semantic_profile"])
        assert (view.hc.streams, view.hc.hidden_size, view.hc.low_rank) == (m["streams"], m["hidden_size"], m["low_rank"])
        assert np.float32(view.hc.rms_eps) == np.float32(m["rms_eps"])
        assert ref.describe() == abi.QW4_OK, (ref.err.subject, ref.err.detail)
    with GgufFile(product_host, mf.path) as f:
        pm = f.moe_model()
        assert as_dict(pm.moe) == {k: m[k] for k in as_dict(pm.moe)}
        assert (pm.blocks, pm.trunk_blocks, pm.mtp_blocks, pm.semantic_profile.decode()) == \
            (m["blocks"], m["trunk_blocks"], m["mtp_blocks"], m["semantic_profile"])
        assert (pm.hc.streams, pm.hc.hidden_size, pm.hc.low_rank, np.float32(pm.hc.rms_eps)) == \
            (m["streams"], m["hidden_size"], m["low_rank"], np.float32(m["rms_eps"]))
        base = f.api.tensor_bytes(f.handle, f.api.tensor(f.handle, 0)) - f.tensors()[0]["file_offset"]
        for layer in range(m["blocks"]):
            rows = orc_gguf.moe_rows(parsed, m, layer)
            assert as_dict(f.layer_config(layer)) == orc_gguf.layer_config(m, layer)
            w = f.moe_weights(layer).struct
            for role, row in rows.items():
                assert expected[row["name"]]["file_offset"] == row["file_offset"]
                view = getattr(w, role)
                lay = view.layout
                assert (lay.gguf_type, lay.k_storage, lay.k_logical, lay.n_out, lay.n_experts, lay.row_bytes, lay.tensor_bytes) == \
                    (row["type"], row["k_storage"], row["k_logical"], row["n_out"], row["experts"], row["row_bytes"], row["bytes"])
                assert (view.span.data - base, view.span.bytes) == (row["file_offset"], row["bytes"])
                if ref:
                    st, t = ref.get(layer, ROLE_OF[role])
                    assert st == abi.QW4_OK
                    assert (t.storage.name.decode(), t.storage.type, t.storage.file_offset, t.storage.bytes, t.logical_shape[0],
                            t.row_bytes) == (row["name"], row["type"], row["file_offset"], row["bytes"], row["k_logical"], row["row_bytes"])
                    assert t.plane_bytes == row["row_bytes"] * row["n_out"]
        with pytest.raises(GgufError) as e:
            f.moe_weights(m["blocks"])
        assert abi.STATUS[e.value.status] == "RANGE"
    if ref:
        ref.close()


def faults():
    p = "qwen4exp."
    yield "zero experts", dict(meta={p + "expert_count": gf.kv_u32(p + "expert_count", 0)}), "RANGE"
    yield "top_k above experts", dict(meta={p + "expert_used_count": gf.kv_u32(p + "expert_used_count", 9)}), "SHAPE"
    yield "missing key", dict(meta={p + "expert_feed_forward_length": None}), "MISSING"
    yield "wrong key type", dict(meta={p + "embedding_length": gf.kv(p + "embedding_length", 5, struct.pack("<i", 256))}), "TYPE"
    yield "unknown key", dict(meta={p + "expert_bias": gf.kv_u32(p + "expert_bias", 1)}), "UNSUPPORTED"
    yield "nan eps", dict(meta={p + "attention.layer_norm_rms_epsilon":
                                gf.kv(p + "attention.layer_norm_rms_epsilon", 6, struct.pack("<I", 0x7fc00000))}), "NONFINITE"
    yield "negative eps", dict(meta={p + "attention.layer_norm_rms_epsilon": gf.kv_f32(p + "attention.layer_norm_rms_epsilon", -1.0)}), "RANGE"
    yield "physical K", dict(meta={"ds4.qwen4.down.physical_input": gf.kv_u32("ds4.qwen4.down.physical_input", 7)}), "SHAPE"
    yield "logical K", dict(meta={"ds4.qwen4.down.logical_input": gf.kv_u32("ds4.qwen4.down.logical_input", 32)}), "SHAPE"
    yield "all layers MTP", dict(meta={p + "nextn_predict_layers": gf.kv_u32(p + "nextn_predict_layers", 3)}), "RANGE"
    yield "too many blocks", dict(meta={p + "block_count": gf.kv_u32(p + "block_count", 4097)}), "RANGE"
    yield "mixed profile", dict(tensors={"blk.0.ffn_down_exps.weight": (39, (64, 256, 4))}), "UNSUPPORTED"
    yield "no layer-0 experts", dict(drop={"blk.0.ffn_gate_exps.weight"}), "FORMAT"


@pytest.mark.parametrize("name,fault,status", list(faults()), ids=[f[0] for f in faults()])
def test_config_faults(tmp_path, product_host, reference, name, fault, status):
    mf = gf.ModelFile(profile="q2")
    mf.meta_overrides, mf.tensor_overrides, mf.dropped = fault.get("meta", {}), fault.get("tensors", {}), fault.get("drop", set())
    mf.write(tmp_path / "m.gguf")
    parsed = orc_gguf.parse(open(mf.path, "rb").read())
    st, refusal = oracle_status(orc_gguf.moe_model, parsed)
    assert st == status
    with GgufFile(product_host, mf.path) as f:
        with pytest.raises(GgufError) as e:
            f.moe_model()
        assert (abi.STATUS[e.value.status], e.value.subject, e.value.detail) == (st, refusal.subject, refusal.detail)
    if reference is not None:
        ref = RefModel(reference.lib, mf.path)
        st_ref, _ = ref.load_config()
        assert (abi.STATUS[st_ref], ref.err.subject.decode(), ref.err.detail.decode()) == (st, refusal.subject, refusal.detail)
        ref.close()


def catalog_faults():
    yield "missing tensor", dict(drop={"blk.1.ffn_up_shexp.weight"}), "MISSING", 1
    yield "wrong format", dict(tensors={"blk.1.ffn_gate_shexp.weight": (1, (256, 32))}), "FORMAT", 1
    yield "wrong rank", dict(tensors={"blk.0.ffn_gate_inp_shexp.weight": (0, (256, 1))}), "SHAPE", 0
    yield "wrong shape", dict(tensors={"blk.1.ffn_down_exps.weight": (10, (256, 256, 5))}), "SHAPE", 1
    yield "trunk formats in the MTP layer", dict(tensors={"blk.2.ffn_gate_exps.weight": (16, (256, 64, 4))}), "FORMAT", 2


@pytest.mark.parametrize("name,fault,status,layer", list(catalog_faults()), ids=[f[0] for f in catalog_faults()])
def test_catalog_faults(tmp_path, product_host, reference, name, fault, status, layer):
    mf = gf.ModelFile(profile="q2")
    mf.tensor_overrides, mf.dropped = fault.get("tensors", {}), fault.get("drop", set())
    mf.write(tmp_path / "m.gguf")
    parsed = orc_gguf.parse(open(mf.path, "rb").read())
    m = orc_gguf.moe_model(parsed)
    st, refusal = oracle_status(orc_gguf.moe_rows, parsed, m, layer)
    assert st == status
    for other in range(m["blocks"]):
        if other != layer:
            orc_gguf.moe_rows(parsed, m, other)
    with GgufFile(product_host, mf.path) as f:
        with pytest.raises(GgufError) as e:
            f.moe_weights(layer)
        assert (abi.STATUS[e.value.status], e.value.subject, e.value.detail) == (st, refusal.subject, refusal.detail)
    if reference is not None:
        ref = RefModel(reference.lib, mf.path)
        assert ref.load_config()[0] == abi.QW4_OK
        st_ref = ref.describe()
        assert (abi.STATUS[st_ref], ref.err.subject.decode(), ref.err.detail.decode()) == (st, refusal.subject, refusal.detail)
        ref.close()


def test_null_arguments(product_host):
    api = pf.gguf.GgufApi(product_host.lib)
    err = abi.Qwen4Error()
    handle = C.c_void_p(1)
    assert api.open(None, C.byref(handle), C.byref(err)) == abi.QW4_INVALID_ARGUMENT and not handle
    assert api.open(b"/nonexistent/x.gguf", C.byref(handle), C.byref(err)) == abi.QW4_IO and err.os_errno != 0 and not handle
    assert api.moe_model(None, None, None) == abi.QW4_INVALID_ARGUMENT
    assert api.moe_weights(None, None, 0, None, None) == abi.QW4_INVALID_ARGUMENT
    assert api.moe_create(None, None, 0, C.byref(handle), None) == abi.QW4_INVALID_ARGUMENT and not handle
    assert api.tensor_count(None) == 0 and not api.tensor(None, 0) and not api.find(None, b"x")
    api.close(None)


@pytest.mark.parametrize("profile", ["q2", "q4"])
def test_views_show_the_bytes_that_were_written(tmp_path, product_host, oracle, profile):
    """The spans handed to qwen4_moe_create hold exactly the tensors' bytes; the CPU oracle, given those views,
    computes what it computes on the same tensors held in memory."""
    mf = gf.ModelFile(profile=profile, kinds=("gdn",), mtp=1, moe_only=True, seed=4)
    expected = mf.write(tmp_path / "m.gguf")
    x = pf.rms_normalise(pf.Synth().normal((3, mf.d["hidden"]), 11))
    with GgufFile(product_host, mf.path) as f:
        for layer in range(2):
            fw = f.moe_weights(layer)
            raw, types = [], []
            for role in pf.layer.ROLE:
                view = getattr(fw.struct, role)
                name = f"blk.{layer}.{SUFFIX[role]}"
                want = mf.values(name, expected[name]["type"], expected[name]["shape"])
                got = np.frombuffer(C.string_at(view.span.data, view.span.bytes), dtype=np.uint8)
                np.testing.assert_array_equal(got, want)
                raw.append(got.copy())
                types.append(expected[name]["type"])
            held = pf.LayerWeights(fw.cfg, raw, types)
            with pf.MoeLayer(oracle, fw.cfg, fw, 3) as a, pf.MoeLayer(oracle, fw.cfg, held, 3) as b:
                ya, yb = a.forward(x), b.forward(x)
            for u, v in zip(ya[1:], yb[1:]):
                np.testing.assert_array_equal(u, v)
