"""Writer of small GGUF v3 files for the loader's tests.

Two kinds of file:
 * `one_tensor(...)`: a header with one descriptor, the shape of the malformed-layout cases of the
   reference's reader tests (tests/test_gguf.py:40-94 with the fixture of
   tests/test_qwen4_inventory.py:19-26): every argument can be made invalid.
 * `ModelFile`: a whole small qwen4exp model (every metadata key and every tensor the reference's
   config loader and weight catalog insist on, src/qwen4_config.c:152-279, src/qwen4_weights.c:57-125),
   so that the reference's own code accepts it and its answers can be compared.  The MoE tensors
   carry real quantised values; every other tensor is a hole in a sparse file.

The writer records where it put everything (`expected`), which is the layout the readers must report.
"""
import struct

import numpy as np

from picoforge_amd import abi


def string(text):
    raw = text.encode() if isinstance(text, str) else text
    return struct.pack("<Q", len(raw)) + raw


def kv(key, kind, payload):
    return string(key) + struct.pack("<I", kind) + payload


def kv_u32(key, value):
    return kv(key, 4, struct.pack("<I", value))


def kv_f32(key, value):
    return kv(key, 6, struct.pack("<f", value))


def kv_str(key, value):
    return kv(key, 8, string(value))


def kv_u64s(key, values):
    return kv(key, 9, struct.pack("<IQ", 10, len(values)) + struct.pack(f"<{len(values)}Q", *values))


def descriptor(name, dims, kind, offset):
    return string(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", n) for n in dims) + \
        struct.pack("<IQ", kind, offset)


def one_tensor(dims=(768, 2), kind=10, offset=0, duplicate=False, architecture="qwen4exp", name="down.weight",
               extra_meta=(), payload=504, version=3, magic=b"GGUF"):
    meta = [kv_str("general.architecture", architecture)] + list(extra_meta)
    tensor = descriptor(name, dims, kind, offset)
    data = magic + struct.pack("<IQQ", version, 2 if duplicate else 1, len(meta)) + b"".join(meta) + tensor
    if duplicate:
        data += tensor
    return data + bytes(-len(data) % 32) + bytes(payload)


def tensor_bytes(kind, dims):
    block, nbytes = abi.BLOCK[kind]
    assert dims[0] % block == 0
    return dims[0] // block * nbytes * int(np.prod(dims[1:], dtype=np.int64))


SMALL = dict(hidden=256, vocab=512, streams=2, low_rank=32, heads=4, kv_heads=2, head_dim=32, index_heads=2,
             index_dim=32, budget=8, rotary=16, key_dim=32, key_heads=2, value_heads=4, inner=128, conv=4,
             experts=4, top_k=2, inter=64, shared=32, context=1024, eps=1e-6, theta=1e6)


class ModelFile:
    """kinds: per layer "gdn" or an integer compress ratio (QSA); the last `mtp` layers are MTP layers.
    profile "q2" (IQ2_XXS gate/up, Q2_K down padded to 256) or "q4" (Q4_K gate/up, MXFP4 down)."""

    def __init__(self, profile="q2", kinds=("gdn", 4), mtp=1, dims=None, alignment=32, seed=1, moe_only=False,
                 std=0.05):
        self.d = dict(SMALL, **(dims or {}))
        self.profile, self.mtp, self.alignment, self.seed, self.std = profile, mtp, alignment, seed, std
        self.kinds = list(kinds) + [4] * mtp
        self.moe_only = moe_only          # only the MoE tensors: enough for this build's loader, not for the reference's
        d = self.d
        self.down_physical = (d["inter"] + 255) // 256 * 256 if profile == "q2" else d["inter"]
        self.trunk = (16, 16, 10) if profile == "q2" else (12, 12, 39)
        self.meta_overrides, self.tensor_overrides, self.dropped = {}, {}, set()

    # ---- metadata ----
    def metadata(self):
        d, p = self.d, "qwen4exp."
        ratios = [0 if k == "gdn" else int(k) for k in self.kinds]
        items = {
            "general.architecture": kv_str("general.architecture", "qwen4exp"),
            "general.alignment": kv_u32("general.alignment", self.alignment),
            p + "block_count": kv_u32(p + "block_count", len(self.kinds)),
            p + "context_length": kv_u32(p + "context_length", d["context"]),
            p + "embedding_length": kv_u32(p + "embedding_length", d["hidden"]),
            p + "vocab_size": kv_u32(p + "vocab_size", d["vocab"]),
            p + "nextn_predict_layers": kv_u32(p + "nextn_predict_layers", self.mtp),
            p + "attention.head_count": kv_u32(p + "attention.head_count", d["heads"]),
            p + "attention.head_count_kv": kv_u32(p + "attention.head_count_kv", d["kv_heads"]),
            p + "attention.key_length": kv_u32(p + "attention.key_length", d["head_dim"]),
            p + "attention.value_length": kv_u32(p + "attention.value_length", d["head_dim"]),
            p + "attention.indexer.head_count": kv_u32(p + "attention.indexer.head_count", d["index_heads"]),
            p + "attention.indexer.key_length": kv_u32(p + "attention.indexer.key_length", d["index_dim"]),
            p + "attention.indexer.top_k": kv_u32(p + "attention.indexer.top_k", d["budget"]),
            p + "expert_count": kv_u32(p + "expert_count", d["experts"]),
            p + "expert_used_count": kv_u32(p + "expert_used_count", d["top_k"]),
            p + "expert_feed_forward_length": kv_u32(p + "expert_feed_forward_length", d["inter"]),
            p + "expert_shared_feed_forward_length": kv_u32(p + "expert_shared_feed_forward_length", d["shared"]),
            p + "ssm.conv_kernel": kv_u32(p + "ssm.conv_kernel", d["conv"]),
            p + "ssm.state_size": kv_u32(p + "ssm.state_size", d["key_dim"]),
            p + "ssm.group_count": kv_u32(p + "ssm.group_count", d["key_heads"]),
            p + "ssm.time_step_rank": kv_u32(p + "ssm.time_step_rank", d["value_heads"]),
            p + "ssm.inner_size": kv_u32(p + "ssm.inner_size", d["inner"]),
            p + "hyper_connection.count": kv_u32(p + "hyper_connection.count", d["streams"]),
            p + "hyper_connection.low_rank": kv_u32(p + "hyper_connection.low_rank", d["low_rank"]),
            p + "rope.dimension_count": kv_u32(p + "rope.dimension_count", d["rotary"]),
            p + "attention.layer_norm_rms_epsilon": kv_f32(p + "attention.layer_norm_rms_epsilon", d["eps"]),
            p + "rope.freq_base": kv_f32(p + "rope.freq_base", d["theta"]),
            p + "attention.compress_ratios": kv_u64s(p + "attention.compress_ratios", ratios),
        }
        if self.profile == "q2":
            items["ds4.qwen4.down.logical_input"] = kv_u32("ds4.qwen4.down.logical_input", d["inter"])
            items["ds4.qwen4.down.physical_input"] = kv_u32("ds4.qwen4.down.physical_input", self.down_physical)
        for key, blob in self.meta_overrides.items():
            if blob is None:
                items.pop(key, None)
            else:
                items[key] = blob
        return list(items.values())

    # ---- tensors ----
    def moe_tensors(self, layer):
        d = self.d
        mtp = layer >= len(self.kinds) - self.mtp
        gate, up, down = (12, 12, 39) if mtp else self.trunk
        k_down = d["inter"] if mtp else self.down_physical
        h, e, f, fs = d["hidden"], d["experts"], d["inter"], d["shared"]
        b = f"blk.{layer}."
        return [(b + "ffn_gate_inp.weight", 0, (h, e)), (b + "ffn_gate_inp_shexp.weight", 0, (h,)),
                (b + "ffn_gate_shexp.weight", 8, (h, fs)), (b + "ffn_up_shexp.weight", 8, (h, fs)),
                (b + "ffn_down_shexp.weight", 8, (fs, h)), (b + "ffn_gate_exps.weight", gate, (h, f, e)),
                (b + "ffn_up_exps.weight", up, (h, f, e)), (b + "ffn_down_exps.weight", down, (k_down, h, e))]

    def other_tensors(self):
        d = self.d
        h, x, r = d["hidden"], d["hidden"] * d["streams"], d["low_rank"]
        q, kvd = d["heads"] * d["head_dim"], d["kv_heads"] * d["head_dim"]
        gc = 2 * d["key_heads"] * d["key_dim"] + d["inner"]

        def hc(prefix):
            return [(prefix + "_norm.weight", 0, (x,)), (prefix + "_down.weight", 1, (x, r)), (prefix + "_up.weight", 1, (r, x))]
        out = [("token_embd.weight", 30, (h, d["vocab"])), ("output.weight", 8, (h, d["vocab"]))] + hc("output_hc")
        for layer, kind in enumerate(self.kinds):
            b = f"blk.{layer}."
            out += [(b + n, t, s) for n, t, s in hc("hc_attn") + hc("hc_ffn")]
            out += [(b + "hc_attn_inject.weight", 1, (x, d["streams"])), (b + "hc_ffn_inject.weight", 1, (x, d["streams"]))]
            if kind == "gdn":
                out += [(b + "attn_qkv.weight", 8, (h, gc)), (b + "attn_gate.weight", 8, (h, d["inner"])),
                        (b + "ssm_out.weight", 8, (d["inner"], h)), (b + "ssm_alpha.weight", 0, (h, d["value_heads"])),
                        (b + "ssm_beta.weight", 0, (h, d["value_heads"])), (b + "ssm_a", 0, (d["value_heads"],)),
                        (b + "ssm_dt.bias", 0, (d["value_heads"],)), (b + "ssm_norm.weight", 0, (d["inner"] // d["value_heads"],)),
                        (b + "ssm_conv1d.weight", 0, (d["conv"], gc))]
            else:
                out += [(b + "attn_q.weight", 8, (h, 2 * q)), (b + "attn_k.weight", 8, (h, kvd)), (b + "attn_v.weight", 8, (h, kvd)),
                        (b + "attn_output.weight", 8, (q, h)), (b + "attn_q_norm.weight", 0, (d["head_dim"],)),
                        (b + "attn_k_norm.weight", 0, (d["head_dim"],)),
                        (b + "indexer.q_proj.weight", 8, (h, d["index_heads"] * d["index_dim"])),
                        (b + "indexer.k_proj.weight", 8, (h, d["index_dim"])), (b + "indexer.q_norm.weight", 0, (d["index_dim"],)),
                        (b + "indexer.k_norm.weight", 0, (d["index_dim"],))]
            if layer >= len(self.kinds) - self.mtp:
                out += [(b + "nextn.eh_proj.weight", 8, (2 * h, h)), (b + "nextn.enorm.weight", 0, (h,)),
                        (b + "nextn.hnorm.weight", 0, (x,))] + [(b + n, t, s) for n, t, s in hc("nextn.hc_head")]
        return out

    def tensor_list(self):
        out = [] if self.moe_only else self.other_tensors()
        for layer in range(len(self.kinds)):
            out += self.moe_tensors(layer)
        fixed = []
        for name, kind, shape in out:
            if name in self.dropped:
                continue
            kind, shape = self.tensor_overrides.get(name, (kind, shape))
            fixed.append((name, kind, tuple(shape)))
        return fixed

    def values(self, name, kind, shape):
        """Seeded contents of a MoE tensor as GGUF bytes (None: leave a hole)."""
        if ".ffn_" not in name:
            return None
        from picoforge_amd import Synth
        synth = Synth()
        stream = self.seed * 1000 + (sum(name.encode()) * 31 + len(name)) % 997
        count = int(np.prod(shape, dtype=np.int64))
        if kind == abi.GGUF_F32:
            return synth.normal((count,), stream, 2.0 / np.sqrt(shape[0]) if "gate_inp" in name else self.std).view(np.uint8)   # logits of spread 2
        if kind == abi.GGUF_Q4_K:
            return synth.q4k_normal(count // 256, stream, self.std)
        if kind == abi.GGUF_IQ2_XXS:
            return synth.iq2xxs_uniform(count // 256, stream, 2.0 ** -9)
        if kind in (abi.GGUF_F16, abi.GGUF_BF16):
            x = synth.normal((count,), stream, self.std)
            return (x.astype(np.float16) if kind == abi.GGUF_F16 else (x.view(np.uint32) >> 16).astype(np.uint16)).view(np.uint8)
        return synth.quantised_normal(kind, count, stream, self.std)

    def write(self, path):
        """Writes the file; returns {name: dict(type, shape, file_offset, bytes)} and keeps it in self.expected."""
        tensors = self.tensor_list()
        meta = self.metadata()
        header = bytearray(b"GGUF" + struct.pack("<IQQ", 3, len(tensors), len(meta)) + b"".join(meta))
        a, offset, placed = self.alignment, 0, []
        for name, kind, shape in tensors:
            offset = (offset + a - 1) // a * a
            size = tensor_bytes(kind, shape)
            header += descriptor(name, shape, kind, offset)
            placed.append((name, kind, shape, offset, size))
            offset += size
        start = (len(header) + a - 1) // a * a
        self.expected = {n: dict(type=k, shape=list(s), file_offset=start + o, bytes=z) for n, k, s, o, z in placed}
        self.data_offset = start
        with open(path, "wb") as f:
            f.write(header)
            f.truncate(start + offset)
            for name, kind, shape, o, size in placed:
                raw = self.values(name, kind, shape)
                if raw is not None:
                    assert raw.size == size, (name, raw.size, size)
                    f.seek(start + o)
                    f.write(raw.tobytes())
        self.path = str(path)
        return self.expected
