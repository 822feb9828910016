"""CPU oracle for the GGUF loader of the MoE path.  TEST INFRASTRUCTURE ONLY.

A plain-Python restatement of what the reference does between a GGUF v3 file and the
eight weight views of one layer's MoE block.  Only tests/, __graft_entry__.smoke()
and bench.py's cpu_baseline leg may import this module; the shipped loader is
picoforge_amd/csrc/pf_gguf.c and never calls it.

Pinned by tests/test_oracle_gguf.py: against the layout the file writer of the tests
knows by construction, against the reference's own reader, config and catalog where
oracle/_ref was built, and on the malformed files of the reference's reader tests
(tests/test_gguf.py:40-94).

    parse(data)            src/gguf.c:31-105, src/gguf_reader.c
    moe_model(parsed)      src/qwen4_config.c:152-216 with the checks of :28-45, :61-84
    layer_config(model, l) src/qwen4_weights.c:97-99, src/qwen4_forward_gpu.m:707
    moe_rows(parsed, m, l) src/qwen4_weights.c:19-56 for the rows of :91-99

Failures raise Refused(status, subject, detail) with the reference's status names
and texts; where the reference's reader ends the process, the status is the one the
shipped loader documents (FORMAT unless stated).
"""
import struct

FORMATS = {0: ("F32", 1, 4), 1: ("F16", 1, 2), 8: ("Q8_0", 32, 34), 10: ("Q2_K", 256, 84), 12: ("Q4_K", 256, 144),
           16: ("IQ2_XXS", 256, 66), 30: ("BF16", 1, 2), 39: ("MXFP4", 32, 17)}       # src/gguf.c:12-16
WIDTHS = [1, 1, 2, 2, 4, 4, 4, 1, 0, 0, 8, 8, 8]                                          # src/gguf_reader.c:55
HEADER_LIMIT = 128 << 20
SIZE_MAX = 2 ** 64 - 1
KNOWN_KEYS = """block_count nextn_predict_layers context_length embedding_length vocab_size attention.head_count
attention.head_count_kv attention.key_length attention.value_length attention.layer_norm_rms_epsilon
attention.indexer.head_count attention.indexer.key_length attention.indexer.top_k expert_count expert_used_count
expert_feed_forward_length expert_shared_feed_forward_length ssm.conv_kernel ssm.state_size ssm.group_count
ssm.time_step_rank ssm.inner_size full_attention_interval hyper_connection.count hyper_connection.low_rank
rope.dimension_count rope.freq_base attention.compress_ratios ple.layers ple.ngram_size ple.heads_per_ngram
ple.conv_kernel ple.eos_token_id embedding_length_per_layer_input ple.seed ple.vocab_base ple.vocab_divisor
ple.row_count ple.row_dimension ple.layer_multipliers ple.head_offsets ple.head_vocab_sizes
ssm.output_gate_type""".split()                                                         # src/qwen4_config.c:62-74


class Refused(Exception):
    def __init__(self, status, subject, detail):
        super().__init__(f"{status}: {subject}: {detail}")
        self.status, self.subject, self.detail = status, subject, detail


class _Cursor:
    def __init__(self, data, size, pos=0):
        self.data, self.size, self.pos = data, size, pos

    def take(self, n):                                  # gguf_bytes, src/gguf_reader.c:16-22
        if self.pos > self.size or n > self.size - self.pos:
            raise Refused("FORMAT", "gguf", "gguf: truncated or oversized header")
        self.pos += n
        return self.data[self.pos - n:self.pos]

    def uint(self, width):                              # gguf_uint, :24-31
        return int.from_bytes(self.take(width), "little")

    def string(self):                                   # gguf_string, :33-38
        n = self.uint(8)
        if n > 16 << 20:
            raise Refused("FORMAT", "gguf", "gguf: oversized string")
        return self.take(n)

    def name(self, capacity=128):                       # gguf_name, :40-52
        raw = self.string()
        if not raw or len(raw) >= capacity:
            raise Refused("FORMAT", "gguf", "gguf: invalid name length")
        if any(not (chr(b).isascii() and (chr(b).isalnum() or chr(b) in "_.-")) for b in raw):
            raise Refused("FORMAT", "gguf", "gguf: unsupported identifier byte")
        return raw.decode("ascii")

    def skip(self, kind):                               # gguf_skip_value, :54-72
        if kind >= len(WIDTHS):
            raise Refused("FORMAT", "gguf", "gguf: unsupported metadata type")
        if kind == 8:
            self.string()
        elif kind == 9:
            element, count = self.uint(4), self.uint(8)
            if element >= len(WIDTHS) or element == 9 or count > 2000000:
                raise Refused("FORMAT", "gguf", "gguf: invalid metadata array")
            if element in (7, 8):
                for _ in range(count):
                    self.skip(element)
            else:
                self.take(count * WIDTHS[element])
        elif kind == 7:
            if self.uint(1) > 1:
                raise Refused("FORMAT", "gguf", "gguf: invalid boolean")
        else:
            self.take(WIDTHS[kind])


def parse(data):
    """-> dict(data_offset, file_size, tensors=[...] in file order, metadata={name: (type, value bytes)})."""
    file_size = len(data)
    if file_size < 24:
        raise Refused("IO", "gguf", "gguf: cannot open a complete regular file")
    c = _Cursor(data, min(file_size, HEADER_LIMIT))
    if c.take(4) != b"GGUF" or c.uint(4) != 3:
        raise Refused("FORMAT", "gguf", "gguf: expected little-endian GGUF v3")
    n_tensors, n_meta = c.uint(8), c.uint(8)
    if not n_tensors or n_tensors > 100000 or n_meta > 100000:
        raise Refused("FORMAT", "gguf", "gguf: invalid descriptor counts")
    alignment, architecture, names, metadata = 32, False, [], {}
    for _ in range(n_meta):
        name, kind = c.name(), c.uint(4)
        start = c.pos
        c.skip(kind)
        value = data[start:c.pos]
        if name == "general.architecture":
            if kind != 8:
                raise Refused("FORMAT", "gguf", "gguf: architecture must be a string")
            architecture = value[8:] == b"qwen4exp"
        elif name == "general.alignment":
            if kind != 4:
                raise Refused("FORMAT", "gguf", "gguf: alignment must be uint32")
            alignment = int.from_bytes(value[:4], "little")
        names.append(name)
        metadata[name] = (kind, value)
    if len(set(names)) != len(names):
        raise Refused("FORMAT", "gguf", "gguf: duplicate metadata key")
    if not architecture:
        raise Refused("UNSUPPORTED", "gguf", "gguf: expected qwen4exp architecture")
    if not alignment or alignment & (alignment - 1) or alignment > HEADER_LIMIT:
        raise Refused("FORMAT", "gguf", "gguf: invalid alignment")
    tensors = []
    for _ in range(n_tensors):
        name, rank = c.name(), c.uint(4)
        if not rank or rank > 4:
            raise Refused("FORMAT", "gguf", "gguf: invalid tensor rank")
        shape = []
        for _ in range(rank):
            shape.append(c.uint(8))
            if not shape[-1]:
                raise Refused("FORMAT", "gguf", "gguf: zero tensor dimension")
        kind, offset = c.uint(4), c.uint(8)
        if kind not in FORMATS:
            raise Refused("FORMAT", name, f"gguf: unsupported tensor format {kind}")
        _, block, nbytes = FORMATS[kind]
        if shape[0] % block or offset % alignment:
            raise Refused("FORMAT", name, f"gguf: unaligned tensor row or offset: {name}")
        size = shape[0] // block
        for factor in [nbytes] + shape[1:]:
            size *= factor
            if size > SIZE_MAX:
                raise Refused("OVERFLOW", name, "gguf: size overflow")
        tensors.append(dict(name=name, type=kind, rank=rank, shape=shape, file_offset=offset, bytes=size))
    data_offset = (c.pos + alignment - 1) & ~(alignment - 1)
    c.take(data_offset - c.pos)
    by_name = sorted(t["name"] for t in tensors)
    for a, b in zip(by_name, by_name[1:]):
        if a == b:
            raise Refused("FORMAT", a, "gguf: duplicate tensor name")
    tensors.sort(key=lambda t: t["file_offset"])
    end = data_offset
    for t in tensors:
        if t["file_offset"] + data_offset > SIZE_MAX:
            raise Refused("OVERFLOW", t["name"], "gguf: offset overflow")
        t["file_offset"] += data_offset
        if t["file_offset"] < end or t["file_offset"] > file_size or t["bytes"] > file_size - t["file_offset"]:
            raise Refused("FORMAT", t["name"], f"gguf: overlapping or out-of-file tensor: {t['name']}")
        end = t["file_offset"] + t["bytes"]
    return dict(data_offset=data_offset, file_size=file_size, tensors=tensors, metadata=metadata)


def _meta(parsed, key, kind):                           # qw4a_meta, src/qwen4_config.c:6-27
    if key not in parsed["metadata"]:
        raise Refused("MISSING", key, "required metadata")
    found, value = parsed["metadata"][key]
    if found != kind:
        raise Refused("TYPE", key, "metadata type")
    return value


def _u32(parsed, key):                                  # uint_field, :101-108
    value = _meta(parsed, key, 4)
    if len(value) != 4:
        raise Refused("FORMAT", key, "uint32 width")
    return int.from_bytes(value, "little")


def _dim(parsed, short):                                # the U() macro, :158-160
    value = _u32(parsed, "qwen4exp." + short)
    if not value:
        raise Refused("RANGE", short, "positive dimension")
    return value


def _positive_float(parsed, key):                       # float_field, :109-119
    value = _meta(parsed, key, 6)
    if len(value) != 4:
        raise Refused("FORMAT", key, "float32 width")
    x = struct.unpack("<f", value)[0]
    if x != x or x in (float("inf"), float("-inf")):
        raise Refused("NONFINITE", key, "finite value required")
    if x <= 0:
        raise Refused("RANGE", key, "positive value required")
    return x


def _find(parsed, name):
    hits = [t for t in parsed["tensors"] if t["name"] == name]
    return hits[0] if hits else None


def moe_model(parsed):
    for key in parsed["metadata"]:
        if key.startswith("qwen4exp.") and key[9:] not in KNOWN_KEYS:
            raise Refused("UNSUPPORTED", "config", "unknown computational metadata")
    m = dict(blocks=_dim(parsed, "block_count"), hidden_size=_dim(parsed, "embedding_length"),
             mtp_blocks=_u32(parsed, "qwen4exp.nextn_predict_layers"), experts=_dim(parsed, "expert_count"),
             top_k=_dim(parsed, "expert_used_count"), intermediate=_dim(parsed, "expert_feed_forward_length"),
             shared_intermediate=_dim(parsed, "expert_shared_feed_forward_length"),
             streams=_dim(parsed, "hyper_connection.count"), low_rank=_dim(parsed, "hyper_connection.low_rank"))
    m["rms_eps"] = _positive_float(parsed, "qwen4exp.attention.layer_norm_rms_epsilon")
    gate, down = _find(parsed, "blk.0.ffn_gate_exps.weight"), _find(parsed, "blk.0.ffn_down_exps.weight")
    if not gate or not down:
        raise Refused("FORMAT", "experts", "layer 0 routed expert tensors")
    if (gate["type"], down["type"]) == (16, 10):
        if _u32(parsed, "ds4.qwen4.down.logical_input") != m["intermediate"]:
            raise Refused("SHAPE", "down", "logical K mismatch")
        m.update(down_physical=_u32(parsed, "ds4.qwen4.down.physical_input"), trunk_type=[16, 16, 10],
                 semantic_profile="qwen38-q2-text-f32-v1")
    elif (gate["type"], down["type"]) == (12, 39):
        m.update(down_physical=m["intermediate"], trunk_type=[12, 12, 39], semantic_profile="qwen38-q4-text-f32-v1")
    else:
        raise Refused("UNSUPPORTED", "experts", "routed expert formats are neither the Q2 nor the Q4 profile")
    m["norm_topk_prob"] = True
    if m["blocks"] > 4096 or m["mtp_blocks"] >= m["blocks"]:
        raise Refused("RANGE", "config", "layer/order admission")
    m["trunk_blocks"] = m["blocks"] - m["mtp_blocks"]
    if m["top_k"] > m["experts"]:
        raise Refused("SHAPE", "config", "head/rotary/expert dimensions")
    padded = (m["intermediate"] + 255) // 256 * 256 if m["trunk_type"][2] == 10 else m["intermediate"]
    if padded > 2 ** 32 - 1 or padded != m["down_physical"]:
        raise Refused("SHAPE", "down", "physical K must round logical K to 256")
    if m["hidden_size"] * m["streams"] > 2 ** 32 - 1:
        raise Refused("OVERFLOW", "config", "derived dimension exceeds uint32")
    return m


def layer_config(model, layer):
    if layer >= model["blocks"]:
        raise Refused("RANGE", "weights", "layer/role index")
    c = {k: model[k] for k in ("hidden_size", "experts", "top_k", "intermediate", "shared_intermediate",
                               "down_physical", "norm_topk_prob")}
    c["trunk_type"] = list(model["trunk_type"])
    if layer >= model["trunk_blocks"]:
        c.update(trunk_type=[12, 12, 39], down_physical=c["intermediate"])
    return c


ROLES = ("router", "gate", "up", "down", "shared_gate", "shared_up", "shared_down", "shared_router")


def moe_rows(parsed, model, layer):
    """The eight tensors of the layer as {role: dict(name, type, k_storage, k_logical, n_out, experts,
    row_bytes, file_offset, bytes)}, checked in the catalog's order."""
    c = layer_config(model, layer)
    d, f, fs, ne = c["hidden_size"], c["intermediate"], c["shared_intermediate"], c["experts"]
    rows = [("router", "ffn_gate_inp.weight", 0, 2, d, ne, 1, d),
            ("shared_router", "ffn_gate_inp_shexp.weight", 0, 1, d, 1, 1, d),
            ("shared_gate", "ffn_gate_shexp.weight", 8, 2, d, fs, 1, d),
            ("shared_up", "ffn_up_shexp.weight", 8, 2, d, fs, 1, d),
            ("shared_down", "ffn_down_shexp.weight", 8, 2, fs, d, 1, fs),
            ("gate", "ffn_gate_exps.weight", c["trunk_type"][0], 3, d, f, ne, d),
            ("up", "ffn_up_exps.weight", c["trunk_type"][1], 3, d, f, ne, d),
            ("down", "ffn_down_exps.weight", c["trunk_type"][2], 3, c["down_physical"], d, ne, f)]
    out = {}
    for role, suffix, kind, rank, k, n, experts, logical in rows:
        name = f"blk.{layer}.{suffix}"
        t = _find(parsed, name)
        if t is None:
            raise Refused("MISSING", name, "required tensor")
        if t["type"] != kind:
            raise Refused("FORMAT", name, "Q2 recipe format mismatch")
        if t["rank"] != rank:
            raise Refused("SHAPE", name, "rank mismatch")
        if t["shape"] != [k, n, experts][:rank]:
            raise Refused("SHAPE", name, "physical shape mismatch")
        _, block, nbytes = FORMATS[kind]
        if not k or k % block or not logical or logical > k:
            raise Refused("SHAPE", name, "packed row alignment")
        row = k // block * nbytes
        if row * n * experts > SIZE_MAX:
            raise Refused("OVERFLOW", name, "tensor extent")
        if row * n * experts != t["bytes"]:
            raise Refused("FORMAT", name, "physical byte count")
        out[role] = dict(name=name, type=kind, k_storage=k, k_logical=logical, n_out=n, experts=experts,
                         row_bytes=row, file_offset=t["file_offset"], bytes=t["bytes"])
    return out
