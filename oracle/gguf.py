"""GGUF reader and writer in plain Python: TEST INFRASTRUCTURE ONLY (the checker for vexel_amd/host/gguf.cpp).

The reader restates inference/pkg/gguf/gguf.go of the reference function by function; the writer is its inverse
and exists so that tests can make checkpoints (the reference has no writer and ships no .gguf file). Pinned by the
reference's own tests: the handcrafted minimal file of gguf_test.go:109-183, the invalid-magic and old-version
cases (:185-206), the type tables (:9-65), NumElements (:67-85), AsUint32 (:87-107) and the name mapping of
loader_test.go:7-51.
"""
import struct

MAGIC = 0x46554747  # gguf.go:13
# gguf.go:21-36
MT_U8, MT_I8, MT_U16, MT_I16, MT_U32, MT_I32, MT_F32, MT_BOOL, MT_STRING, MT_ARRAY, MT_U64, MT_I64, MT_F64 = range(13)
# gguf.go:40-60
T_F32, T_F16, T_Q4_0, T_Q4_1, T_Q5_0, T_Q5_1, T_Q8_0, T_Q8_1 = 0, 1, 2, 3, 6, 7, 8, 9
T_Q2_K, T_Q3_K, T_Q4_K, T_Q5_K, T_Q6_K, T_Q8_K, T_BF16 = 10, 11, 12, 13, 14, 15, 30

_SCALAR = {MT_U8: "<B", MT_I8: "<b", MT_U16: "<H", MT_I16: "<h", MT_U32: "<I", MT_I32: "<i", MT_U64: "<Q",
           MT_I64: "<q", MT_F32: "<f", MT_F64: "<d", MT_BOOL: "<B"}


def type_string(t):  # gguf.go:62-91
    names = {T_F32: "F32", T_F16: "F16", T_Q4_0: "Q4_0", T_Q4_1: "Q4_1", T_Q5_0: "Q5_0", T_Q5_1: "Q5_1", T_Q8_0: "Q8_0",
             T_Q8_1: "Q8_1", T_Q4_K: "Q4_K", T_Q5_K: "Q5_K", T_Q6_K: "Q6_K", T_BF16: "BF16"}
    return names.get(t, "Unknown(%d)" % t)


def block_size(t):  # gguf.go:94-106
    if t in (T_F32, T_F16, T_BF16):
        return 1
    if t in (T_Q4_0, T_Q4_1, T_Q5_0, T_Q5_1, T_Q8_0, T_Q8_1):
        return 32
    if t in (T_Q4_K, T_Q5_K, T_Q6_K):
        return 256
    return 32


def bytes_per_block(t):  # gguf.go:108-131
    return {T_F32: 4, T_F16: 2, T_BF16: 2, T_Q4_0: 18, T_Q5_0: 22, T_Q5_1: 24, T_Q8_0: 34, T_Q4_K: 144, T_Q5_K: 176,
            T_Q6_K: 210}.get(t, 32)


class MetaValue:
    def __init__(self, type_, value, array_type=None):
        self.type, self.value, self.array_type = type_, value, array_type

    def as_uint32(self):  # gguf.go:158-169
        if self.type in (MT_U32, MT_U64, MT_I32):
            return self.value & 0xFFFFFFFF
        return 0

    def as_uint64(self):  # gguf.go:172-181
        return self.value if self.type in (MT_U64, MT_U32) else 0

    def as_float32(self):  # gguf.go:189-198
        if self.type == MT_F32:
            return self.value
        if self.type == MT_F64:
            return struct.unpack("<f", struct.pack("<f", self.value))[0]
        return 0.0

    def as_string(self):
        return self.value if self.type == MT_STRING else ""


class TensorInfo:
    def __init__(self, name, dims, type_, offset):
        self.name, self.dims, self.type, self.offset = name, list(dims), type_, offset

    def num_elements(self):  # gguf.go:209-218
        if not self.dims:
            return 0
        n = 1
        for d in self.dims:
            n *= d
        return n

    def num_bytes(self):  # gguf.go:600-604
        bs = block_size(self.type)
        return (self.num_elements() + bs - 1) // bs * bytes_per_block(self.type)


class ParseError(Exception):
    pass


class File:
    """Result of parse(): version, metadata (dict, last value of a repeated key), keys in file order, tensors,
    data_offset, and the extracted configuration."""

    def __init__(self):
        self.version, self.metadata, self.keys, self.tensors, self.data_offset = 0, {}, [], [], 0

    def get_tensor(self, name):  # gguf.go:584-591
        for t in self.tensors:
            if t.name == name:
                return t
        return None

    def config(self):  # gguf.go:504-582 (LLaMA keys)
        md = self.metadata
        arch = md["general.architecture"].as_string() if "general.architecture" in md else ""
        prefix = (arch or "llama") + "."
        c = dict(architecture=arch, num_layers=0, hidden=0, num_heads=0, num_kv_heads=0, ffn=0, context_length=0, vocab=0,
                 rope_dim_count=0, head_dim=0, rope_theta=10000.0, rms_eps=0.0)
        for key, field in (("block_count", "num_layers"), ("embedding_length", "hidden"), ("attention.head_count", "num_heads"),
                           ("feed_forward_length", "ffn"), ("context_length", "context_length"),
                           ("rope.dimension_count", "rope_dim_count"), ("attention.key_length", "head_dim")):
            if prefix + key in md:
                c[field] = md[prefix + key].as_uint32()
        c["num_kv_heads"] = md[prefix + "attention.head_count_kv"].as_uint32() if prefix + "attention.head_count_kv" in md \
            else c["num_heads"]
        if prefix + "rope.freq_base" in md:
            c["rope_theta"] = md[prefix + "rope.freq_base"].as_float32()
        if prefix + "attention.layer_norm_rms_epsilon" in md:
            c["rms_eps"] = md[prefix + "attention.layer_norm_rms_epsilon"].as_float32()
        tok = md.get("tokenizer.ggml.tokens")
        if tok is not None and tok.type == MT_ARRAY:
            c["vocab"] = len(tok.value)
        return c


class _Reader:
    def __init__(self, buf):
        self.buf, self.pos = buf, 0

    def get(self, fmt):
        n = struct.calcsize(fmt)
        if self.pos + n > len(self.buf):
            raise ParseError("unexpected end of file")
        v = struct.unpack_from(fmt, self.buf, self.pos)[0]
        self.pos += n
        return v

    def string(self):  # gguf.go:337-350
        n = self.get("<Q")
        if n > 65535:
            raise ParseError("string too long: %d" % n)
        if self.pos + n > len(self.buf):
            raise ParseError("unexpected end of file")
        s = bytes(self.buf[self.pos:self.pos + n]).decode("utf-8", errors="surrogateescape")
        self.pos += n
        return s


def _read_scalar(r, t):
    if t == MT_STRING:
        return r.string()
    if t not in _SCALAR:
        raise ParseError("unknown metadata type: %d" % t)
    v = r.get(_SCALAR[t])
    return (v != 0) if t == MT_BOOL else v


def parse(buf):
    """parseHeader (gguf.go:278-335). Nested arrays are refused (the reference consumes no bytes for their elements
    and loses its place)."""
    f, r = File(), _Reader(buf)
    if r.get("<I") != MAGIC:
        raise ParseError("invalid magic")
    f.version = r.get("<I")
    if f.version < 2 or f.version > 3:
        raise ParseError("unsupported version: %d" % f.version)
    n_tensors, n_meta = r.get("<Q"), r.get("<Q")
    for _ in range(n_meta):
        key = r.string()
        t = r.get("<I")
        if t == MT_ARRAY:
            at, n = r.get("<I"), r.get("<Q")
            if at == MT_ARRAY or at > MT_F64:
                raise ParseError("unsupported array element type: %d" % at)
            v = MetaValue(MT_ARRAY, [_read_scalar(r, at) for _ in range(n)], at)
        else:
            v = MetaValue(t, _read_scalar(r, t))
        if key not in f.metadata:
            f.keys.append(key)
        f.metadata[key] = v
    for _ in range(n_tensors):  # gguf.go:465-502
        name = r.string()
        nd = r.get("<I")
        dims = [r.get("<Q") for _ in range(nd)]
        f.tensors.append(TensorInfo(name, dims, r.get("<I"), r.get("<Q")))
    alignment = f.metadata["general.alignment"].as_uint64() if "general.alignment" in f.metadata else 32
    if alignment == 0:
        raise ParseError("general.alignment is zero or not an unsigned integer")
    f.data_offset = (r.pos + alignment - 1) // alignment * alignment
    return f


def tensor_bytes(buf, f, info):  # ReadTensorData (gguf.go:594-620)
    at = f.data_offset + info.offset
    n = info.num_bytes()
    if at + n > len(buf):
        raise ParseError("tensor %s lies outside the file" % info.name)
    return bytes(buf[at:at + n])


# pkg/gguf/loader.go:121-228, LLaMA-family names
_GLOBAL = {"model.embed_tokens.weight": "token_embd.weight", "lm_head.weight": "output.weight",
           "model.norm.weight": "output_norm.weight", "model.norm.bias": "output_norm.bias"}
_SUFFIX = {"self_attn.q_proj.weight": "attn_q.weight", "self_attn.k_proj.weight": "attn_k.weight",
           "self_attn.v_proj.weight": "attn_v.weight", "self_attn.q_proj.bias": "attn_q.bias",
           "self_attn.k_proj.bias": "attn_k.bias", "self_attn.v_proj.bias": "attn_v.bias",
           "self_attn.o_proj.weight": "attn_output.weight", "self_attn.o_proj.bias": "attn_output.bias",
           "mlp.gate_proj.weight": "ffn_gate.weight", "mlp.up_proj.weight": "ffn_up.weight",
           "mlp.down_proj.weight": "ffn_down.weight", "input_layernorm.weight": "attn_norm.weight",
           "input_layernorm.bias": "attn_norm.bias", "post_attention_layernorm.weight": "ffn_norm.weight",
           "post_attention_layernorm.bias": "ffn_norm.bias"}


def layer_tensor_name(hf_name):
    if not hf_name.startswith("model.layers."):
        return _GLOBAL.get(hf_name, hf_name)
    parts = hf_name.split(".")
    if len(parts) < 4:
        return hf_name
    suffix = ".".join(parts[3:])
    return "blk.%s.%s" % (parts[2], _SUFFIX[suffix]) if suffix in _SUFFIX else hf_name


# ---- writer (no counterpart in the reference)
def _w_string(out, s):
    b = s.encode("utf-8", errors="surrogateescape")
    out += struct.pack("<Q", len(b)) + b


def _w_scalar(out, t, v):
    if t == MT_STRING:
        _w_string(out, v)
    else:
        out += struct.pack(_SCALAR[t], int(v) if t == MT_BOOL else v)


def build(metadata, tensors, version=3, alignment=None, pad_byte=0):
    """metadata: list of (key, type, value) or (key, MT_ARRAY, (element type, values)); tensors: list of
    (name, dims in file order, type, bytes). Returns the file's bytes; tensor offsets are assigned in order, each
    aligned as llama.cpp writes them."""
    out = bytearray()
    out += struct.pack("<IIQQ", MAGIC, version, len(tensors), len(metadata))
    align = 32
    for key, t, v in metadata:
        _w_string(out, key)
        out += struct.pack("<I", t)
        if t == MT_ARRAY:
            et, vals = v
            out += struct.pack("<IQ", et, len(vals))
            for x in vals:
                _w_scalar(out, et, x)
        else:
            _w_scalar(out, t, v)
            if key == "general.alignment":
                align = v
    if alignment is not None:
        align = alignment
    offsets, off = [], 0
    for name, dims, t, data in tensors:
        offsets.append(off)
        off = (off + len(data) + align - 1) // align * align
    for (name, dims, t, data), o in zip(tensors, offsets):
        _w_string(out, name)
        out += struct.pack("<I", len(dims))
        for d in dims:
            out += struct.pack("<Q", d)
        out += struct.pack("<IQ", t, o)
    out += bytes([pad_byte]) * ((len(out) + align - 1) // align * align - len(out))
    base = len(out)
    for (name, dims, t, data), o in zip(tensors, offsets):
        out += bytes([pad_byte]) * (base + o - len(out))
        out += data
    return bytes(out)
