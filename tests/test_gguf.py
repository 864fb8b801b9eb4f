"""GGUF reader: the oracle restatement (oracle/gguf.py) against the reference's own test vectors, then the C++
reader of libvexel_host.so against the oracle on generated files. No GPU is touched here; the GPU-side loader
test lives in test_gpu_model.py."""
import os
import struct

import numpy as np
import pytest

from oracle import gguf as og


def _s(s):
    b = s.encode()
    return struct.pack("<Q", len(b)) + b


def _minimal_file():
    """The bytes TestParseMinimalGGUF writes (pkg/gguf/gguf_test.go:109-139)."""
    buf = struct.pack("<IIQQ", og.MAGIC, 3, 1, 2)
    buf += _s("general.architecture") + struct.pack("<I", og.MT_STRING) + _s("llama")
    buf += _s("llama.block_count") + struct.pack("<II", og.MT_U32, 22)
    buf += _s("model.embed_tokens.weight") + struct.pack("<IQQIQ", 2, 32000, 2048, og.T_F32, 0)
    return buf


# ---------------------------------------------------------------- oracle vs the reference's vectors
def test_oracle_parses_the_reference_minimal_file():
    f = og.parse(_minimal_file())                      # gguf_test.go:141-182
    assert f.version == 3
    assert f.metadata["general.architecture"].as_string() == "llama"
    assert f.metadata["llama.block_count"].as_uint32() == 22
    assert len(f.tensors) == 1 and f.tensors[0].name == "model.embed_tokens.weight"
    assert f.tensors[0].num_elements() == 32000 * 2048
    c = f.config()
    assert c["architecture"] == "llama" and c["num_layers"] == 22
    assert f.data_offset == (len(_minimal_file()) + 31) // 32 * 32


def test_oracle_rejects_bad_magic_and_old_version():
    with pytest.raises(og.ParseError):                 # gguf_test.go:185-194
        og.parse(struct.pack("<I", 0x12345678))
    with pytest.raises(og.ParseError):                 # gguf_test.go:196-206
        og.parse(struct.pack("<II", og.MAGIC, 1))


def test_oracle_type_tables_and_accessors():
    # gguf_test.go:9-65
    for t, name in ((og.T_F32, "F32"), (og.T_F16, "F16"), (og.T_Q4_0, "Q4_0"), (og.T_Q8_0, "Q8_0"), (og.T_BF16, "BF16"),
                    (999, "Unknown(999)")):
        assert og.type_string(t) == name
    for t, bs in ((og.T_F32, 1), (og.T_F16, 1), (og.T_Q4_0, 32), (og.T_Q8_0, 32), (og.T_Q4_K, 256)):
        assert og.block_size(t) == bs
    for t, bb in ((og.T_F32, 4), (og.T_F16, 2), (og.T_Q4_0, 18), (og.T_Q8_0, 34), (og.T_Q4_K, 144)):
        assert og.bytes_per_block(t) == bb
    # gguf_test.go:67-85
    for dims, n in (([], 0), ([10], 10), ([10, 20], 200), ([10, 20, 30], 6000)):
        assert og.TensorInfo("t", dims, 0, 0).num_elements() == n
    # gguf_test.go:87-107
    assert og.MetaValue(og.MT_U32, 42).as_uint32() == 42
    assert og.MetaValue(og.MT_U64, 100).as_uint32() == 100
    assert og.MetaValue(og.MT_I32, 55).as_uint32() == 55
    assert og.MetaValue(og.MT_STRING, "test").as_uint32() == 0


NAMES = [  # loader_test.go:12-28
    ("model.embed_tokens.weight", "token_embd.weight"), ("lm_head.weight", "output.weight"),
    ("model.norm.weight", "output_norm.weight"),
    ("model.layers.0.self_attn.q_proj.weight", "blk.0.attn_q.weight"),
    ("model.layers.5.self_attn.k_proj.weight", "blk.5.attn_k.weight"),
    ("model.layers.21.self_attn.v_proj.weight", "blk.21.attn_v.weight"),
    ("model.layers.0.self_attn.o_proj.weight", "blk.0.attn_output.weight"),
    ("model.layers.0.mlp.gate_proj.weight", "blk.0.ffn_gate.weight"),
    ("model.layers.0.mlp.up_proj.weight", "blk.0.ffn_up.weight"),
    ("model.layers.0.mlp.down_proj.weight", "blk.0.ffn_down.weight"),
    ("model.layers.0.input_layernorm.weight", "blk.0.attn_norm.weight"),
    ("model.layers.0.post_attention_layernorm.weight", "blk.0.ffn_norm.weight"),
    ("unknown.tensor.name", "unknown.tensor.name"),
]


def test_name_mapping_oracle_and_library():
    from vexel_amd.gguf import layer_tensor_name
    for hf, want in NAMES:
        assert og.layer_tensor_name(hf) == want
        assert layer_tensor_name(hf) == want
    assert layer_tensor_name("model.layers.3.mlp.fc1.weight") == og.layer_tensor_name("model.layers.3.mlp.fc1.weight")


# ---------------------------------------------------------------- library vs oracle on generated files
def _compare(path, raw):
    from vexel_amd.gguf import GGUFFile
    want = og.parse(raw)
    with GGUFFile(path) as g:
        assert g.version == want.version and g.data_offset == want.data_offset
        assert g.metadata_keys() == want.keys
        for key, v in want.metadata.items():
            assert g.meta_type(key) == v.type
            assert g.meta_u32(key) == v.as_uint32()
            assert g.meta_u64(key) == v.as_uint64()
            got_f, want_f = np.float32(g.meta_f32(key)), np.float32(v.as_float32())
            assert got_f.view(np.uint32) == want_f.view(np.uint32)
            assert g.meta_str(key) == (v.value if v.type == og.MT_STRING else None)
            assert g.meta_array_len(key) == (len(v.value) if v.type == og.MT_ARRAY else -1)
        assert g.meta_type("no.such.key") == -1 and g.meta_u32("no.such.key") == 0
        ts = g.tensors()
        assert len(ts) == len(want.tensors)
        for got, w in zip(ts, want.tensors):
            assert (got["name"], got["dims"], got["type"], got["offset"], got["n_bytes"]) == \
                   (w.name, w.dims, w.type, w.offset, w.num_bytes())
            inside = want.data_offset + w.offset + w.num_bytes() <= len(raw)
            assert (got["data"] is not None) == inside
            if inside:
                assert got["data"] == og.tensor_bytes(raw, want, w)
            assert g.get_tensor(w.name)["name"] == w.name
        assert g.get_tensor("no.such.tensor") is None
        gc, wc = g.config(), want.config()
        for k, v in wc.items():
            if isinstance(v, float):
                assert np.float32(gc[k]).view(np.uint32) == np.float32(v).view(np.uint32), k
            else:
                assert gc[k] == v, k


def _rich(rng, version=3, alignment=None, arch="llama"):
    md = [("general.architecture", og.MT_STRING, arch), ("general.name", og.MT_STRING, "synthetic é"),
          (arch + ".block_count", og.MT_U32, 3), (arch + ".embedding_length", og.MT_U64, 512),
          (arch + ".attention.head_count", og.MT_I32, 8), (arch + ".feed_forward_length", og.MT_U32, 1024),
          (arch + ".context_length", og.MT_U32, 4096), (arch + ".rope.freq_base", og.MT_F32, 500000.0),
          (arch + ".attention.layer_norm_rms_epsilon", og.MT_F64, 1e-6), (arch + ".attention.key_length", og.MT_U32, 64),
          ("x.u8", og.MT_U8, 200), ("x.i8", og.MT_I8, -5), ("x.u16", og.MT_U16, 60000), ("x.i16", og.MT_I16, -300),
          ("x.i64", og.MT_I64, -(1 << 40)), ("x.u64big", og.MT_U64, (1 << 40) + 7), ("x.bool", og.MT_BOOL, True),
          ("tokenizer.ggml.tokens", og.MT_ARRAY, (og.MT_STRING, ["tok%d" % i for i in range(37)])),
          ("tokenizer.ggml.scores", og.MT_ARRAY, (og.MT_F32, [float(i) / 3 for i in range(37)])),
          ("tokenizer.ggml.token_type", og.MT_ARRAY, (og.MT_I32, list(range(37)))),
          ("x.empty", og.MT_ARRAY, (og.MT_U8, [])),
          (arch + ".block_count", og.MT_U32, 5)]          # a repeated key: the last value wins
    if alignment:
        md.append(("general.alignment", og.MT_U32, alignment))
    tensors = []
    for name, dims, t in (("token_embd.weight", [512, 37], og.T_F16), ("blk.0.attn_q.weight", [512, 512], og.T_Q4_0),
                          ("blk.0.attn_v.weight", [512, 128], og.T_Q6_K), ("blk.0.ffn_down.weight", [1024, 512], og.T_Q4_K),
                          ("blk.0.attn_norm.weight", [512], og.T_F32), ("odd.q8", [96, 3], og.T_Q8_0),
                          ("odd.q5k", [256, 2], og.T_Q5_K), ("odd.unknown", [64], 19), ("three.d", [4, 3, 2], og.T_F32)):
        info = og.TensorInfo(name, dims, t, 0)
        tensors.append((name, dims, t, rng.integers(0, 256, info.num_bytes(), dtype=np.uint8).tobytes()))
    return og.build(md, tensors, version=version)


@pytest.mark.parametrize("case", ["minimal", "rich", "v2", "align64", "mistral", "truncated data"])
def test_library_reader_matches_oracle(tmp_path, case):
    rng = np.random.default_rng(5)
    raw = {"minimal": _minimal_file, "rich": lambda: _rich(rng), "v2": lambda: _rich(rng, version=2),
           "align64": lambda: _rich(rng, alignment=64), "mistral": lambda: _rich(rng, arch="mistral"),
           "truncated data": lambda: _rich(rng)[:-1000]}[case]()
    path = os.path.join(tmp_path, "f.gguf")
    with open(path, "wb") as fh:
        fh.write(raw)
    _compare(path, raw)


@pytest.mark.parametrize("case", ["bad magic", "version 1", "truncated header", "long string", "nested array",
                                  "unknown metadata type", "zero alignment"])
def test_library_reader_rejects_what_the_oracle_rejects(tmp_path, case):
    from vexel_amd.backend import VexelError
    from vexel_amd.gguf import GGUFFile
    good = _rich(np.random.default_rng(6))
    raw = {
        "bad magic": struct.pack("<I", 0x12345678) + good[4:],
        "version 1": good[:4] + struct.pack("<I", 1) + good[8:],
        "truncated header": good[:200],
        "long string": struct.pack("<IIQQ", og.MAGIC, 3, 0, 1) + struct.pack("<Q", 70000) + b"k" * 70000,
        "nested array": struct.pack("<IIQQ", og.MAGIC, 3, 0, 1) + _s("a") + struct.pack("<IIQ", og.MT_ARRAY, og.MT_ARRAY, 1),
        "unknown metadata type": struct.pack("<IIQQ", og.MAGIC, 3, 0, 1) + _s("a") + struct.pack("<I", 77),
        "zero alignment": struct.pack("<IIQQ", og.MAGIC, 3, 0, 1) + _s("general.alignment") + struct.pack("<II", og.MT_U32, 0),
    }[case]
    with pytest.raises(og.ParseError):
        og.parse(raw)
    path = os.path.join(tmp_path, "bad.gguf")
    with open(path, "wb") as fh:
        fh.write(raw)
    with pytest.raises(VexelError):
        GGUFFile(path)
