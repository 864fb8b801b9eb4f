"""The oracle against the known-answer tests the reference's own (untagged and
Metal-tagged) test files hold. Tables are transcribed by hand; each cites file:line."""
import math

import numpy as np
import pytest

from oracle import numerics as nx
from oracle import quantize as qz
from oracle import host_logic as hl


# ---- inference/pkg/gguf/dequant_test.go:9-36
@pytest.mark.parametrize("h,want", [(0x0000, 0.0), (0x3C00, 1.0), (0x4000, 2.0), (0x3800, 0.5),
                                    (0xBC00, -1.0), (0x7C00, math.inf), (0xFC00, -math.inf)])
def test_f16_table(h, want):
    assert nx.f16_to_f32(h) == want
    assert nx.f16_to_f32_cpu(h) == want


# ---- dequant_test.go:38-81
def test_q8_0_kat():
    data = np.zeros(34, dtype=np.uint8)
    data[0:2] = [0x00, 0x3C]
    data[2:] = np.arange(32)
    assert np.array_equal(nx.dequantize(nx.FMT_Q8_0, data, 32), np.arange(32, dtype=np.float32))
    data[0:2] = [0x00, 0x38]
    data[2:] = 2
    assert np.array_equal(nx.dequantize(nx.FMT_Q8_0, data, 32), np.ones(32, dtype=np.float32))


# ---- dequant_test.go:83-119 (nibble order)
def test_q4_0_kat():
    data = np.zeros(18, dtype=np.uint8)
    data[0:2] = [0x00, 0x3C]
    data[2] = 0x98
    data[3] = 0xBA
    r = nx.dequantize(nx.FMT_Q4_0, data, 32)
    assert r[0] == 0.0 and r[1] == 2.0 and r[16] == 1.0 and r[17] == 3.0
    # all other nibbles are 0 -> (0-8)*1
    assert r[2] == -8.0 and r[18] == -8.0


# ---- dequant_test.go:142-161
def test_bf16_kat():
    data = np.array([0x80, 0x3F, 0x00, 0x40], dtype=np.uint8)
    assert np.array_equal(nx.dequantize(nx.FMT_BF16, data, 2), np.array([1.0, 2.0], dtype=np.float32))


# ---- dequant_test.go:184-250 (all_zero, split_halves, with_scale)
def test_q5_0_kats():
    data = np.zeros(22, dtype=np.uint8)
    data[0:2] = [0x00, 0x3C]
    data[2:6] = 0xFF
    assert np.array_equal(nx.dequantize(nx.FMT_Q5_0, data, 32), np.zeros(32, dtype=np.float32))
    data[2:6] = [0x00, 0x00, 0xFF, 0xFF]
    data[6:22] = 0x88
    r = nx.dequantize(nx.FMT_Q5_0, data, 32)
    assert np.all(r[:16] == -8.0) and np.all(r[16:] == 8.0)
    data = np.zeros(22, dtype=np.uint8)
    data[0:2] = [0x00, 0x38]
    data[6] = 0x0F
    r = nx.dequantize(nx.FMT_Q5_0, data, 32)
    assert r[0] == -0.5 and r[16] == -8.0


# ---- dequant_test.go:307-320: a buffer too short for one block dequantises to zeros
def test_short_buffer_zeros():
    for fmt in (nx.FMT_Q4_0, nx.FMT_Q8_0, nx.FMT_Q4_K, nx.FMT_Q6_K, nx.FMT_Q5_0, nx.FMT_Q5_K):
        data = np.full(nx.BLOCK_BYTES[fmt] - 1, 0xFF, dtype=np.uint8)
        assert np.all(nx.dequantize(fmt, data, 32) == 0)
    data = np.full(100, 0x55, dtype=np.uint8)  # 100 bytes < 144
    assert np.all(nx.dequantize(nx.FMT_Q4_K, data, 32) == 0)


# ---- inference/backend/metal/q6k_kernel_test.go:153-180 (TestQ6_KDequantization):
# scales all 1, d = 1, values i%64-32 -> dequantised value == the integer
def test_q6_k_encoder_roundtrip_kat():
    vals = np.array([(i % 64) - 32 for i in range(256)], dtype=np.int8)
    blk = qz.encode_q6_k_block(1.0, np.ones(16, dtype=np.int8), vals)
    r = nx.dequantize(nx.FMT_Q6_K, blk, 256)
    assert np.array_equal(r, vals.astype(np.float32))


# ---- inference/backend/metal/q4_kernel_test.go:192-247: all-eights weights give exactly 0
def test_q4_0_all_eights_zero():
    k, n = 64, 4
    row = np.concatenate([qz.encode_q4_0_block(0.5, [8] * 32) for _ in range(k // 32)])
    w = np.tile(row, n)
    a = np.arange(k, dtype=np.float32) - 7
    assert np.all(nx.matmul_q4_0(a, w, 1, n, k) == 0)


# ---- inference/backend/metal/q8_0_matmul_test.go:83-130 style: ones x known rows
def test_q8_0_rows():
    k = 64
    rows = []
    for j in range(3):
        rows.append(np.concatenate([qz.encode_q8_0_block(0.25, [j + 1] * 32) for _ in range(k // 32)]))
    w = np.concatenate(rows)
    a = np.ones(k, dtype=np.float32)
    out = nx.matmul_quant(nx.FMT_Q8_0, a, w, 1, 3, k)
    assert np.array_equal(out[0], np.array([16.0, 32.0, 48.0], dtype=np.float32))


# ---- inference/backend/cpu/kernels_test.go:8-59
def test_matmul_2x3_3x2():
    a = [1, 2, 3, 4, 5, 6]
    b = [7, 8, 9, 1, 2, 3]
    assert np.array_equal(nx.matmul_f32(a, b, 2, 2, 3).ravel(), [31, 19, 85, 55])
    bt = np.array(b, dtype=np.float32).reshape(3, 2).T.copy()
    assert np.array_equal(nx.matmul_t_f32(a, bt, 2, 2, 3).ravel(), [31, 19, 85, 55])


# ---- inference/backend/cpu/rmsnorm_test.go:8-43
def test_rmsnorm_kat():
    out = nx.rmsnorm([1, 2, 3, 4, 2, 2, 2, 2], [1, 1, 1, 1], 2, 4, 1e-5)
    assert abs(out[0, 0] - 1.0 / 2.73861278) < 1e-4
    assert abs(out[0, 3] - 4.0 / 2.73861278) < 1e-4
    assert abs(out[1, 0] - 1.0) < 1e-4


# ---- inference/backend/cpu/softmax_test.go:8-34
def test_softmax_kat():
    out = nx.softmax([1.0, 2.0, 3.0], 1, 3)[0]
    for g, w in zip(out, [0.09003, 0.24473, 0.66524]):
        assert abs(g - w) < 1e-4


# ---- inference/backend/cpu/silu_test.go:9-40
def test_silu_kat():
    out = nx.silu([-1, 0, 1])
    want = [-1.0 / (1.0 + math.exp(1.0)), 0.0, 1.0 / (1.0 + math.exp(-1.0))]
    for g, w in zip(out, want):
        assert abs(g - w) < 1e-4
    out2 = nx.silu_mul([-1, 0, 1], [2, 2, 2])
    for g, w in zip(out2, want):
        assert abs(g - 2 * w) < 2e-4


# ---- inference/backend/cpu/embed_test.go:8-45
def test_embedding_kat():
    out = nx.embedding([0, 2], [1, 1, 2, 2, 3, 3], 3, 2)
    assert np.array_equal(out.ravel(), [1, 1, 3, 3])


# ---- cpu.go:549-552: out-of-range id leaves the row untouched
def test_embedding_oob_row_skipped():
    out = np.full((2, 2), 9.0, dtype=np.float32)
    nx.embedding([5, 1], [1, 1, 2, 2, 3, 3], 3, 2, out=out)
    assert np.array_equal(out.ravel(), [9, 9, 2, 2])


# ---- inference/backend/cpu/sdpa_test.go:19-125
def test_sdpa_kats():
    sc = np.float32(1.0 / math.sqrt(4.0))
    v = [0.5, 0.6, 0.7, 0.8]
    out = nx.sdpa([1, 0, 0, 0], [1, 0, 0, 0], v, 1, 1, 1, 4, sc, 4)
    assert np.allclose(out[0], v, atol=1e-5)
    out = nx.sdpa([1, 0, 0, 0], [1, 0, 0, 0, 0, 1, 0, 0], [1, 1, 1, 1, 0, 0, 0, 0], 2, 1, 1, 4, sc, 8)
    exp = math.exp(0.5) / (math.exp(0.5) + 1.0)
    assert np.allclose(out[0], exp, atol=1e-4)
    v = [0.1, 0.2, 0.3, 0.4]
    out = nx.sdpa([1, 0, 0, 0, 0, 1, 0, 0], [1, 1, 0, 0], v, 1, 2, 1, 4, sc, 4)
    assert np.allclose(out[0], v, atol=1e-5) and np.allclose(out[1], v, atol=1e-5)
    sc2 = np.float32(1.0 / math.sqrt(2.0))
    out = nx.sdpa([1, 1], [1, 0, 0, 1, 1, 1], [1, 0, 0, 1, 0.5, 0.5], 3, 1, 1, 2, sc2, 6)
    assert np.all(out >= 0) and np.all(out <= 1)


# ---- inference/backend/cpu/rope_test.go:10-46
def test_rope_kats():
    q, _ = nx.rope([1, 0, 1, 0], None, 4, 1, 0, 1, 1, 0, 10000.0, False)
    assert not (q[0] == 1.0 and q[1] == 0.0)
    q, _ = nx.rope([1, 1, 0, 0], None, 4, 1, 0, 1, 1, 4, 10000.0, True)
    assert not (q[0] == 1.0 and q[2] == 0.0)
    q, _ = nx.rope([1, 0, 1, 0], None, 4, 1, 0, 1, 1, 2, 10000.0, False)
    assert q[2] == 1.0 and q[3] == 0.0
    assert not (q[0] == 1.0 and q[1] == 0.0)


# ---- inference/backend/cpu/rope_shift_test.go:9-90: RoPE(2) then shift 3 is RoPE(5); shift 0 is the identity;
# a shift changes several tokens at once
def test_rope_shift_kats():
    theta, hd, hk = 10000.0, 4, 2
    base = np.array([1, 2, 3, 4, 5, 6, 7, 8], dtype=np.float32)
    _, k5 = nx.rope(np.zeros(8, dtype=np.float32), base, hd, hk, hk, 1, 5, 0, theta, False)
    _, k2 = nx.rope(np.zeros(8, dtype=np.float32), base, hd, hk, hk, 1, 2, 0, theta, False)
    k23 = nx.rope_shift(k2, hd, hk, 1, 3, theta)
    assert np.max(np.abs(k5 - k23)) <= 1e-5
    assert np.array_equal(nx.rope_shift(base, hd, hk, 1, 0, theta), base)
    many = np.arange(1, 3 * hk * hd + 1, dtype=np.float32)
    moved = nx.rope_shift(many, hd, hk, 3, 10, theta)
    assert np.count_nonzero(moved != many) > 0
    # a shift is the rotation RoPE gives a one-token call at that position, for every token alike
    _, want = nx.rope_positions(np.zeros(3 * hk * hd, dtype=np.float32), many, hd, hk, hk, [10, 10, 10], 0, theta, False)
    assert np.array_equal(moved.view(np.uint32), want.reshape(-1).view(np.uint32))


# ---- test/golden/golden_test.go:267-319: position 0 is the identity
def test_rope_pos0_identity():
    rng = np.random.default_rng(1)
    x = rng.standard_normal(2 * 4 * 64).astype(np.float32)
    k = rng.standard_normal(2 * 2 * 64).astype(np.float32)
    q2, k2 = nx.rope(x[:4 * 64], k[:2 * 64], 64, 4, 2, 1, 0, 0, 10000.0, False)
    assert np.array_equal(q2, x[:4 * 64]) and np.array_equal(k2, k[:2 * 64])


# ---- test/golden data files: residual identities hold exactly in float32
def test_golden_residual_identities(golden_dir):
    import os
    d = os.path.join(golden_dir, "ref_activations")
    ld = lambda n: np.load(os.path.join(d, n + ".npy")).reshape(-1)
    prev = ld("embedding")
    for i in (0, 1):
        sa, mlp, out = ld("layer_%d.self_attn" % i), ld("layer_%d.mlp" % i), ld("layer_%d.output" % i)
        got = nx.add(nx.add(prev, sa), mlp)
        assert np.array_equal(got, out)
        prev = out
    assert np.array_equal(ld("layer_0.self_attn"), ld("layer_0.o_proj"))
    assert np.array_equal(ld("layer_0.mlp"), ld("layer_0.down_proj"))


# ---- inference/kv/paged_test.go:301-446 (TestTruncateSequence) replayed on the GPU-pool
# logic (same block arithmetic, gpu_block_pool.go:162-190)
def _fill(pool, sid, n):
    for pos in range(n):
        for layer in range(pool.num_layers):
            pool.store_kv_slots(layer, sid, pos, 1)


def test_truncate_sequence_kats():
    mk = lambda: hl.GPUBlockPool(2, 2, 4, 4, 20)
    p = mk(); p.create_sequence(1); _fill(p, 1, 3); p.truncate_sequence(1, 2)
    assert p.seqs[1].seq_len == 2 and len(p.seqs[1].block_tables[0]) == 1
    p = mk(); p.create_sequence(1)
    free0 = len(p.free_lists[0])
    _fill(p, 1, 10)
    assert len(p.seqs[1].block_tables[0]) == 3 and len(p.free_lists[0]) == free0 - 3
    p.truncate_sequence(1, 3)
    assert p.seqs[1].seq_len == 3 and len(p.seqs[1].block_tables[0]) == 1
    assert len(p.free_lists[0]) == free0 - 1
    p = mk(); p.create_sequence(1); _fill(p, 1, 5); p.truncate_sequence(1, 0)
    assert p.seqs[1].seq_len == 0 and len(p.seqs[1].block_tables[0]) == 0
    assert len(p.free_lists[0]) == 20 and len(p.free_lists[1]) == 20
    p = mk(); p.truncate_sequence(999, 5)  # no-op, no error
    p = mk(); p.create_sequence(1); _fill(p, 1, 3); p.truncate_sequence(1, 10)
    assert p.seqs[1].seq_len == 3


# ---- inference/scheduler/verification_test.go:352-402
@pytest.mark.parametrize("start,acc,want", [(10, 4, 15), (10, 0, 11), (10, 2, 13), (0, 3, 4)])
def test_cache_truncation_calculation(start, acc, want):
    assert hl.cache_len_after_verify(start, acc) == want


# ---- inference/medusa/tree_test.go:115-217
def _tree():
    hlg = [[3.0, 1.0, 0.0, 0.0], [0.0, 0.0, 2.0, 0.5]]
    return hl.build_candidate_tree(hlg, 2, 32)


def test_tree_paths_linearize_mask():
    t = _tree()
    assert t.num_nodes == 6
    paths = t.paths()
    assert paths[0][0] == [0, 2]                      # tree_test.go:109-112
    assert all(paths[i][1] <= paths[i - 1][1] for i in range(1, len(paths)))
    tokens, parent = t.linearize()
    assert tokens == [0, 1, 2, 3, 2, 3] and parent == [-1, -1, 0, 0, 1, 1]
    n = len(tokens)
    mask = hl.build_tree_attention_mask(n, parent)
    assert len(mask) == n * n
    for i in range(n):
        j = i
        while j >= 0:
            assert mask[i * n + j]
            j = parent[j]
    assert not mask[0 * n + 1] and not mask[1 * n + 0]


def test_tree_15_nodes_4x2():
    """benchmark config 5: 4 heads x top-2 capped at 15 nodes = 2+4+8+1."""
    toks = [[10, 11], [20, 21], [30, 31], [40, 41]]
    vals = [[2.0, 1.0]] * 4
    t = hl.build_candidate_tree_from_topk(toks, vals, 15)
    assert t.num_nodes == 15
    tokens, parent = t.linearize()
    depth = hl.tree_depths(parent)
    assert [depth.count(d) for d in range(4)] == [2, 4, 8, 1]


# ---- tree.go:211-238 / medusa_scheduler.go:934-977 agree on a linear path
def test_verify_path_rules():
    assert hl.verify_tree_path([5, 6, 7], [5, 6, 7, 9]) == (3, 9)      # all accepted + bonus
    assert hl.verify_tree_path([5, 6, 7], [5, 8, 7, 9]) == (1, 8)      # first rejection -> correction
    assert hl.verify_tree_path([5, 6, 7], [4, 6, 7, 9]) == (0, 4)
    assert hl.select_best_tree_path([5, 6, 7], [5, 6, 7, 9]) == (0, 3, 9)
    assert hl.select_best_tree_path([5, 6, 7], [5, 8, 7, 9]) == (0, 1, 8)
    assert hl.select_best_tree_path([5, 6, 7], [4, 6, 7, 9]) == (0, 0, 4)


# ---- sampler.go:80-91
def test_argmax_rules():
    assert nx.argmax([1, 3, 3, 2]) == 1                 # first strict max
    assert nx.argmax([float("nan"), 1, 2]) == 2         # NaN never wins
    assert nx.argmax([float("-inf")] * 4) == 0
    assert hl.argmax_list([1, 3, 3, 2]) == 1
