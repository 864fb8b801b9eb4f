"""Whole-tree speculative verification in the oracle, pinned against the reference's own linear verification:
every root-to-node path of the tree must see exactly what VerifySpeculativeWithPagedKV (decode.go:1446-1569)
shows on [input token, path tokens], and after acceptance and rollback (medusa_scheduler.go:852-861) the pool
must be what a plain prefill of the accepted tokens leaves."""
import copy

import numpy as np

from oracle import host_logic as hl
from oracle import model as om
from oracle import numerics as nx

CFG = om.ModelConfig(num_layers=2, hidden=256, num_heads=4, num_kv_heads=2, head_dim=64, ffn=512, vocab=512)


def _model(seed=5):
    m = om.random_model(CFG, seed, nx.FMT_Q4_0, nx.FMT_Q8_0, max_blocks=16)
    rng = np.random.default_rng(seed + 1)
    prompt = rng.integers(0, CFG.vocab, 21).tolist()          # ends inside a block
    m.prefill_with_paged_kv(prompt, 7, 0)
    return m, rng


def _tree(rng, heads=4, top_k=2, max_nodes=15, plant=None):
    toks = [rng.choice(CFG.vocab, top_k, replace=False).tolist() for _ in range(heads)]
    if plant:
        for h, t in enumerate(plant[:heads]):
            toks[h][h % top_k] = t                             # not always the first child
            if toks[h][0] == toks[h][1]:
                toks[h][(h + 1) % top_k] = (t + 1) % CFG.vocab
    vals = [[2.0, 1.0]] * heads
    tree = hl.build_candidate_tree_from_topk(toks, vals, max_nodes)
    return tree.linearize()


def _path(parent_idx, node):
    p = []
    while node >= 0:
        p.append(node)
        node = parent_idx[node]
    return p[::-1]


def test_chain_tree_is_linear_verification():
    m, rng = _model()
    m2 = copy.deepcopy(m)
    draft = rng.integers(0, CFG.vocab, 5).tolist()
    want = m2.verify_with_paged_kv([3] + draft, 7, 21)
    got = m.verify_tree(3, draft, [-1, 0, 1, 2, 3], 7, 21)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    for layer in range(CFG.num_layers):
        assert np.array_equal(m.kv[layer], m2.kv[layer])
    assert m.pool.seqs[7].block_tables == m2.pool.seqs[7].block_tables


def test_every_path_of_a_tree_sees_its_linear_verification():
    m, rng = _model()
    base = copy.deepcopy(m)
    tokens, parent = _tree(rng)
    assert len(tokens) == 15 and parent[:2] == [-1, -1]
    logits = m.verify_tree(9, tokens, parent, 7, 21)
    assert logits.shape == (16, CFG.vocab)
    leaves = [i for i in range(15) if i not in parent]
    for leaf in leaves:
        path = _path(parent, leaf)
        lin = copy.deepcopy(base).verify_with_paged_kv([9] + [tokens[i] for i in path], 7, 21)
        for j, row in enumerate([0] + [i + 1 for i in path]):
            assert np.array_equal(logits[row].view(np.uint32), lin[j].view(np.uint32)), (leaf, j)


def test_tree_step_accepts_greedily_and_rolls_back_to_the_prefill_state():
    m, rng = _model()
    base = copy.deepcopy(m)
    # the model's own greedy continuation of token 9, planted down one branch of the tree for 3 levels
    probe = copy.deepcopy(base)
    greedy, tok = [], 9
    for i in range(4):
        tok = nx.argmax(probe.decode_with_paged_kv(tok, 7, 21 + i))
        greedy.append(tok)
    tokens, parent = _tree(rng, plant=greedy[:3])
    accepted, final, _ = m.tree_step(9, tokens, parent, 7, 21)
    assert [tokens[i] for i in accepted] == greedy[:3]
    assert final == greedy[3]
    assert accepted != [0, 1, 2]                               # the rollback had rows to move
    want = copy.deepcopy(base)
    want.prefill_with_paged_kv([9] + greedy[:3], 7, 21)
    st, wt = m.pool.seqs[7], want.pool.seqs[7]
    assert st.seq_len == wt.seq_len == 21 + 1 + 3
    assert st.block_tables == wt.block_tables
    assert m.pool.free_lists == want.pool.free_lists
    # the live K/V rows hold the same bits; the next decode step therefore gives the same logits
    a = m.decode_with_paged_kv(final, 7, 25)
    b = want.decode_with_paged_kv(final, 7, 25)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_tree_step_with_nothing_accepted_keeps_only_the_input_token():
    m, rng = _model()
    base = copy.deepcopy(m)
    tokens, parent = _tree(rng)
    root_next = nx.argmax(copy.deepcopy(base).decode_with_paged_kv(9, 7, 21))
    tokens = [t if t != root_next else (t + 1) % CFG.vocab for t in tokens]
    free_before = [len(f) for f in m.pool.free_lists]
    accepted, final, _ = m.tree_step(9, tokens, parent, 7, 21)
    assert accepted == [] and final == root_next
    assert m.pool.seqs[7].seq_len == 22
    # 21 + 16 rows needed a third block; the rollback gives it back
    assert [len(f) for f in m.pool.free_lists] == free_before
    want = copy.deepcopy(base)
    want.prefill_with_paged_kv([9], 7, 21)
    assert m.pool.seqs[7].block_tables == want.pool.seqs[7].block_tables


def _arch_cfg(name):
    import math
    if name == "phi":     # LayerNorm, biases, partial split-pair RoPE, GELU MLP, parallel residual
        return om.ModelConfig(num_layers=2, hidden=256, num_heads=4, num_kv_heads=4, head_dim=64, ffn=512, vocab=512,
                              norm_type="layer", mlp_type="gelu", parallel_residual=True, rope_dim=32, rope_neox=True)
    if name == "gemma":   # scaled embeddings, GeGLU, post-norms, soft-capped first chunk
        return om.ModelConfig(num_layers=2, hidden=256, num_heads=4, num_kv_heads=2, head_dim=64, ffn=512, vocab=512,
                              eps=1e-6, mlp_type="geglu", post_norms=True, attn_softcap=50.0,
                              embedding_scale=float(np.float32(math.sqrt(256.0))))
    return om.ModelConfig(num_layers=2, hidden=256, num_heads=4, num_kv_heads=2, head_dim=64, ffn=512, vocab=512,
                          eps=1e-6, rope_neox=True, rope_theta=1000000.0)   # Qwen 2: split pairs, Q/K/V biases below


def test_every_path_sees_its_linear_verification_in_the_other_architectures():
    """The same property under ExecuteWithPagedKV's switches (block.go:834-1077): the tree pass takes the layer's
    multi-query arm row by row, so each path must still equal the linear verification bit for bit."""
    for name in ("phi", "gemma", "qwen"):
        cfg = _arch_cfg(name)
        m = om.random_model(cfg, 15, nx.FMT_Q4_0, nx.FMT_Q8_0, max_blocks=16)
        rng = np.random.default_rng(16)
        if name == "qwen":
            for lw in m.layers:
                lw.wq_bias = (0.05 * rng.standard_normal(256)).astype(np.float32)
                lw.wk_bias = (0.05 * rng.standard_normal(128)).astype(np.float32)
                lw.wv_bias = (0.05 * rng.standard_normal(128)).astype(np.float32)
        m.prefill_with_paged_kv(rng.integers(0, cfg.vocab, 21).tolist(), 7, 0)
        base = copy.deepcopy(m)
        tokens, parent = _tree(rng, max_nodes=10)
        logits = m.verify_tree(9, tokens, parent, 7, 21)
        leaves = [i for i in range(len(tokens)) if i not in parent]
        for leaf in leaves:
            path = _path(parent, leaf)
            lin = copy.deepcopy(base).verify_with_paged_kv([9] + [tokens[i] for i in path], 7, 21)
            for j, row in enumerate([0] + [i + 1 for i in path]):
                assert np.array_equal(logits[row].view(np.uint32), lin[j].view(np.uint32)), (name, leaf, j)
