"""End-to-end parity of the decode drivers against the CPU oracle on identical seeded
random-init weights and inputs (the benchmark configs at sizes the oracle finishes in seconds:
real head geometry and hidden sizes, fewer layers).

Bars (the benchmark's north star): logits within 1e-2 absolute / 1e-3 relative in float32; greedy
tokens identical; block tables / slot state bit-exact."""
import numpy as np
import pytest

from oracle import model as om
from oracle import numerics as nx

from helpers import gpu_model_from_oracle, install_context, assert_logits_close

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def be():
    from vexel_amd.backend import HipBackend
    b = HipBackend(0)
    yield b
    b.close()


def _greedy_margin(logits):
    s = np.sort(logits)
    return float(s[-1] - s[-2])


def test_c1_prefill_then_greedy_decode(be):
    """benchmark config 1 shape (TinyLlama head geometry, Q4_0, Q8_0 embeddings and head), batch 1:
    32-token prompt, greedy decode of 64 tokens. 2 layers so the CPU side stays in seconds."""
    cfg = om.ModelConfig(num_layers=2, hidden=2048, num_heads=32, num_kv_heads=4, head_dim=64, ffn=5632,
                         vocab=32000, eps=1e-5, rope_theta=10000.0)
    omodel = om.random_model(cfg, 0, nx.FMT_Q4_0, nx.FMT_Q8_0, max_blocks=16)
    mr = gpu_model_from_oracle(be, omodel, pool_blocks=16, max_batch=8)
    rng = np.random.default_rng(0)
    prompt = rng.integers(0, cfg.vocab, 32).tolist()
    want = omodel.prefill_with_paged_kv(prompt, 1, 0)
    got = mr.prefill_with_paged_kv(prompt, 1, 0)
    worst = assert_logits_close(got, want, "prefill logits")
    tok_o, tok_g = nx.argmax(want), int(np.argmax(got))
    assert tok_o == tok_g
    pos = len(prompt)
    min_margin = 1e9
    for step in range(64):
        want = omodel.decode_with_paged_kv(tok_o, 1, pos)
        got, am = mr.decode_with_paged_kv_batched([tok_g], [1], [pos])
        worst = max(worst, assert_logits_close(got[0], want, "decode step %d" % step))
        min_margin = min(min_margin, _greedy_margin(want))
        tok_o = nx.argmax(want)
        tok_g = int(am[0])
        assert tok_o == tok_g, "greedy token differs at step %d (margin %.3e)" % (step, _greedy_margin(want))
        pos += 1
    assert mr.block_table(1) == omodel.pool.seqs[1].block_tables[0]
    assert mr.seq_len(1) == omodel.pool.seqs[1].seq_len == 96
    print("C1: worst logit error %.3e, smallest top-1 margin %.3e" % (worst, min_margin))
    mr.close()


def _ragged_setup(be, cfg, fmt, head_fmt, ctx_lens, seed, pool_blocks, fmt_overrides=None, max_blocks_per_seq=None):
    omodel = om.random_model(cfg, seed, fmt, head_fmt, max_blocks=pool_blocks, fmt_overrides=fmt_overrides)
    mr = gpu_model_from_oracle(be, omodel, pool_blocks=pool_blocks, max_seqs=len(ctx_lens) + 2,
                               max_blocks_per_seq=max_blocks_per_seq or max(ctx_lens) // cfg.block_size + 8,
                               max_batch=len(ctx_lens))
    rng = np.random.default_rng(seed + 1)
    perm = rng.permutation(pool_blocks)       # block tables are a seeded random permutation
    off = 0
    for i, L in enumerate(ctx_lens):
        nb = (L + cfg.block_size - 1) // cfg.block_size
        install_context(omodel, mr, be, 100 + i, perm[off:off + nb], L, rng)
        off += nb
    return omodel, mr, rng


def test_c2_batched_decode_ragged_paged(be):
    """benchmark config 2 shape: 8 sequences, ragged contexts, KV pre-filled with N(0,1), permuted block
    tables; batched decode steps against the oracle's sequential per-sequence loop."""
    cfg = om.ModelConfig(num_layers=2, hidden=2048, num_heads=32, num_kv_heads=4, head_dim=64, ffn=5632,
                         vocab=32000)
    rng0 = np.random.default_rng(5)
    ctx = [int(x) for x in rng0.integers(128, 700, 8)]
    ctx[3] = 16 * 9            # exactly on a block boundary: the step must take a new block
    omodel, mr, rng = _ragged_setup(be, cfg, nx.FMT_Q4_0, nx.FMT_Q8_0, ctx, 7, pool_blocks=400)
    ids = [100 + i for i in range(8)]
    toks = rng.integers(0, cfg.vocab, 8).tolist()
    pos = list(ctx)
    toks_g = list(toks)
    for step in range(4):
        want = omodel.decode_batched(toks, ids, pos)
        got, am = mr.decode_with_paged_kv_batched(toks_g, ids, pos)
        assert_logits_close(got, want, "C2 step %d" % step)
        toks = [nx.argmax(want[i]) for i in range(8)]
        toks_g = [int(a) for a in am]
        assert toks == toks_g
        pos = [p + 1 for p in pos]
    for i, sid in enumerate(ids):
        assert mr.block_table(sid) == omodel.pool.seqs[sid].block_tables[0]
        assert mr.block_table(sid) == omodel.pool.seqs[sid].block_tables[cfg.num_layers - 1]
    assert mr.block_stats()[1] == omodel.pool.block_stats()[1]
    mr.close()


def test_fused_and_unfused_runtime_give_identical_logits(be):
    """The runtime's fused decode blocks and its one-call-per-operation sequence are the same function up
    to the float32 summation order of the split-K slices: logits within 1e-3, same greedy tokens, over
    several steps of a ragged batch (33 rows: more than one 16-row tile and a partial one)."""
    cfg = om.ModelConfig(num_layers=3, hidden=1024, num_heads=16, num_kv_heads=4, head_dim=64, ffn=2816,
                         vocab=4096)
    rng0 = np.random.default_rng(21)
    ctx = [int(x) for x in rng0.integers(5, 300, 33)]
    runs = []
    for fused in (True, False):
        omodel, mr, rng = _ragged_setup(be, cfg, nx.FMT_Q4_0, nx.FMT_Q8_0, ctx, 23, pool_blocks=700)
        mr.set_fused(fused)
        ids = [100 + i for i in range(len(ctx))]
        toks, pos, logs = rng.integers(0, cfg.vocab, len(ctx)).tolist(), list(ctx), []
        for step in range(3):
            got, am = mr.decode_with_paged_kv_batched(toks, ids, pos)
            logs.append((got.copy(), [int(a) for a in am]))
            toks, pos = [int(a) for a in am], [p + 1 for p in pos]
        runs.append(logs)
        mr.close()
    for (a, ta), (b, tb) in zip(*runs):
        assert np.abs(a - b).max() <= 1e-3 * max(1.0, np.abs(b).max())
        assert ta == tb


def test_device_driven_graph_decode_matches_host_driven(be):
    """The hipGraph-captured, device-packed greedy loop gives the same tokens as the host-driven
    step and as the oracle, and leaves the device block tables equal to the host's."""
    cfg = om.ModelConfig(num_layers=2, hidden=1024, num_heads=8, num_kv_heads=8, head_dim=128, ffn=2816,
                         vocab=4096)
    ctx = [30, 47, 16, 200, 333, 64]
    steps = 20   # several sequences cross block boundaries
    omodel, mr, rng = _ragged_setup(be, cfg, nx.FMT_Q4_0, nx.FMT_Q4_0, ctx, 11, pool_blocks=120)
    ids = [100 + i for i in range(len(ctx))]
    first = rng.integers(0, cfg.vocab, len(ctx)).tolist()
    # oracle greedy loop
    toks, pos, want_tokens = list(first), list(ctx), []
    for s in range(steps):
        lg = omodel.decode_batched(toks, ids, pos)
        toks = [nx.argmax(lg[i]) for i in range(len(ctx))]
        want_tokens.append(list(toks))
        pos = [p + 1 for p in pos]
    out, ms = mr.decode_graph(first, ids, ctx, steps, use_graph=True)
    assert out.tolist() == want_tokens
    assert mr.device_matches_host()
    for sid in ids:
        assert mr.block_table(sid) == omodel.pool.seqs[sid].block_tables[0]
        assert mr.seq_len(sid) == omodel.pool.seqs[sid].seq_len
    # continue on the device without re-uploading anything: replays of the cached graph
    more, _ = mr.decode_graph(None, None, None, 5, use_graph=True, batch=len(ctx))
    for s in range(5):
        lg = omodel.decode_batched(toks, ids, pos)
        toks = [nx.argmax(lg[i]) for i in range(len(ctx))]
        assert more[s].tolist() == toks
        pos = [p + 1 for p in pos]
    assert mr.device_matches_host()
    # eager device-driven steps (no graph) agree too
    eager, _ = mr.decode_graph(None, None, None, 3, use_graph=False, batch=len(ctx))
    for s in range(3):
        lg = omodel.decode_batched(toks, ids, pos)
        toks = [nx.argmax(lg[i]) for i in range(len(ctx))]
        assert eager[s].tolist() == toks
        pos = [p + 1 for p in pos]
    mr.close()


def _greedy_oracle(omodel, toks, ids, pos, steps):
    toks, pos, out = list(toks), list(pos), []
    for _ in range(steps):
        lg = omodel.decode_batched(toks, ids, pos)
        toks = [nx.argmax(lg[i]) for i in range(len(ids))]
        out.append(list(toks))
        pos = [p + 1 for p in pos]
    return out, toks, pos


def test_graph_decode_after_the_scratch_buffers_moved():
    """A kept graph holds the library's scratch addresses. A prefill of more rows than the decode batch makes
    those buffers grow (and move); the next device-driven call must notice and record the step again instead of
    replaying the old graph over freed memory."""
    from vexel_amd.backend import HipBackend
    own = HipBackend(0)   # a backend of its own: its scratch is as small as this test's first calls leave it
    cfg = om.ModelConfig(num_layers=2, hidden=512, num_heads=8, num_kv_heads=2, head_dim=64, ffn=1024, vocab=1024)
    ctx = [20, 33, 50]
    omodel, mr, rng = _ragged_setup(own, cfg, nx.FMT_Q4_0, nx.FMT_Q8_0, ctx, 41, pool_blocks=96, max_blocks_per_seq=24)
    ids = [100 + i for i in range(3)]
    first = rng.integers(0, cfg.vocab, 3).tolist()
    want, toks, pos = _greedy_oracle(omodel, first, ids, ctx, 4)
    out, _ = mr.decode_graph(first, ids, ctx, 4, use_graph=True)
    assert out.tolist() == want
    gen = own.scratch_generation()
    # another request arrives: a 300-token prompt goes through the same library scratch
    prompt = rng.integers(0, cfg.vocab, 300).tolist()
    omodel.pool.create_sequence(7)
    mr.create_sequence(7)
    assert_logits_close(mr.prefill_with_paged_kv(prompt, 7, 0), omodel.prefill_with_paged_kv(prompt, 7, 0), "prefill between graphs")
    assert own.scratch_generation() > gen, "the prefill was meant to outgrow the decode batch's scratch"
    want2, toks, pos = _greedy_oracle(omodel, toks, ids, pos, 6)
    more, _ = mr.decode_graph(None, None, None, 6, use_graph=True, batch=3)
    assert more.tolist() == want2
    assert mr.device_matches_host()
    mr.close()
    own.close()


def test_device_driven_decode_refuses_steps_the_pool_cannot_hold(be):
    """More steps than the free blocks allow are refused before anything runs on the device: tables, free list and
    the K/V rows stay as they were, and a shorter run afterwards matches the oracle."""
    from vexel_amd.backend import VexelError
    cfg = om.ModelConfig(num_layers=2, hidden=512, num_heads=8, num_kv_heads=2, head_dim=64, ffn=1024, vocab=1024)
    ctx = [30, 47, 16]    # 2 + 3 + 1 blocks of the pool's 9: three are free
    omodel, mr, rng = _ragged_setup(be, cfg, nx.FMT_Q4_0, nx.FMT_Q8_0, ctx, 43, pool_blocks=9)
    ids = [100 + i for i in range(3)]
    first = rng.integers(0, cfg.vocab, 3).tolist()
    # 40 steps: sequence 0 would need 5 blocks (+3), sequence 1 six (+3), sequence 2 four (+3)
    with pytest.raises(VexelError, match="free blocks"):
        mr.decode_graph(first, ids, ctx, 40, use_graph=True)
    assert mr.device_matches_host()
    for sid, c in zip(ids, ctx):
        assert mr.seq_len(sid) == c
    # one sequence over its own limit
    with pytest.raises(VexelError, match="max_blocks_per_seq"):
        mr.decode_graph(first, ids, ctx, 16 * 20, use_graph=True)
    want, toks, pos = _greedy_oracle(omodel, first, ids, ctx, 6)   # within the three free blocks
    out, _ = mr.decode_graph(first, ids, ctx, 6, use_graph=True)
    assert out.tolist() == want
    assert mr.device_matches_host()
    # the batch on the device loses a sequence: continuing is refused, not a null dereference
    mr.delete_sequence(ids[1])
    with pytest.raises(VexelError, match="deleted"):
        mr.decode_graph(None, None, None, 1, use_graph=True, batch=3)
    mr.close()


@pytest.mark.parametrize("name,fmt,head,over", [
    ("q4_k_m mix", nx.FMT_Q4_K, nx.FMT_Q6_K, {"wv": nx.FMT_Q6_K, "w2": nx.FMT_Q6_K}),   # config 3
    ("q8_0", nx.FMT_Q8_0, nx.FMT_Q8_0, None),                                            # config 4
    ("q6_k", nx.FMT_Q6_K, nx.FMT_Q6_K, None),                                            # config 5
    ("q5_k_m mix", nx.FMT_Q5_K, nx.FMT_Q6_K, {"wv": nx.FMT_Q6_K, "w2": nx.FMT_Q6_K}),   # llama.cpp's Q5_K_M recipe
    ("q5_0", nx.FMT_Q5_0, nx.FMT_Q8_0, None),
])
def test_other_formats_batched_decode(be, name, fmt, head, over):
    """7B/8B head geometry (head_dim 128), one layer, 32 ragged sequences: the M=32 path."""
    kvh = 8 if fmt == nx.FMT_Q8_0 else 32
    cfg = om.ModelConfig(num_layers=1, hidden=4096, num_heads=32, num_kv_heads=kvh, head_dim=128, ffn=2048,
                         vocab=2048, rope_theta=500000.0 if fmt == nx.FMT_Q8_0 else 10000.0)
    rng0 = np.random.default_rng(21)
    ctx = [int(x) for x in np.clip(np.exp(rng0.normal(np.log(200), 0.6, 32)), 64, 600)]
    omodel, mr, rng = _ragged_setup(be, cfg, fmt, head, ctx, 23, pool_blocks=900, fmt_overrides=over)
    ids = [100 + i for i in range(32)]
    toks = rng.integers(0, cfg.vocab, 32).tolist()
    want = omodel.decode_batched(toks, ids, ctx)
    got, am = mr.decode_with_paged_kv_batched(toks, ids, ctx)
    assert_logits_close(got, want, name)
    assert [nx.argmax(want[i]) for i in range(32)] == [int(a) for a in am]
    mr.close()


def test_chunked_prefill_and_verify(be):
    """Second chunk (startPos > 0) goes through multi-query paged attention over the f16 pool
    (runtime/block.go:881-890); verify returns logits for every position."""
    cfg = om.ModelConfig(num_layers=2, hidden=1024, num_heads=8, num_kv_heads=2, head_dim=128, ffn=2048,
                         vocab=4096)
    omodel = om.random_model(cfg, 31, nx.FMT_Q8_0, nx.FMT_Q8_0, max_blocks=32)
    mr = gpu_model_from_oracle(be, omodel, pool_blocks=32, max_batch=4)
    rng = np.random.default_rng(32)
    toks = rng.integers(0, cfg.vocab, 70).tolist()
    w1 = omodel.prefill_with_paged_kv(toks[:40], 5, 0)
    g1 = mr.prefill_with_paged_kv(toks[:40], 5, 0)
    assert_logits_close(g1, w1, "chunk 0")
    w2 = omodel.prefill_with_paged_kv(toks[40:], 5, 40)
    g2 = mr.prefill_with_paged_kv(toks[40:], 5, 40)
    assert_logits_close(g2, w2, "chunk 1")
    draft = rng.integers(0, cfg.vocab, 5).tolist()
    wv = omodel.verify_with_paged_kv(draft, 5, 70)
    gv = mr.prefill_with_paged_kv(draft, 5, 70, all_logits=True)
    assert_logits_close(gv, wv, "verify")
    # rollback after 2 accepted drafts (medusa_scheduler.go:852-861)
    new_len = 70 + 1 + 2
    omodel.pool.truncate_sequence(5, new_len)
    mr.truncate_sequence(5, new_len)
    assert mr.seq_len(5) == omodel.pool.seqs[5].seq_len == new_len
    assert mr.block_table(5) == omodel.pool.seqs[5].block_tables[0]
    assert mr.block_stats()[1] == omodel.pool.block_stats()[1]
    mr.close()


@pytest.mark.parametrize("kv_heads,max_nodes", [(8, 15), (2, 10)])
def test_c5_tree_verification_batched(be, kv_heads, max_nodes):
    """benchmark config 5 at oracle size: Q6_K weights, several sequences at ragged contexts, a 15-node candidate
    tree (4 heads x top-2) per sequence verified in one pass under tree masks over the paged f16 pool, greedy
    acceptance, rollback in the block tables; two rounds, the second on top of the first one's rollback.
    Second case: grouped-query heads and 11-row trees, which do not fill the attention's entries of query rows."""
    import copy
    from oracle import host_logic as hl
    cfg = om.ModelConfig(num_layers=2, hidden=1024, num_heads=8, num_kv_heads=kv_heads, head_dim=128, ffn=2816,
                         vocab=4096)
    ctx = [291, 256, 517, 333]     # 256: the input token opens a new block
    omodel, mr, rng = _ragged_setup(be, cfg, nx.FMT_Q6_K, nx.FMT_Q6_K, ctx, 41, pool_blocks=160)
    if kv_heads == 2:
        mr.set_fused(False)        # the second case also takes the one-call-per-operation layer
    ids = [100 + i for i in range(4)]
    inputs = rng.integers(0, cfg.vocab, 4).tolist()
    start = list(ctx)
    moved = 0
    for rnd in range(2):
        trees = []
        for i, sid in enumerate(ids):
            # sequences 0 and 2 get their own greedy continuation planted down one branch (3 and 1 levels deep)
            plant = []
            if i in (0, 2):
                probe = copy.deepcopy(omodel)
                tok = inputs[i]
                for d in range(3 if i == 0 else 1):
                    tok = nx.argmax(probe.decode_with_paged_kv(tok, sid, start[i] + d))
                    plant.append(tok)
            toks = [rng.choice(cfg.vocab, 2, replace=False).tolist() for _ in range(4)]
            for h, t in enumerate(plant):
                toks[h][(h + 1) % 2] = t
                if toks[h][0] == toks[h][1]:
                    toks[h][h % 2] = (t + 1) % cfg.vocab
            tree = hl.build_candidate_tree_from_topk(toks, [[2.0, 1.0]] * 4, max_nodes)
            trees.append(tree.linearize())
        want = omodel.tree_step_batched(inputs, trees, ids, start)
        acc, fin, logits = mr.verify_tree(ids, inputs, start, trees)
        for i, sid in enumerate(ids):
            assert_logits_close(logits[i], want[i][2], "C5 round %d seq %d" % (rnd, i))
            assert acc[i] == want[i][0] and fin[i] == want[i][1]
            assert mr.seq_len(sid) == omodel.pool.seqs[sid].seq_len == start[i] + 1 + len(acc[i])
            assert mr.block_table(sid) == omodel.pool.seqs[sid].block_tables[0]
            moved += sum(1 for k, node in enumerate(acc[i]) if node != k)
        # (a 10-node tree stops inside its third level: the planted branch may end after two)
        assert len(acc[0]) >= (3 if max_nodes == 15 else 2) and len(acc[2]) >= 1
        assert mr.block_stats()[1] == omodel.pool.block_stats()[1]
        inputs = list(fin)
        start = [start[i] + 1 + len(acc[i]) for i in range(4)]
    assert moved > 0   # the rollback had rows to move
    # the compacted K/V rows serve an ordinary decode step
    wl = omodel.decode_batched(inputs, ids, start)
    gl, am = mr.decode_with_paged_kv_batched(inputs, ids, start)
    assert_logits_close(gl, wl, "C5 decode after rollback")
    assert [nx.argmax(wl[i]) for i in range(4)] == [int(a) for a in am]
    assert mr.device_matches_host()
    mr.close()


GGUF_TYPE = {nx.FMT_Q4_0: 2, nx.FMT_Q8_0: 8, nx.FMT_Q4_K: 12, nx.FMT_Q6_K: 14, nx.FMT_Q5_0: 6, nx.FMT_Q5_K: 13,
             nx.FMT_BF16: 30}


@pytest.mark.parametrize("case", ["q4_k_m mix with output", "tied q8_0 embedding", "tied f16 embedding, q4_0",
                                  "q5_k mix with q5_0 and bf16, tied q5_0 embedding"])
def test_load_gguf_checkpoint(be, tmp_path, case):
    """A checkpoint written as a GGUF file (oracle/gguf.py writer: llama.* metadata, llama.cpp tensor names) and read
    back by the C++ loader gives the logits and greedy tokens of the oracle model built from the same tensors:
    raw quantized projection matrices and head, token_embd and norms converted to float32 (from a quantized type,
    F16 and F32), a missing output.weight tied to the embedding (runtime/loader.go:28-212, 596-600)."""
    import os
    from oracle import gguf as og
    from oracle import quantize as qz
    from vexel_amd.runtime import ModelRuntime
    rng = np.random.default_rng(55)
    cfg = om.ModelConfig(num_layers=2, hidden=512, num_heads=8, num_kv_heads=2, head_dim=64, ffn=1024, vocab=768,
                         eps=1e-6, rope_theta=500000.0)
    fmt = nx.FMT_Q4_0 if "q4_0" in case else nx.FMT_Q5_K if "q5_k" in case else nx.FMT_Q4_K
    over = {"wv": nx.FMT_Q6_K, "w2": nx.FMT_Q6_K} if "mix" in case else {}
    if "q5_k" in case:
        over = {"wv": nx.FMT_Q5_0, "wo": nx.FMT_BF16, "w2": nx.FMT_Q5_0}
    qd, kvd = cfg.num_heads * cfg.head_dim, cfg.num_kv_heads * cfg.head_dim
    tensors, layers = [], []
    f16 = lambda a: nx.f16_to_f32_array(nx.f32_to_f16_array(a.astype(np.float32)))
    for l in range(cfg.num_layers):
        ws = {}
        for name, gname, n, k in (("wq", "attn_q", qd, cfg.hidden), ("wk", "attn_k", kvd, cfg.hidden),
                                  ("wv", "attn_v", kvd, cfg.hidden), ("wo", "attn_output", cfg.hidden, qd),
                                  ("w1", "ffn_gate", cfg.ffn, cfg.hidden), ("w3", "ffn_up", cfg.ffn, cfg.hidden),
                                  ("w2", "ffn_down", cfg.hidden, cfg.ffn)):
            f = over.get(name, fmt)
            data = qz.random_quant(f, rng, n, k)
            ws[name] = om.QWeight(f, data, n, k)
            tensors.append(("blk.%d.%s.weight" % (l, gname), [k, n], GGUF_TYPE[f], data.tobytes()))
        an = (1 + 0.1 * rng.standard_normal(cfg.hidden)).astype(np.float32)
        fn = f16(1 + 0.1 * rng.standard_normal(cfg.hidden))          # stored as F16 in the file
        tensors.append(("blk.%d.attn_norm.weight" % l, [cfg.hidden], og.T_F32, an.tobytes()))
        tensors.append(("blk.%d.ffn_norm.weight" % l, [cfg.hidden], og.T_F16, nx.f32_to_f16_array(fn).tobytes()))
        layers.append(om.LayerWeights(attn_norm=an, ffn_norm=fn, **ws))
    final_norm = (1 + 0.1 * rng.standard_normal(cfg.hidden)).astype(np.float32)
    tensors.append(("output_norm.weight", [cfg.hidden], og.T_F32, final_norm.tobytes()))
    if "f16 embedding" in case:
        emb = f16(0.05 * rng.standard_normal((cfg.vocab, cfg.hidden)))
        tensors.append(("token_embd.weight", [cfg.hidden, cfg.vocab], og.T_F16, nx.f32_to_f16_array(emb.reshape(-1)).tobytes()))
        head = om.QWeight(0, emb, cfg.vocab, cfg.hidden)               # tied, float32
    else:
        ef = nx.FMT_Q8_0 if "q8_0" in case else nx.FMT_Q5_0 if "q5_0 embedding" in case else nx.FMT_Q4_0
        eq = qz.random_quant(ef, rng, cfg.vocab, cfg.hidden)
        emb = nx.dequantize(ef, eq, cfg.vocab * cfg.hidden).reshape(cfg.vocab, cfg.hidden)
        tensors.append(("token_embd.weight", [cfg.hidden, cfg.vocab], GGUF_TYPE[ef], eq.tobytes()))
        if "tied" in case:
            head = om.QWeight(ef, eq, cfg.vocab, cfg.hidden)           # tied, raw blocks
        else:
            hq = qz.random_quant(nx.FMT_Q6_K, rng, cfg.vocab, cfg.hidden)
            tensors.append(("output.weight", [cfg.hidden, cfg.vocab], GGUF_TYPE[nx.FMT_Q6_K], hq.tobytes()))
            head = om.QWeight(nx.FMT_Q6_K, hq, cfg.vocab, cfg.hidden)
    md = [("general.architecture", og.MT_STRING, "llama"), ("llama.block_count", og.MT_U32, cfg.num_layers),
          ("llama.embedding_length", og.MT_U32, cfg.hidden), ("llama.attention.head_count", og.MT_U32, cfg.num_heads),
          ("llama.attention.head_count_kv", og.MT_U32, cfg.num_kv_heads), ("llama.feed_forward_length", og.MT_U32, cfg.ffn),
          ("llama.context_length", og.MT_U32, 2048), ("llama.rope.freq_base", og.MT_F32, cfg.rope_theta),
          ("llama.attention.layer_norm_rms_epsilon", og.MT_F32, cfg.eps),
          ("tokenizer.ggml.tokens", og.MT_ARRAY, (og.MT_STRING, ["t%d" % i for i in range(cfg.vocab)]))]
    rng.shuffle(tensors)                                               # file order is not the loader's order
    path = os.path.join(tmp_path, "model.gguf")
    with open(path, "wb") as fh:
        fh.write(og.build(md, [tuple(t) for t in tensors]))
    omodel = om.OracleModel(cfg, emb, layers, final_norm, head, max_blocks=16)
    mr = ModelRuntime.from_gguf(be, path, pool_blocks=16, max_seqs=4, max_batch=48)
    c = mr.cfg
    assert (c.num_layers, c.hidden, c.num_heads, c.num_kv_heads, c.head_dim, c.ffn, c.vocab) == \
           (cfg.num_layers, cfg.hidden, cfg.num_heads, cfg.num_kv_heads, cfg.head_dim, cfg.ffn, cfg.vocab)
    assert np.float32(c.eps) == np.float32(cfg.eps) and np.float32(c.rope_theta) == np.float32(cfg.rope_theta)
    prompt = rng.integers(0, cfg.vocab, 40).tolist()
    want = omodel.prefill_with_paged_kv(prompt, 1, 0)
    got = mr.prefill_with_paged_kv(prompt, 1, 0)
    assert_logits_close(got, want, "prefill logits from the loaded checkpoint")
    tok, pos = nx.argmax(want), len(prompt)
    assert tok == int(np.argmax(got))
    for step in range(8):
        want = omodel.decode_with_paged_kv(tok, 1, pos)
        got, am = mr.decode_with_paged_kv_batched([tok], [1], [pos])
        assert_logits_close(got[0], want, "decode step %d" % step)
        tok = nx.argmax(want)
        assert tok == int(am[0])
        pos += 1
    mr.close()
    # a checkpoint the loader cannot take says why
    from vexel_amd.backend import VexelError
    bad = [t for t in tensors if t[0] != "blk.1.ffn_up.weight"]
    with open(path, "wb") as fh:
        fh.write(og.build(md, [tuple(t) for t in bad]))
    with pytest.raises(VexelError, match="ffn_up"):
        ModelRuntime.from_gguf(be, path, pool_blocks=16, max_seqs=4, max_batch=48)


@pytest.mark.parametrize("chunk", [0, 16])
def test_scheduler_loop_matches_oracle(be, chunk):
    """Continuous batching (scheduler/scheduler.go:166-483, sequence.go): six requests with prompts of 0 to 45 tokens
    join at different steps; at most four run per step; one stops on the EOS token, the others on their own or
    the scheduler's length limit; finished sequences are removed and their blocks return to the pool. After every
    step the C++ scheduler and its oracle restatement over the CPU model agree on every sequence's state, position
    and generated tokens; at the end on block tables and pool statistics. chunk = 16 feeds prompts in pieces.
    Two of the requests sample (temperature, top-k, top-p) from the same uniform stream on both sides."""
    from oracle import host_logic as hl
    from vexel_amd.runtime import Scheduler
    cfg = om.ModelConfig(num_layers=2, hidden=512, num_heads=8, num_kv_heads=2, head_dim=64, ffn=1024, vocab=1024)
    omodel = om.random_model(cfg, 71, nx.FMT_Q4_0, nx.FMT_Q8_0, max_blocks=48)
    mr = gpu_model_from_oracle(be, omodel, pool_blocks=48, max_seqs=8, max_blocks_per_seq=8, max_batch=48)
    rng = np.random.default_rng(72)
    prompts = {11: 45, 12: 0, 13: 7, 14: 33, 15: 16, 16: 1}
    prompts = {i: rng.integers(0, cfg.vocab, n).tolist() for i, n in prompts.items()}
    limits = {11: 9, 12: 0, 13: 5, 14: 0, 15: 12, 16: 3}
    arrivals = {0: [11, 12, 13], 2: [14, 15], 5: [16]}
    # the EOS token: what sequence 14 generates third in a dry run of the oracle (so that one request stops on it)
    dry_model = om.random_model(cfg, 71, nx.FMT_Q4_0, nx.FMT_Q8_0, max_blocks=48)
    dry = hl.Scheduler(dry_model, 4, 14, -1, chunk)
    dry.add_sequence(14, prompts[14])
    for _ in range(6):
        dry.step()
    eos = dry.seqs[14].generated[2]
    want = hl.Scheduler(omodel, 4, 14, eos, chunk)
    got = Scheduler(mr, 4, max_tokens=14, eos_token=eos, prefill_chunk=chunk)
    finished_at = {}
    # two requests are sampled (in decode steps on the device, after their prompt on the host), the others greedy
    sampled = {13: (0.8, 20, 0.95, 1234), 15: (1.1, 0, 0.9, 99)}
    for step in range(40):
        for i in arrivals.get(step, []):
            want.add_sequence(i, prompts[i], limits[i])
            got.add_sequence(i, prompts[i], limits[i])
            if i in sampled:          # same parameters and the same uniform stream on both sides
                want.seqs[i].sampling = sampled[i]
                got.set_sampling(i, *sampled[i])
        nw, ng = want.step(), got.step()
        assert nw == ng, "tokens produced in step %d" % step
        for i, q in want.seqs.items():
            assert got.state(i) == q.state and got.position(i) == q.position, (step, i)
            assert got.generated(i) == q.generated, (step, i)
            if q.state == hl.FINISHED and i not in finished_at:
                finished_at[i] = step
        assert got.sequence_count() == len(want.seqs)
        for i in [i for i, q in want.seqs.items() if q.state == hl.FINISHED and finished_at[i] < step]:
            assert mr.block_table(i) == omodel.pool.seqs[i].block_tables[0]
            want.remove_sequence(i)
            got.remove_sequence(i)
        assert mr.block_stats()[1] == omodel.pool.block_stats()[1]
        if step > 6 and not want.seqs:
            break
    assert not want.seqs and got.sequence_count() == 0 and len(finished_at) == 6
    assert mr.block_stats()[1] == omodel.pool.block_stats()[1] == 48 * cfg.num_layers
    # a sampled request runs to its limit inside the vocabulary (its draws follow the library's own stream)
    got.add_sequence(30, prompts[13], 6)
    got.set_sampling(30, 0.8, 20, 0.95, 1234)
    for _ in range(8):
        got.step()
        if got.state(30) == hl.FINISHED:
            break
    toks = got.generated(30)
    assert got.state(30) == hl.FINISHED and 1 <= len(toks) <= 6 and all(0 <= t < cfg.vocab for t in toks)
    got.step()                                   # nothing left to run: the finished request is dropped, its blocks freed
    assert got.sequence_count() == 0 and mr.block_stats()[1] == 48 * cfg.num_layers
    got.close()
    mr.close()


def test_config4_scheduler_q8_0_with_512_token_chunks(be):
    """Benchmark config 4 as a whole, one layer deep: Q8_0 weights, 32 query / 8 KV heads of 128, RoPE theta 500000,
    continuous batching with 512-token prefill chunks mixed with decode in every step. A 600-token and a 30-token
    request start together, a 1150-token prompt arrives while they run (chunks at start positions 0, 512 and 1024:
    dense causal attention for the first, paged multi-query attention over the f16 pool for the later ones,
    runtime/block.go:875-895), then a 513-token one (a 1-token last chunk) and a 5-token one that waits for a free
    slot. After every step the C++ scheduler over the HIP model and hl.Scheduler over the CPU model agree on every
    sequence's state, position and generated tokens; at the end on the block tables and the pool's free count."""
    from oracle import host_logic as hl
    from vexel_amd.runtime import Scheduler
    cfg = om.ModelConfig(num_layers=1, hidden=512, num_heads=32, num_kv_heads=8, head_dim=128, ffn=1024, vocab=2048,
                         rope_theta=500000.0)
    omodel = om.random_model(cfg, 81, nx.FMT_Q8_0, nx.FMT_Q8_0, max_blocks=200)
    mr = gpu_model_from_oracle(be, omodel, pool_blocks=200, max_seqs=8, max_blocks_per_seq=80, max_batch=512)
    rng = np.random.default_rng(82)
    prompts = {21: 600, 22: 30, 23: 1150, 24: 513, 25: 5}
    prompts = {i: rng.integers(0, cfg.vocab, n).tolist() for i, n in prompts.items()}
    limits = {21: 6, 22: 9, 23: 5, 24: 4, 25: 7}
    arrivals = {0: [21, 22], 1: [23], 3: [24, 25]}
    want = hl.Scheduler(omodel, 4, 8, -1, 512)
    got = Scheduler(mr, 4, max_tokens=8, eos_token=-1, prefill_chunk=512)
    seen_prefill_positions = set()
    for step in range(24):
        for i in arrivals.get(step, []):
            want.add_sequence(i, prompts[i], limits[i])
            got.add_sequence(i, prompts[i], limits[i])
        nw, ng = want.step(), got.step()
        assert nw == ng, "tokens produced in step %d" % step
        for i, q in want.seqs.items():
            assert got.state(i) == q.state and got.position(i) == q.position, (step, i)
            assert got.generated(i) == q.generated, (step, i)
            if q.state == hl.PREFILL:
                seen_prefill_positions.add(q.position)
        for i in [i for i, q in want.seqs.items() if q.state == hl.FINISHED]:
            assert mr.block_table(i) == omodel.pool.seqs[i].block_tables[0]
            want.remove_sequence(i)
            got.remove_sequence(i)
        assert mr.block_stats()[1] == omodel.pool.block_stats()[1]
        if step > 4 and not want.seqs:
            break
    assert not want.seqs and got.sequence_count() == 0
    assert {512, 1024} <= seen_prefill_positions      # the long prompt did go through two later chunks
    assert mr.block_stats()[1] == 200 * cfg.num_layers
    got.close()
    mr.close()


def test_batched_greedy_64_steps_c2_shape(be):
    """64 greedy steps on the batched (MFMA) path against the oracle: benchmark config 2's shape, two layers deep,
    8 ragged sequences. Every step's tokens are the oracle's."""
    cfg = om.ModelConfig(num_layers=2, hidden=2048, num_heads=32, num_kv_heads=4, head_dim=64, ffn=5632, vocab=32000)
    rng0 = np.random.default_rng(55)
    ctx = [int(x) for x in rng0.integers(128, 500, 8)]
    omodel, mr, rng = _ragged_setup(be, cfg, nx.FMT_Q4_0, nx.FMT_Q8_0, ctx, 57, pool_blocks=360)
    ids = [100 + i for i in range(8)]
    first = rng.integers(0, cfg.vocab, 8).tolist()
    nx.set_row_threads(16)     # the oracle's matmuls on 16 row slices: same bits, a sixteenth of the wait
    try:
        want, _, _ = _greedy_oracle(omodel, first, ids, ctx, 64)
    finally:
        nx.set_row_threads(1)
    out, _ = mr.decode_graph(first, ids, ctx, 64, use_graph=True)
    assert out.tolist() == want
    assert mr.device_matches_host()
    mr.close()


def _f64_logit_gap(omodel, token, seq_id, pos, a, b):
    """logit[a] - logit[b] of one decode step of a LLaMA-type oracle model, evaluated in float64 from the oracle's
    inputs: the exactly dequantised weights and the K/V rows its pool holds for positions 0 .. pos (the step's own
    row included, as the oracle stored it). RoPE angles are the reference's float32 angles (cpu.go:256-260)."""
    c = omodel.cfg
    deq = lambda q: nx.dequantize(q.fmt, q.data, q.n * q.k).reshape(q.n, q.k).astype(np.float64)
    rms = lambda v, w: v / np.sqrt((v * v).mean() + c.eps) * w.astype(np.float64)
    x = omodel.embedding[token].astype(np.float64)
    D, Hq, Hk, bs = c.head_dim, c.num_heads, c.num_kv_heads, c.block_size
    j = np.arange(D // 2)
    freq = (1.0 / np.power(np.float64(c.rope_theta), 2.0 * j / D)).astype(np.float32)
    ang = (np.float32(pos) * freq).astype(np.float64)
    cs, sn = np.cos(ang), np.sin(ang)
    for l, lw in enumerate(omodel.layers):
        h = rms(x, lw.attn_norm)
        q = (deq(lw.wq) @ h).reshape(Hq, D)
        qr = q.copy()
        qr[:, 0::2] = q[:, 0::2] * cs - q[:, 1::2] * sn
        qr[:, 1::2] = q[:, 0::2] * sn + q[:, 1::2] * cs
        bt = omodel.pool.seqs[seq_id].block_tables[l]
        kv = omodel.kv[l]
        per_block = 2 * bs * Hk * D
        K = np.empty((pos + 1, Hk, D))
        V = np.empty((pos + 1, Hk, D))
        for t in range(pos + 1):
            base = bt[t // bs] * per_block + (t % bs) * Hk * D
            K[t] = nx.f16_to_f32_array(kv[base:base + Hk * D]).reshape(Hk, D)
            V[t] = nx.f16_to_f32_array(kv[base + bs * Hk * D:base + bs * Hk * D + Hk * D]).reshape(Hk, D)
        out = np.empty((Hq, D))
        for hq in range(Hq):
            hk = hq // (Hq // Hk)
            sc = K[:, hk, :] @ qr[hq] / np.sqrt(np.float64(D))
            w = np.exp(sc - sc.max())
            out[hq] = (w / w.sum()) @ V[:, hk, :]
        x = x + deq(lw.wo) @ out.reshape(-1)
        h2 = rms(x, lw.ffn_norm)
        g, u = deq(lw.w1) @ h2, deq(lw.w3) @ h2
        x = x + deq(lw.w2) @ (g / (1.0 + np.exp(-g)) * u)
    hn = rms(x, omodel.final_norm)
    head = omodel.lm_head
    rows = head.data.reshape(head.n, -1)
    la = nx.dequantize(head.fmt, rows[a], head.k).astype(np.float64) @ hn
    lb = nx.dequantize(head.fmt, rows[b], head.k).astype(np.float64) @ hn
    return float(la - lb)


def test_batched_greedy_64_steps_7b_geometry_32_sequences(be):
    """The north-star batch shape, one layer deep: hidden 4096, 32 heads of 128, FFN 11008, Q4_0, 32 ragged
    sequences, 64 greedy steps through the graph-captured batched path (2048 tokens). The oracle is run over the
    tokens the GPU produced: at every step and sequence the GPU's token must be the oracle's argmax. With 2048
    draws from 4096 near-flat random-init logits a top-two gap can fall below the float32 summation noise of the
    reference loop itself (K = 11008 sequential float32 sums). Where the GPU took the oracle's runner-up, the pair
    of logits is evaluated in float64 from the oracle's inputs, and the pick stands only if (a) it is the float64
    maximum of the two, or (b) the oracle's own float32 gap at that pair is off the float64 gap by more than the gap
    itself (the reference's arithmetic cannot tell the two apart), or (c) the float64 gap is under 1e-4: the size of
    the differences that a change of float32 summation order makes in logits of magnitude 1 to 4 here (the library
    sums 256-column chunks on the matrix cores, the reference one column after the other), a hundredth of the
    north star's 1e-2 logit tolerance. Anything else fails, and at most three picks may need (b) or (c). The
    smallest top-1 margin of every step and every settled pick are printed."""
    cfg = om.ModelConfig(num_layers=1, hidden=4096, num_heads=32, num_kv_heads=32, head_dim=128, ffn=11008, vocab=4096)
    rng0 = np.random.default_rng(61)
    ctx = [int(x) for x in np.clip(np.exp(rng0.normal(np.log(150), 0.6, 32)), 16, 400)]
    omodel, mr, rng = _ragged_setup(be, cfg, nx.FMT_Q4_0, nx.FMT_Q8_0, ctx, 63, pool_blocks=32 * 32)
    ids = [100 + i for i in range(32)]
    first = rng.integers(0, cfg.vocab, 32).tolist()
    out, _ = mr.decode_graph(first, ids, ctx, 64, use_graph=True)
    assert mr.device_matches_host()
    nx.set_row_threads(16)
    ties, margins = [], []
    try:
        toks, pos = list(first), list(ctx)
        for s in range(64):
            lg = omodel.decode_batched(toks, ids, pos)
            assert np.isfinite(lg).all()
            top2 = np.sort(lg, axis=1)[:, -2:]
            margins.append(float((top2[:, 1] - top2[:, 0]).min()))
            for i in range(32):
                best, got = nx.argmax(lg[i]), int(out[s][i])
                if got != best:
                    gap32 = float(lg[i][best] - lg[i][got])
                    gap64 = _f64_logit_gap(omodel, toks[i], ids[i], pos[i], best, got)
                    rule = "a" if gap64 <= 0.0 else ("b" if abs(gap32 - gap64) >= gap32 else ("c" if gap64 < 1e-4 else None))
                    assert rule, ("step %d sequence %d: token %d is %.3e below the oracle's %d in float32 and %.3e in float64"
                                  % (s, i, got, gap32, best, gap64))
                    ties.append((s, i, gap32, gap64, rule))
            toks = [int(t) for t in out[s]]
            pos = [p + 1 for p in pos]
    finally:
        nx.set_row_threads(1)
    print("smallest top-1 margin per step: %s" % " ".join("%.1e" % m for m in margins))
    print("picks settled in float64 (step, sequence, float32 gap, float64 gap, rule): %s" % ties)
    assert len([t for t in ties if t[4] != "a"]) <= 3, ties
    for sid in ids:
        assert mr.block_table(sid) == omodel.pool.seqs[sid].block_tables[0]
    mr.close()


def test_prefix_sharing_decodes_over_shared_blocks(be):
    """gpu_block_pool.go:568-607 end to end: sequence B takes the first two blocks of A's prompt by reference,
    prefills only the rest, and both decode. B's logits are those of a sequence that prefilled the whole prompt in
    the same two pieces (the second piece reads the f16 pool either way, runtime/block.go:875-895); the shared
    blocks survive A's deletion and B keeps decoding over them; oracle and device agree on tables and counts."""
    cfg = om.ModelConfig(num_layers=2, hidden=512, num_heads=8, num_kv_heads=2, head_dim=64, ffn=1024, vocab=1024)
    omodel = om.random_model(cfg, 91, nx.FMT_Q4_0, nx.FMT_Q8_0, max_blocks=40)
    mr = gpu_model_from_oracle(be, omodel, pool_blocks=40, max_seqs=8, max_blocks_per_seq=8, max_batch=64)
    rng = np.random.default_rng(92)
    prompt = rng.integers(0, cfg.vocab, 45).tolist()
    A, B, Cq = 1, 2, 3
    for sid in (A, B, Cq):
        omodel.pool.create_sequence(sid)
        mr.create_sequence(sid)
    assert_logits_close(mr.prefill_with_paged_kv(prompt, A, 0), omodel.prefill_with_paged_kv(prompt, A, 0), "A")
    omodel.pool.share_blocks(A, B, 32)
    mr.share_blocks(A, B, 32)
    assert mr.block_stats() == omodel.pool.block_stats() and mr.block_stats()[2] == 2 * cfg.num_layers
    wb = omodel.prefill_with_paged_kv(prompt[32:], B, 32)
    gb = mr.prefill_with_paged_kv(prompt[32:], B, 32)
    assert_logits_close(gb, wb, "B after the shared prefix")
    assert mr.block_table(B)[:2] == mr.block_table(A)[:2] == omodel.pool.seqs[A].block_tables[0][:2]
    # a sequence that computes the same prompt itself, in the same two pieces
    mr.prefill_with_paged_kv(prompt[:32], Cq, 0)
    gc = mr.prefill_with_paged_kv(prompt[32:], Cq, 32)
    assert np.abs(gb - gc).max() <= 1e-5 * np.abs(gc).max()
    mr.delete_sequence(Cq)
    omodel.pool.delete_sequence(Cq)
    # both decode, then A goes away and B goes on over the blocks it shares no longer with anyone
    toks, pos = [7, nx.argmax(wb)], [45, 45]
    for step in range(3):
        want = omodel.decode_batched(toks, [A, B], pos)
        got, am = mr.decode_with_paged_kv_batched(toks, [A, B], pos)
        assert_logits_close(got, want, "shared decode %d" % step)
        toks = [nx.argmax(want[i]) for i in range(2)]
        assert toks == [int(a) for a in am]
        pos = [p + 1 for p in pos]
    omodel.pool.delete_sequence(A)
    mr.delete_sequence(A)
    assert mr.block_stats() == omodel.pool.block_stats() and mr.block_stats()[2] == 0
    for step in range(3):
        want = omodel.decode_batched(toks[1:], [B], pos[1:])
        got, am = mr.decode_with_paged_kv_batched(toks[1:], [B], pos[1:])
        assert_logits_close(got, want, "B alone %d" % step)
        toks = [toks[0], nx.argmax(want[0])]
        assert toks[1] == int(am[0])
        pos = [p + 1 for p in pos]
    assert mr.block_table(B) == omodel.pool.seqs[B].block_tables[0]
    mr.close()


@pytest.mark.parametrize("kv_f16", [True, False])
def test_fragment_cache_insert_with_rope_shift(be, kv_f16):
    """kv/fragment.go + kv/paged_cache.go:285-343: a prefilled document is cached under a name, its sequence
    deleted; two other sequences put it behind prompts of different lengths (K rotated by 13 and by 32 positions on
    insertion, V copied) and decode. Pool contents are compared bit for bit with the oracle's (same float32
    operations, same rounding to the pool's type), logits within the usual tolerance, tables and counts exactly."""
    cfg = om.ModelConfig(num_layers=2, hidden=512, num_heads=8, num_kv_heads=2, head_dim=64, ffn=1024, vocab=1024)
    omodel = om.random_model(cfg, 93, nx.FMT_Q4_0, nx.FMT_Q8_0, max_blocks=48, kv_fp16=kv_f16)
    mr = gpu_model_from_oracle(be, omodel, pool_blocks=48, max_seqs=8, max_blocks_per_seq=8, max_batch=64)
    rng = np.random.default_rng(94)
    # the document's K/V: the same values on both sides (a prefill would leave last-bit differences between the two
    # implementations in the source rows, and the comparison below is exact)
    install_context(omodel, mr, be, 1, [5, 9, 2], 37, rng)
    omodel.pool.cache_content("doc", 1)
    mr.cache_fragment("doc", 1)
    omodel.pool.delete_sequence(1)
    mr.delete_sequence(1)
    assert mr.fragment_tokens("doc") == 37 and mr.fragment_count() == 1 and mr.fragment_tokens("other") == -1
    assert mr.block_stats() == omodel.pool.block_stats()
    per_block = 2 * cfg.block_size * cfg.num_kv_heads * cfg.head_dim
    esz, dt = (2, np.uint16) if kv_f16 else (4, np.float32)
    for sid, plen in ((2, 13), (3, 32)):
        head = rng.integers(0, cfg.vocab, plen).tolist()
        omodel.pool.create_sequence(sid)
        mr.create_sequence(sid)
        assert_logits_close(mr.prefill_with_paged_kv(head, sid, 0), omodel.prefill_with_paged_kv(head, sid, 0), "head")
        assert omodel.insert_fragment(sid, "doc", plen) == 37
        assert mr.insert_fragment(sid, "doc", plen) == 37
        assert mr.seq_len(sid) == plen + 37 == omodel.pool.seqs[sid].seq_len
        assert mr.block_table(sid) == omodel.pool.seqs[sid].block_tables[0]
        row = cfg.num_kv_heads * cfg.head_dim
        for layer in range(cfg.num_layers):        # the inserted rows, K and V, bit for bit
            for b in set(mr.block_table(sid)[plen // 16:]):
                got = be.download(mr.kv_pool(layer) + b * per_block * esz, (per_block,), dt)
                want = np.ascontiguousarray(omodel.kv[layer][b * per_block:(b + 1) * per_block])
                lb = mr.block_table(sid).index(b)
                for off in range(16):
                    if plen <= lb * 16 + off < plen + 37:
                        for base in (off * row, 16 * row + off * row):
                            assert np.array_equal(got[base:base + row].view(np.uint8), want[base:base + row].view(np.uint8)), \
                                (sid, layer, b, off)
        tok, pos = 5, plen + 37
        for step in range(3):
            want = omodel.decode_with_paged_kv(tok, sid, pos)
            got, am = mr.decode_with_paged_kv_batched([tok], [sid], [pos])
            assert_logits_close(got[0], want, "decode after the fragment %d" % step)
            tok = nx.argmax(want)
            assert tok == int(am[0])
            pos += 1
    assert mr.insert_fragment(2, "no such fragment", mr.seq_len(2)) == 0
    from vexel_amd.backend import VexelError
    with pytest.raises(VexelError, match="end of sequence"):
        mr.insert_fragment(2, "doc", 3)
    omodel.pool.delete_fragment("doc")
    mr.delete_fragment("doc")
    assert mr.fragment_count() == 0 and mr.block_stats() == omodel.pool.block_stats()
    mr.close()


def test_pool_errors_and_lifecycle(be):
    """Host-forced failure paths: pool exhaustion, unknown sequence, truncate no-ops."""
    from vexel_amd.backend import VexelError
    cfg = om.ModelConfig(num_layers=1, hidden=256, num_heads=2, num_kv_heads=2, head_dim=128, ffn=256, vocab=256)
    omodel = om.random_model(cfg, 41, nx.FMT_Q4_0, nx.FMT_Q4_0, max_blocks=2)
    mr = gpu_model_from_oracle(be, omodel, pool_blocks=2, max_seqs=4, max_blocks_per_seq=4, max_batch=4)
    mr.prefill_with_paged_kv(list(range(32)), 1, 0)            # uses both blocks
    with pytest.raises(VexelError) as e:
        mr.decode_with_paged_kv_batched([1], [1], [32])       # needs a third block
    assert "no free blocks" in str(e.value)
    mr.truncate_sequence(999, 5)                               # unknown: no-op
    mr.truncate_sequence(1, 100)                               # beyond length: no-op
    assert mr.seq_len(1) == 32
    mr.truncate_sequence(1, 16)
    assert mr.block_stats() == (2, 1, 0)
    mr.create_sequence(2)
    mr.share_blocks(1, 2, 16)
    assert mr.block_stats() == (2, 1, 1)
    mr.delete_sequence(1)
    assert mr.block_stats() == (2, 1, 0) and mr.has_sequence(2) and not mr.has_sequence(1)
    with pytest.raises(VexelError):
        mr.share_blocks(7, 2, 16)
    mr.close()


def test_fragment_insert_that_runs_out_of_blocks_leaves_the_sequence_as_it_was(be):
    """A fragment of 3 blocks is put behind a 13-token prompt in a pool with one free block: the insertion fails, and the
    sequence keeps its table, its length and its logits, the pool its counts (host-forced failure, no kernel involved);
    after room is made the same insertion succeeds and, undone again, leaves the logits of the next step unchanged."""
    from vexel_amd.backend import VexelError
    cfg = om.ModelConfig(num_layers=2, hidden=256, num_heads=4, num_kv_heads=2, head_dim=64, ffn=256, vocab=256)
    omodel = om.random_model(cfg, 43, nx.FMT_Q4_0, nx.FMT_Q4_0, max_blocks=8)
    mr = gpu_model_from_oracle(be, omodel, pool_blocks=8, max_seqs=4, max_blocks_per_seq=8, max_batch=4)
    mr.prefill_with_paged_kv(list(range(37)), 1, 0)            # 3 blocks
    mr.cache_fragment("doc", 1)
    mr.delete_sequence(1)
    mr.prefill_with_paged_kv(list(range(64)), 3, 0)            # 4 more: one block left
    mr.create_sequence(2)
    mr.prefill_with_paged_kv(list(range(13)), 2, 0)            # the last one
    table, stats = mr.block_table(2), mr.block_stats()
    with pytest.raises(VexelError, match="no free blocks"):
        mr.insert_fragment(2, "doc", 13)
    assert mr.block_table(2) == table and mr.block_stats() == stats and mr.seq_len(2) == 13
    before, _ = mr.decode_with_paged_kv_batched([7], [2], [13])
    mr.truncate_sequence(2, 13)
    mr.delete_sequence(3)
    assert mr.insert_fragment(2, "doc", 13) == 37 and mr.seq_len(2) == 50 and len(mr.block_table(2)) == 4
    mr.truncate_sequence(2, 13)
    again, _ = mr.decode_with_paged_kv_batched([7], [2], [13])
    assert np.array_equal(before.view(np.uint32), again.view(np.uint32))
    mr.close()


# ------------------------------------------------------------------ the architectures beside LLaMA
def _arch_config(name):
    """Small models with the layer shapes of Phi-2 (LayerNorm, biases, 32 of 80 head dimensions rotated in split
    pairs, GELU MLP, parallel residual), Gemma 2 (scaled embeddings, GeGLU, post-norms, soft-capped attention, heads
    of 256) and Qwen 2 (Q/K/V biases, split-pair RoPE, theta 1e6)."""
    import math
    if name == "phi":
        return om.ModelConfig(num_layers=2, hidden=640, num_heads=8, num_kv_heads=8, head_dim=80, ffn=2560, vocab=1000,
                              norm_type="layer", mlp_type="gelu", parallel_residual=True, rope_dim=32, rope_neox=True)
    if name == "gemma":
        return om.ModelConfig(num_layers=2, hidden=512, num_heads=4, num_kv_heads=2, head_dim=256, ffn=1024, vocab=1000,
                              eps=1e-6, mlp_type="geglu", post_norms=True, attn_softcap=50.0, rope_neox=True,
                              embedding_scale=float(np.float32(math.sqrt(512.0))))
    if name == "qwen_g7":   # 7 query heads per KV head (Qwen 2 7B's 28 / 4) at heads of 128: the fused blocks and the
        return om.ModelConfig(num_layers=2, hidden=1024, num_heads=14, num_kv_heads=2, head_dim=128, ffn=1536,  # split merge
                              vocab=1000, eps=1e-6, rope_neox=True, rope_theta=1000000.0)
    return om.ModelConfig(num_layers=2, hidden=512, num_heads=8, num_kv_heads=2, head_dim=64, ffn=1536, vocab=1000,
                          eps=1e-6, rope_neox=True, rope_theta=1000000.0)


@pytest.mark.parametrize("name", ["phi", "gemma", "qwen", "qwen_g7"])
def test_other_architectures_prefill_decode_graph(be, name):
    """ExecuteWithPagedKV's general sequence (block.go:834-1077) through vh_prefill (first chunk and a later one),
    vh_decode_batched, the device-driven vh_decode_graph and vh_verify_tree, against the oracle's layer for the same
    switches."""
    cfg = _arch_config(name)
    omodel = om.random_model(cfg, 21, nx.FMT_Q4_0, nx.FMT_Q8_0, max_blocks=40)
    if name.startswith("qwen"):
        rng = np.random.default_rng(22)
        qd, kvd = cfg.num_heads * cfg.head_dim, cfg.num_kv_heads * cfg.head_dim
        for lw in omodel.layers:
            lw.wq_bias = (0.05 * rng.standard_normal(qd)).astype(np.float32)
            lw.wk_bias = (0.05 * rng.standard_normal(kvd)).astype(np.float32)
            lw.wv_bias = (0.05 * rng.standard_normal(kvd)).astype(np.float32)
    mr = gpu_model_from_oracle(be, omodel, pool_blocks=40, max_seqs=4, max_batch=8)
    rng = np.random.default_rng(23)
    # a chunk of 130 rows: the general sequence then takes its activation kernels that leave W2's prepared operand
    long_prompt = rng.integers(0, cfg.vocab, 130).tolist()
    assert_logits_close(mr.prefill_with_paged_kv(long_prompt, 3, 0), omodel.prefill_with_paged_kv(long_prompt, 3, 0),
                        "%s 130-row chunk" % name)
    mr.delete_sequence(3)
    omodel.pool.delete_sequence(3)
    prompts = {1: rng.integers(0, cfg.vocab, 21).tolist(), 2: rng.integers(0, cfg.vocab, 35).tolist()}
    toks, worst = {}, 0.0
    for sid, p in prompts.items():
        want = omodel.prefill_with_paged_kv(p[:17], sid, 0)
        got = mr.prefill_with_paged_kv(p[:17], sid, 0)
        worst = max(worst, assert_logits_close(got, want, "%s first chunk" % name))
        want = omodel.prefill_with_paged_kv(p[17:], sid, 17)
        got = mr.prefill_with_paged_kv(p[17:], sid, 17)
        worst = max(worst, assert_logits_close(got, want, "%s second chunk" % name))
        toks[sid] = nx.argmax(want)
        assert toks[sid] == int(np.argmax(got))
    ids = [1, 2]
    pos = [len(prompts[1]), len(prompts[2])]
    cur = [toks[1], toks[2]]
    for step in range(12):
        want = omodel.decode_batched(cur, ids, pos)
        got, am = mr.decode_with_paged_kv_batched(cur, ids, pos)
        worst = max(worst, assert_logits_close(got, want, "%s decode step %d" % (name, step)))
        nxt = [nx.argmax(w) for w in want]
        assert nxt == [int(a) for a in am]
        cur, pos = nxt, [p + 1 for p in pos]
    # the device-driven loop continues from here; the oracle follows step by step
    out, _ = mr.decode_graph(cur, ids, pos, 6)
    for step in range(6):
        want = omodel.decode_batched(cur, ids, pos)
        cur, pos = [nx.argmax(w) for w in want], [p + 1 for p in pos]
        assert out[step].tolist() == cur, "graph step %d" % step
    assert mr.block_table(1) == omodel.pool.seqs[1].block_tables[0]
    assert mr.device_matches_host()
    # tree verification under the same switches: a 10-node tree per sequence, sequence 1's own greedy continuation
    # planted two levels deep, acceptance and rollback against the oracle's pass, then a decode step on the result
    import copy
    from oracle import host_logic as hl
    rng = np.random.default_rng(24)
    probe, tok, plant = copy.deepcopy(omodel), cur[0], []
    for d in range(2):
        tok = nx.argmax(probe.decode_with_paged_kv(tok, 1, pos[0] + d))
        plant.append(tok)
    trees = []
    for i in range(2):
        tk = [rng.choice(cfg.vocab, 2, replace=False).tolist() for _ in range(4)]
        if i == 0:
            for h, t in enumerate(plant):
                tk[h][(h + 1) % 2] = t
                if tk[h][0] == tk[h][1]:
                    tk[h][h % 2] = (t + 1) % cfg.vocab
        trees.append(hl.build_candidate_tree_from_topk(tk, [[2.0, 1.0]] * 4, 10).linearize())
    want = omodel.tree_step_batched(cur, trees, ids, pos)
    acc, fin, logits = mr.verify_tree(ids, cur, pos, trees)
    for i, sid in enumerate(ids):
        worst = max(worst, assert_logits_close(logits[i], want[i][2], "%s tree rows of sequence %d" % (name, sid)))
        assert acc[i] == want[i][0] and fin[i] == want[i][1]
        assert mr.seq_len(sid) == omodel.pool.seqs[sid].seq_len == pos[i] + 1 + len(acc[i])
        assert mr.block_table(sid) == omodel.pool.seqs[sid].block_tables[0]
    assert len(acc[0]) >= 2
    cur, pos = list(fin), [pos[i] + 1 + len(acc[i]) for i in range(2)]
    want = omodel.decode_batched(cur, ids, pos)
    got, am = mr.decode_with_paged_kv_batched(cur, ids, pos)
    worst = max(worst, assert_logits_close(got, want, "%s decode after the rollback" % name))
    assert [nx.argmax(w) for w in want] == [int(a) for a in am]
    assert mr.device_matches_host()
    print("%s: worst logit error %.3e" % (name, worst))
    mr.close()


def test_architecture_switches_are_validated(be):
    cfg = om.ModelConfig(num_layers=1, hidden=256, num_heads=4, num_kv_heads=2, head_dim=64, ffn=512, vocab=300)
    omodel = om.random_model(cfg, 3, nx.FMT_Q4_0, nx.FMT_Q8_0, max_blocks=8)
    mr = gpu_model_from_oracle(be, omodel, pool_blocks=8, max_seqs=2, max_batch=2)
    with pytest.raises(RuntimeError, match="parallel residual"):
        mr.set_architecture(parallel_residual=True)                 # gated MLP
    with pytest.raises(RuntimeError, match="rope_dim"):
        mr.set_architecture(rope_dim=66)
    with pytest.raises(RuntimeError, match="rope_dim"):
        mr.set_architecture(rope_dim=31)
    with pytest.raises(RuntimeError, match="soft cap"):
        mr.set_architecture(attn_softcap=-1.0)
    # rope_dim = head_dim is the default sequence's arithmetic: same logits, bit for bit, as the unfused LLaMA arm
    mr.set_fused(False)
    prompt = list(range(30, 49))
    a = mr.prefill_with_paged_kv(prompt, 1, 0)
    mr.set_architecture(rope_dim=64)
    b = mr.prefill_with_paged_kv(prompt, 2, 0)
    assert_logits_close(b, a, "rope_dim = head_dim")
    mr.close()


def test_scheduler_caps_the_logits_of_sampled_requests(be):
    """FinalLogitSoftCap (model.go:336-350) reaches only the logits a request is sampled from (scheduler.go:772-773):
    a Gemma-2-like model with a small cap, two sampled requests and a greedy one, C++ scheduler against its oracle
    restatement token by token; without the cap the sampled requests would have drawn other tokens."""
    import copy
    from oracle import host_logic as hl
    from vexel_amd.runtime import Scheduler
    cfg = _arch_config("gemma")
    cfg.final_softcap = 0.5
    omodel = om.random_model(cfg, 81, nx.FMT_Q4_0, nx.FMT_Q8_0, max_blocks=24)
    plain = copy.deepcopy(omodel)
    plain.cfg = copy.copy(cfg)
    plain.cfg.final_softcap = 0.0
    mr = gpu_model_from_oracle(be, omodel, pool_blocks=24, max_seqs=4, max_batch=8)
    rng = np.random.default_rng(82)
    prompts = {1: rng.integers(0, cfg.vocab, 9).tolist(), 2: rng.integers(0, cfg.vocab, 20).tolist(),
               3: rng.integers(0, cfg.vocab, 5).tolist()}
    sampled = {1: (1.5, 0, 1.0, 7), 3: (0.9, 50, 0.95, 8)}
    want, other = hl.Scheduler(omodel, 4, 10, -1), hl.Scheduler(plain, 4, 10, -1)
    got = Scheduler(mr, 4, max_tokens=10, eos_token=-1)
    for i, p in prompts.items():
        for sch in (want, other):
            sch.add_sequence(i, p, 10)
            if i in sampled:
                sch.seqs[i].sampling = sampled[i]
        got.add_sequence(i, p, 10)
        if i in sampled:
            got.set_sampling(i, *sampled[i])
    capped, uncapped = {}, {}
    for step in range(12):
        nw, ng = want.step(), got.step()
        other.step()
        assert nw == ng
        for i, q in want.seqs.items():
            assert got.generated(i) == q.generated, (step, i)
            capped[i] = list(q.generated)
        for i, q in other.seqs.items():
            uncapped[i] = list(q.generated)
    assert all(len(capped[i]) == 10 for i in prompts)
    assert capped[1] != uncapped[1] and capped[3] != uncapped[3]
    assert capped[2] == uncapped[2]                                 # the greedy request never sees the cap
    got.close()
    mr.close()


def _gguf_from_oracle(omodel, arch, extra_md=()):
    """The oracle model as the tensors and metadata a GGUF file of that architecture holds (pkg/gguf/loader.go:121-228
    names): Phi with its fused attn_qkv matrix and bias, fc1 / fc2 as ffn_up / ffn_down, no ffn_norm."""
    from oracle import gguf as og
    cfg = omodel.cfg
    f32 = lambda name, a: (name, [int(a.size)], og.T_F32, np.ascontiguousarray(a, dtype=np.float32).tobytes())
    mat = lambda name, q: (name, [q.k, q.n], GGUF_TYPE[q.fmt], q.data.tobytes())
    tensors = []
    for l, lw in enumerate(omodel.layers):
        b = "blk.%d." % l
        tensors.append(f32(b + "attn_norm.weight", lw.attn_norm))
        if arch == "phi2":
            fused = np.concatenate([lw.wq.data, lw.wk.data, lw.wv.data], axis=0)
            tensors.append((b + "attn_qkv.weight", [lw.wq.k, lw.wq.n + 2 * lw.wk.n], GGUF_TYPE[lw.wq.fmt], fused.tobytes()))
            tensors.append(f32(b + "attn_qkv.bias", np.concatenate([lw.wq_bias, lw.wk_bias, lw.wv_bias])))
            tensors += [f32(b + "attn_norm.bias", lw.attn_norm_bias), f32(b + "attn_output.bias", lw.wo_bias),
                        f32(b + "ffn_up.bias", lw.w1_bias), f32(b + "ffn_down.bias", lw.w2_bias)]
            tensors.append(mat(b + "ffn_up.weight", lw.w1))
        elif arch == "phi3":   # fused attn_qkv (no bias) and the gate+up matrix as ffn_up, gate rows first
            fused = np.concatenate([lw.wq.data, lw.wk.data, lw.wv.data], axis=0)
            tensors.append((b + "attn_qkv.weight", [lw.wq.k, lw.wq.n + 2 * lw.wk.n], GGUF_TYPE[lw.wq.fmt], fused.tobytes()))
            both = np.concatenate([lw.w1.data, lw.w3.data], axis=0)
            tensors.append((b + "ffn_up.weight", [lw.w1.k, 2 * lw.w1.n], GGUF_TYPE[lw.w1.fmt], both.tobytes()))
            tensors.append(f32(b + "ffn_norm.weight", lw.ffn_norm))
        else:
            tensors += [mat(b + "attn_q.weight", lw.wq), mat(b + "attn_k.weight", lw.wk), mat(b + "attn_v.weight", lw.wv),
                        mat(b + "ffn_gate.weight", lw.w1), mat(b + "ffn_up.weight", lw.w3),
                        f32(b + "ffn_norm.weight", lw.ffn_norm)]
            if lw.wq_bias is not None:
                tensors += [f32(b + "attn_q.bias", lw.wq_bias), f32(b + "attn_k.bias", lw.wk_bias),
                            f32(b + "attn_v.bias", lw.wv_bias)]
            if lw.post_attn_norm is not None:
                tensors += [f32(b + "post_attention_norm.weight", lw.post_attn_norm),
                            f32(b + "post_ffw_norm.weight", lw.post_ffn_norm)]
        tensors += [mat(b + "attn_output.weight", lw.wo), mat(b + "ffn_down.weight", lw.w2)]
    tensors.append(f32("output_norm.weight", omodel.final_norm))
    if omodel.final_norm_bias is not None:
        tensors.append(f32("output_norm.bias", omodel.final_norm_bias))
    tensors.append(("token_embd.weight", [cfg.hidden, cfg.vocab], og.T_F32, omodel.embedding.tobytes()))
    tensors.append(mat("output.weight", omodel.lm_head))
    p = arch + "."
    md = [("general.architecture", og.MT_STRING, arch), (p + "block_count", og.MT_U32, cfg.num_layers),
          (p + "embedding_length", og.MT_U32, cfg.hidden), (p + "attention.head_count", og.MT_U32, cfg.num_heads),
          (p + "attention.head_count_kv", og.MT_U32, cfg.num_kv_heads), (p + "feed_forward_length", og.MT_U32, cfg.ffn),
          (p + "context_length", og.MT_U32, 2048), (p + "rope.freq_base", og.MT_F32, cfg.rope_theta),
          (p + "attention.layer_norm_rms_epsilon", og.MT_F32, cfg.eps)] + list(extra_md)
    return og.build(md, tensors)


@pytest.mark.parametrize("arch", ["phi2", "gemma2", "qwen2", "phi3"])
def test_load_gguf_other_architectures(be, tmp_path, arch):
    """general.architecture selects the switches as ModelConfigFromGGUF does (runtime/config.go:388-470) and the
    loader finds each architecture's tensors (runtime/loader.go:290-385): the loaded model gives the oracle's logits
    and greedy tokens. Gemma 2 takes interleaved RoPE pairs here, as the reference's table has it. Phi-3: the fused
    attn_qkv matrix and the gate+up matrix (gate rows first, loader.go:1147-1218) are used in place as row ranges."""
    import copy, os
    from oracle import gguf as og
    from vexel_amd.backend import VexelError
    from vexel_amd.runtime import ModelRuntime
    cfg = _arch_config({"phi2": "phi", "gemma2": "gemma", "qwen2": "qwen", "phi3": "qwen"}[arch])  # (Phi-3: Qwen 2's layer without biases)
    extra = []
    if arch == "gemma2":
        cfg.rope_neox, cfg.final_softcap = False, 30.0
        extra = [("gemma2.attention.key_length", og.MT_U32, cfg.head_dim), ("gemma2.attn_logit_softcapping", og.MT_F32, 50.0),
                 ("gemma2.final_logit_softcapping", og.MT_F32, 30.0)]
    if arch == "phi2":
        cfg.eps = 1e-5
        extra = [("phi2.rope.dimension_count", og.MT_U32, cfg.rope_dim)]
    omodel = om.random_model(cfg, 91, nx.FMT_Q4_0, nx.FMT_Q8_0, max_blocks=16)
    if arch == "qwen2":
        rng = np.random.default_rng(92)
        for lw in omodel.layers:
            lw.wq_bias = (0.05 * rng.standard_normal(512)).astype(np.float32)
            lw.wk_bias = (0.05 * rng.standard_normal(128)).astype(np.float32)
            lw.wv_bias = (0.05 * rng.standard_normal(128)).astype(np.float32)
    path = os.path.join(tmp_path, arch + ".gguf")
    with open(path, "wb") as fh:
        fh.write(_gguf_from_oracle(omodel, arch, extra))
    mr = ModelRuntime.from_gguf(be, path, pool_blocks=16, max_seqs=4, max_batch=8)
    assert mr.cfg.head_dim == cfg.head_dim
    prompt = np.random.default_rng(93).integers(0, cfg.vocab, 23).tolist()
    want = omodel.prefill_with_paged_kv(prompt, 1, 0)
    got = mr.prefill_with_paged_kv(prompt, 1, 0)
    assert_logits_close(got, want, arch + " prefill from the loaded checkpoint")
    tok, pos = nx.argmax(want), len(prompt)
    assert tok == int(np.argmax(got))
    for step in range(6):
        want = omodel.decode_with_paged_kv(tok, 1, pos)
        got, am = mr.decode_with_paged_kv_batched([tok], [1], [pos])
        assert_logits_close(got[0], want, "%s decode step %d" % (arch, step))
        tok, pos = nx.argmax(want), pos + 1
        assert tok == int(am[0])
    mr.close()
    # an architecture without a loader is refused by name
    blob = _gguf_from_oracle(omodel, arch, extra).replace(arch.encode(), b"x" * len(arch))
    with open(path, "wb") as fh:
        fh.write(blob)
    with pytest.raises(VexelError, match="no loader here"):
        ModelRuntime.from_gguf(be, path, pool_blocks=16, max_seqs=4, max_batch=8)
