"""Full-depth parity against the CPU oracle: the models of the benchmark configs at their real number of layers, so
that the growth of the float32 differences over depth is measured against the oracle and not only between the
library's own paths.

Generating 22 or 32 layers of N(0, 0.02) weights in numpy takes minutes, so a deep model is grown from a few
generated layers: layer l holds the rows of generated layer l mod base rotated by 17 l positions (another matrix of
the same distribution; what the comparison needs is depth, not 32 independent draws)."""
import copy

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


def _deep_model(cfg, seed, fmt, head_fmt, base, max_blocks):
    small = om.random_model(om.ModelConfig(**{**cfg.__dict__, "num_layers": base}), seed, fmt, head_fmt, max_blocks=16)
    layers = []
    for l in range(cfg.num_layers):
        src = small.layers[l % base]
        lw = copy.copy(src)
        for name in ("wq", "wk", "wv", "wo", "w1", "w3", "w2"):
            q = getattr(src, name)
            rows = q.data.reshape(q.n, -1)
            setattr(lw, name, om.QWeight(q.fmt, np.ascontiguousarray(np.roll(rows, 17 * l, axis=0)), q.n, q.k))
        layers.append(lw)
    return om.OracleModel(cfg, small.embedding, layers, small.final_norm, small.lm_head, max_blocks)


def test_c1_at_22_layers_prefill_and_8_greedy_steps(be):
    """Benchmark config 1 at its real depth: TinyLlama shape, 22 layers, Q4_0 with Q8_0 embeddings and head; a
    32-token prompt and 8 greedy steps. Logits within 1e-2 / 1e-3 of the oracle's at every step, tokens identical."""
    cfg = om.ModelConfig(num_layers=22, hidden=2048, num_heads=32, num_kv_heads=4, head_dim=64, ffn=5632, vocab=32000,
                         eps=1e-5, rope_theta=10000.0)
    omodel = _deep_model(cfg, 3, nx.FMT_Q4_0, nx.FMT_Q8_0, base=2, max_blocks=8)
    mr = gpu_model_from_oracle(be, omodel, pool_blocks=8, max_batch=8)
    rng = np.random.default_rng(4)
    prompt = rng.integers(0, cfg.vocab, 32).tolist()
    nx.set_row_threads(16)
    try:
        want = omodel.prefill_with_paged_kv(prompt, 1, 0)
        got = mr.prefill_with_paged_kv(prompt, 1, 0)
        worst = assert_logits_close(got, want, "prefill logits at 22 layers")
        tok = nx.argmax(want)
        assert tok == int(np.argmax(got))
        pos, margins = len(prompt), []
        for step in range(8):
            want = omodel.decode_with_paged_kv(tok, 1, pos)
            got, am = mr.decode_with_paged_kv_batched([tok], [1], [pos])
            worst = max(worst, assert_logits_close(got[0], want, "decode step %d at 22 layers" % step))
            s = np.sort(want)
            margins.append(float(s[-1] - s[-2]))
            tok = nx.argmax(want)
            assert tok == int(am[0]), "greedy token differs at step %d (top-1 margin %.3e)" % (step, margins[-1])
            pos += 1
    finally:
        nx.set_row_threads(1)
    assert mr.block_table(1) == omodel.pool.seqs[1].block_tables[0]
    print("C1 at 22 layers: worst logit error %.3e, top-1 margins %s" % (worst, ["%.2e" % m for m in margins]))
    mr.close()


def test_north_star_shape_at_32_layers_batched_steps(be):
    """The north-star model at its real depth: 32 layers, hidden 4096, 32 heads of 128, FFN 11008, Q4_0, Q8_0 head
    (vocabulary cut to 4096 rows: the head is one matrix product either way); three ragged sequences with installed
    contexts, two batched greedy steps on the MFMA path (packed weights). Logits within 1e-2 / 1e-3, tokens
    identical, block tables equal."""
    cfg = om.ModelConfig(num_layers=32, hidden=4096, num_heads=32, num_kv_heads=32, head_dim=128, ffn=11008, vocab=4096)
    ctx = [37, 200, 121]
    omodel = _deep_model(cfg, 9, nx.FMT_Q4_0, nx.FMT_Q8_0, base=1, max_blocks=32)
    mr = gpu_model_from_oracle(be, omodel, pool_blocks=32, max_seqs=4, max_blocks_per_seq=16, max_batch=4)
    rng = np.random.default_rng(10)
    perm, off = rng.permutation(32), 0
    for i, L in enumerate(ctx):
        nb = (L + 15) // 16
        install_context(omodel, mr, be, 50 + i, perm[off:off + nb], L, rng)
        off += nb
    ids = [50, 51, 52]
    toks, pos = rng.integers(0, cfg.vocab, 3).tolist(), list(ctx)
    nx.set_row_threads(16)
    try:
        for step in range(2):
            want = omodel.decode_batched(toks, ids, pos)
            got, am = mr.decode_with_paged_kv_batched(toks, ids, pos)
            worst = assert_logits_close(got, want, "32 layers, step %d" % step)
            nxt = [nx.argmax(want[i]) for i in range(3)]
            margins = [float(np.sort(want[i])[-1] - np.sort(want[i])[-2]) for i in range(3)]
            assert nxt == [int(a) for a in am], "step %d: tokens differ (top-1 margins %s)" % (step, margins)
            print("NS at 32 layers, step %d: worst logit error %.3e, top-1 margins %s" % (step, worst, ["%.2e" % m for m in margins]))
            toks, pos = nxt, [p + 1 for p in pos]
    finally:
        nx.set_row_threads(1)
    for sid in ids:
        assert mr.block_table(sid) == omodel.pool.seqs[sid].block_tables[0]
    assert mr.device_matches_host()
    mr.close()
