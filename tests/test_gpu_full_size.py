"""The hot kernels at the benchmark configs' full shapes. The oracle cannot run whole matrices of this size in
seconds, so every check takes the full-size GPU result and compares a sample of it (rows of the weight matrix,
whole attention heads) with the oracle computed on exactly those rows, plus properties that hold at any size."""
import math

import numpy as np
import pytest

from oracle import numerics as nx

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def be():
    from vexel_amd.backend import HipBackend
    b = HipBackend(0)
    yield b
    b.close()


def _close(got, want, rtol, atol, what):
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    lim = atol + rtol * np.abs(want.astype(np.float64))
    assert np.all(err <= lim), "%s: max err %.3e" % (what, err.max())


def _random_blocks(rng, fmt, n, k, d_scale):
    """Random valid rows [n, k] of a 32-element-block format: random codes, finite f16 scales around d_scale."""
    bb = nx.BLOCK_BYTES[fmt]
    nblk = n * (k // 32)
    raw = rng.integers(0, 256, size=(nblk, bb), dtype=np.uint8)
    d = (d_scale * (0.25 + rng.random(nblk))).astype(np.float16)
    raw[:, 0:2] = d.view(np.uint16)[:, None].view(np.uint8).reshape(nblk, 2)
    return raw.reshape(n, -1)


def _sampled_matmul_check(be, fmt, m, n, k, rng, what, d_scale):
    w = _random_blocks(rng, fmt, n, k, d_scale)
    a = rng.standard_normal((m, k)).astype(np.float32)
    da, dw = be.upload(a, permanent=True), be.upload(w, permanent=True)
    dout = be.alloc_permanent(m * n * 4)
    be.matmul_quant(fmt, da, dw, dout, None, m, n, k)
    got = be.download(dout, (m, n), np.float32)
    rows = np.unique(np.concatenate([rng.integers(0, n, 61), [0, 127, 128, n - 129, n - 1]]))
    want = nx.matmul_quant(fmt, a, w[rows], m, len(rows), k)
    _close(got[:, rows], want, 2e-5, 3e-6 * np.abs(want).max() + 1e-7, what)
    for p in (da, dw, dout):
        be.free(p)
    return got


def test_lm_head_at_llama3_vocab(be):
    """Config 4's output head: [128256, 4096] Q8_0, one row (matrix-vector kernel) and 32 rows (MFMA kernel);
    the row-wise argmax of the full logits is numpy's first maximum."""
    rng = np.random.default_rng(401)
    n, k = 128256, 4096
    one = _sampled_matmul_check(be, nx.FMT_Q8_0, 1, n, k, rng, "lm_head, 1 row", 0.02 / 64)
    many = _sampled_matmul_check(be, nx.FMT_Q8_0, 32, n, k, rng, "lm_head, 32 rows", 0.02 / 64)
    assert np.all(np.isfinite(one)) and np.all(np.isfinite(many))
    many[3, 100000] = many[3, 7] = many[3].max() + 1.0          # a tie: the first index wins
    many[9, n - 1] = many[9].max() + 1.0                         # the very last column
    d = be.upload(many, permanent=True)
    di = be.alloc(32 * 4)
    be.argmax_rows(d, 32, n, di)
    assert np.array_equal(be.download(di, (32,), np.int32), np.argmax(many, axis=1).astype(np.int32))
    be.free(d)
    be.reset_pool()


@pytest.mark.parametrize("name,n,k", [("gate|up width", 22016, 4096), ("down", 4096, 11008), ("8B gate", 14336, 4096),
                                      ("8B down", 4096, 14336)])
def test_7b_and_8b_projection_shapes_q4_0(be, name, n, k):
    rng = np.random.default_rng(402 + n)
    _sampled_matmul_check(be, nx.FMT_Q4_0, 32, n, k, rng, name + ", 32 rows", 0.02 / 4)
    _sampled_matmul_check(be, nx.FMT_Q4_0, 1, n, k, rng, name + ", 1 row", 0.02 / 4)


# The packed kernels at the configs' real shapes and row counts: the streaming kernel at 32 rows (two activation
# tiles) and 64 rows (four), the many-rows kernel at 256 rows (a verification step) and 512 (a prompt chunk), in the
# formats the configs hold there. Full-size GPU product, oracle on a sample of the weight rows.
@pytest.mark.parametrize("what,fmt,n,k,m", [
    ("7B gate|up, Q4_0, 32 rows", nx.FMT_Q4_0, 22016, 4096, 32),
    ("7B gate|up, Q4_0, 512 rows", nx.FMT_Q4_0, 22016, 4096, 512),
    ("7B down, Q4_0, 512 rows", nx.FMT_Q4_0, 4096, 11008, 512),
    ("8B gate|up, Q8_0, 64 rows", nx.FMT_Q8_0, 28672, 4096, 64),
    ("8B down, Q8_0, 64 rows", nx.FMT_Q8_0, 4096, 14336, 64),
    ("8B down, Q8_0, 512 rows", nx.FMT_Q8_0, 4096, 14336, 512),
    ("7B gate|up, Q4_K, 32 rows", nx.FMT_Q4_K, 22016, 4096, 32),
    ("7B down, Q6_K, 32 rows", nx.FMT_Q6_K, 4096, 11008, 32),
    ("7B gate|up, Q6_K, 256 rows", nx.FMT_Q6_K, 22016, 4096, 256),
    ("7B down, Q6_K, 256 rows", nx.FMT_Q6_K, 4096, 11008, 256),
])
def test_packed_projections_at_the_configs_shapes(be, what, fmt, n, k, m):
    from oracle import quantize as qz
    rng = np.random.default_rng(n + k + m + fmt)
    if fmt in (nx.FMT_Q4_0, nx.FMT_Q8_0):
        w = _random_blocks(rng, fmt, n, k, 0.02 / (4 if fmt == nx.FMT_Q4_0 else 64))
    else:
        w = qz.random_quant(fmt, rng, n, k)
    a = (rng.standard_normal((m, k)) * (1.0 + 3.0 * (rng.random((1, k)) < 0.1))).astype(np.float32)
    da, dw = be.upload(a, permanent=True), be.upload(w, permanent=True)
    qw = be.qweight(fmt, dw, n, k)
    assert be.qweight_pack(qw)
    dout = be.alloc_permanent(m * n * 4)
    be.matmul_quant(fmt, da, dw, dout, None, m, n, k)
    kernel = be.last_matmul_kernel()
    assert kernel == ("qtiles_kernel" if m > 64 else "qstream_kernel"), kernel
    got = be.download(dout, (m, n), np.float32)
    assert np.all(np.isfinite(got))
    rows = np.unique(np.concatenate([rng.integers(0, n, 45), [0, 15, 16, n - 17, n - 1]]))
    mrows = np.unique(np.concatenate([rng.integers(0, m, 12), [0, m - 1]]))  # (the oracle's rows are independent)
    want = nx.matmul_quant(fmt, a[mrows], w[rows], len(mrows), len(rows), k)
    _close(got[np.ix_(mrows, rows)], want, 2e-5, 3e-6 * np.abs(want).max() + 1e-7, what)
    for p_ in (da, dw, dout):
        be.free(p_)
    be.reset_pool()


def test_paged_attention_at_full_context_and_head_geometry(be):
    """7B geometry (32 x 128 heads, MHA) with contexts at the configs' upper clip (4096), one short of it, a
    multiple of the 512-token split and the lower clip; 8B geometry (32 / 8 heads) likewise. Whole heads of
    every sequence against the oracle."""
    rng = np.random.default_rng(403)
    bs = 16
    for hq, hk, d in ((32, 32, 128), (32, 8, 128)):
        lens = np.array([4096, 4095, 1024, 64, 513], dtype=np.int32)
        nblk = [(int(L) + bs - 1) // bs for L in lens]
        nblocks = sum(nblk) + 3
        elems = nblocks * 2 * bs * hk * d
        pool = nx.f32_to_f16_array(rng.standard_normal(elems).astype(np.float32))
        perm = rng.permutation(nblocks)
        mb = max(nblk)
        tables = np.zeros((len(lens), mb), dtype=np.int32)
        off = 0
        for i, nb in enumerate(nblk):
            tables[i, :nb] = perm[off:off + nb]
            off += nb
        q = rng.standard_normal((len(lens), hq, d)).astype(np.float32)
        sc = np.float32(1 / math.sqrt(d))
        dq, dpool, dt, dl = be.upload(q), be.upload(pool, permanent=True), be.upload(tables), be.upload(lens)
        do = be.alloc(q.nbytes)
        be.sdpa_paged_decode_ragged(dq, dpool, True, dt, dl, do, len(lens), mb, bs, hq, hk, d, sc, int(lens.max()))
        got = be.download(do, q.shape, np.float32)
        for i, L in enumerate(lens):
            nb = nblk[i]
            want = nx.sdpa_paged_decode(q[i], pool, tables[i, :nb], nb, bs, hq, hk, d, sc, int(L) - (nb - 1) * bs)
            _close(got[i], want.reshape(hq, d), 1e-5, 3e-6, "context %d, %d/%d heads" % (L, hq, hk))
        be.free(dpool)
        be.reset_pool()


def test_prompt_chunk_of_512_at_position_3584_8b_geometry(be):
    """Benchmark config 4's largest later chunk: 512 query rows at start position 3584 (the last chunk of a
    4096-token prompt), 32 / 8 heads of 128, F16 pool, on the tiled multi-query kernel. Sampled rows (tile edges, the
    first and the last) against the oracle's per-row attention; every row against the single-query split-KV decode
    kernel of the same library, which was checked against the oracle at these lengths above."""
    rng = np.random.default_rng(405)
    bs, hq, hk, d, start, qn = 16, 32, 8, 128, 3584, 512
    nb = (start + qn) // bs
    nblocks = nb + 5
    pool = nx.f32_to_f16_array(rng.standard_normal(nblocks * 2 * bs * hk * d).astype(np.float32))
    bt = rng.permutation(nblocks)[:nb].astype(np.int32)
    q = rng.standard_normal((qn, hq, d)).astype(np.float32)
    kvl = np.arange(start + 1, start + qn + 1, dtype=np.int32)
    sc = np.float32(1 / math.sqrt(d))
    dq, dpool, dbt, dk = be.upload(q), be.upload(pool, permanent=True), be.upload(bt), be.upload(kvl)
    do = be.alloc(q.nbytes)
    be.sdpa_paged_decode_multiquery(dq, dpool, dbt, do, dk, nb, bs, hq, hk, d, sc, qn, pool_is_f16=True)
    got = be.download(do, q.shape, np.float32)
    for i in (0, 1, 63, 64, 255, 256, 510, 511):
        L = int(kvl[i])
        n_i = (L + bs - 1) // bs
        want = nx.sdpa_paged_decode(q[i], pool, bt[:n_i], n_i, bs, hq, hk, d, sc, L - (n_i - 1) * bs)
        _close(got[i], want.reshape(hq, d), 1e-5, 3e-6, "chunk row %d" % i)
    # all 512 rows as 512 one-query sequences that share the table
    tables = np.tile(bt, (qn, 1))
    dt, do2 = be.upload(tables), be.alloc(q.nbytes)
    be.sdpa_paged_decode_ragged(dq, dpool, True, dt, dk, do2, qn, nb, bs, hq, hk, d, sc, start + qn)
    ref = be.download(do2, q.shape, np.float32)
    _close(got, ref, 2e-5, 6e-6, "tiled chunk against the split-KV decode kernel")
    be.free(dpool)
    be.reset_pool()


def test_pack_batch_at_maximum_batch_and_context(be):
    """The packing kernel at 64 sequences whose positions sit on every kind of boundary up to 4096 tokens:
    bit-exact against the host pool's own bookkeeping."""
    from oracle import host_logic as hl
    rng = np.random.default_rng(404)
    bs, batch = 16, 64
    mb = 4096 // bs + 2
    pos = np.concatenate([[0, 15, 16, 4095, 4080, 4079, 511, 512], rng.integers(0, 4096, batch - 8)]).astype(np.int32)
    nblocks = int(sum(p // bs + 2 for p in pos))
    pool = hl.GPUBlockPool(1, 1, 1, bs, nblocks)
    tables = np.zeros((batch, mb), dtype=np.int32)
    num_blocks = np.zeros(batch, dtype=np.int32)
    for i, p in enumerate(pos):
        pool.create_sequence(i)
        if p > 0:
            pool.store_kv_slots(0, i, 0, int(p))
        bt = pool.seqs[i].block_tables[0]
        tables[i, :len(bt)] = bt
        num_blocks[i] = len(bt)
    free = np.array(pool.free_lists[0], dtype=np.int32)
    d_tab, d_nb = be.upload(tables), be.upload(num_blocks)
    d_free, d_fc = be.upload(np.concatenate([free, np.zeros(batch, dtype=np.int32)])), be.upload(np.array([len(free)], dtype=np.int32))
    d_slots, d_pos = be.upload(np.arange(batch, dtype=np.int32)), be.upload(pos)
    i4 = lambda n: be.alloc(n * 4)
    d_cu, d_tp, d_sm, d_kl, d_st = i4(batch + 1), i4(batch), i4(batch), i4(batch), i4(4)
    be.pack_batch(d_slots, d_pos, 0, batch, batch, d_tab, mb, d_nb, d_free, d_fc, bs, d_cu, d_tp, d_sm, d_kl, d_st)
    want_slots = []
    for i, p in enumerate(pos):
        blk, off = pool.store_kv_slots(0, i, int(p), 1)[0]
        want_slots.append(blk * bs + off)
    assert be.download(d_st, (1,), np.int32)[0] == 0
    assert np.array_equal(be.download(d_sm, (batch,), np.int32), np.array(want_slots, dtype=np.int32))
    assert np.array_equal(be.download(d_kl, (batch,), np.int32), pos + 1)
    assert np.array_equal(be.download(d_tp, (batch,), np.int32), pos)
    got_tab = be.download(d_tab, (batch, mb), np.int32)
    for i in range(batch):
        bt = pool.seqs[i].block_tables[0]
        assert got_tab[i, :len(bt)].tolist() == bt
    assert int(be.download(d_fc, (1,), np.int32)[0]) == len(pool.free_lists[0])
    assert be.download(d_free, (len(pool.free_lists[0]),), np.int32).tolist() == pool.free_lists[0]
    be.reset_pool()


def test_north_star_shape_batched_equals_sequence_by_sequence(be):
    """The whole north-star model (7B shape, 32 layers, Q4_0, 32 ragged sequences up to 4096 tokens) is beyond the
    oracle's reach, but the reference's batched decode is by definition its single-sequence decode in a loop
    (runtime/decode.go:612-654): the batched step (MFMA GEMMs, work-list attention, fused blocks) must give each
    sequence the logits the one-sequence path (matrix-vector kernels, one-row attention) gives it alone, within the
    logits budget, and the same greedy token; checked for a sample of the sequences over two steps."""
    import os, sys
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    import bench
    ctx = bench.ragged_contexts()
    mr, ids = bench.build_model(be, ctx, 8, 32)
    mr2, ids2 = bench.build_model(be, ctx, 8, 32)           # same seeds: the same weights and contexts
    rng = np.random.default_rng(405)
    toks = rng.integers(0, 32000, len(ids)).tolist()
    pos = list(ctx)
    sample = [0, int(np.argmax(ctx)), int(np.argmin(ctx)), 17]
    for step in range(2):
        got, am = mr.decode_with_paged_kv_batched(toks, ids, pos)
        for i in sample:
            one, am1 = mr2.decode_with_paged_kv_batched([toks[i]], [ids2[i]], [pos[i]])
            err = np.abs(got[i].astype(np.float64) - one[0].astype(np.float64))
            assert np.all(err <= 1e-2 + 1e-3 * np.abs(one[0])), "sequence %d step %d: max err %.3e" % (i, step, err.max())
            assert int(am[i]) == int(am1[0])
        toks = [int(a) for a in am]
        pos = [p + 1 for p in pos]
    mr.close()
    mr2.close()
