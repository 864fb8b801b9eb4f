"""vx_sdpa_paged_decode_ragged_noalloc (fixed partial-sum area, no device allocation) against
vx_sdpa_paged_decode_ragged on the same inputs, through the C ABI: bit-identical outputs on two calls in
a row, the second smaller than the first, plus the size and geometry refusals. The allocating entry point
is itself compared with the oracle here, so the file stands on its own when run alone."""
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


def _case(rng, be, lens, hq, hk, d, nblocks, dpool, pool, mb=None):
    bs = 16
    B = len(lens)
    mb = mb or max((L + bs - 1) // bs for L in lens) + 2
    perm = rng.permutation(nblocks)
    mat = np.zeros((B, mb), dtype=np.int32)
    off = 0
    for i, L in enumerate(lens):
        nb = (L + bs - 1) // bs
        mat[i, :nb] = perm[off:off + nb]
        off += nb
    q = rng.standard_normal((B, hq, d)).astype(np.float32)
    sc = np.float32(1 / math.sqrt(d))
    dq, dmat, dl = be.upload(q), be.upload(mat), be.upload(np.array(lens, dtype=np.int32))
    o_ref, o_new = be.alloc(q.nbytes), be.alloc(q.nbytes)
    args = (dq, dpool, True, dmat, dl)
    tail = (B, mb, bs, hq, hk, d, sc, mb * bs)
    be.sdpa_paged_decode_ragged(*args, o_ref, *tail)
    be.sdpa_paged_decode_ragged_noalloc(*args, o_new, *tail)
    ref = be.download(o_ref, q.shape, np.float32)
    new = be.download(o_new, q.shape, np.float32)
    want = nx.sdpa_paged_decode_batched(q, pool, mat, bs, hq, hk, d, sc, np.array(lens, dtype=np.int32))
    err = np.abs(ref.astype(np.float64) - want.astype(np.float64))
    assert np.all(err <= 3e-6 + 1e-5 * np.abs(want)), "allocating entry point against the oracle: %.3e" % err.max()
    assert np.array_equal(ref.view(np.uint32), new.view(np.uint32)), "fixed-area result differs in its bits"


def test_noalloc_matches_allocating_entry_point_twice(be):
    rng = np.random.default_rng(77)
    hq, hk, d, nblocks = 8, 2, 128, 700
    pool = nx.f32_to_f16_array(rng.standard_normal(nblocks * 2 * 16 * hk * d).astype(np.float32))
    dpool = be.upload(pool)
    # first call: nine ragged sequences, up to five 512-token splits each
    _case(rng, be, [1, 16, 511, 512, 513, 1300, 2100, 2049, 77], hq, hk, d, nblocks, dpool, pool)
    # second call, smaller in every dimension: the area still holds the first call's partial sums
    _case(rng, be, [700, 3, 512], hq, hk, d, nblocks, dpool, pool)
    be.reset_pool()


def test_noalloc_refuses_what_does_not_fit(be):
    from vexel_amd.backend import VexelError
    rng = np.random.default_rng(78)
    hq, hk, d = 32, 32, 128
    bs, B, mb = 16, 64, 512           # 64 x 32 heads x 16 splits x 130 floats = 17 MB of partial sums
    dq = be.upload(np.zeros((B, hq, d), dtype=np.float32))
    dpool = be.upload(np.zeros(2 * bs * hk * d, dtype=np.uint16))
    dmat = be.upload(np.zeros((B, mb), dtype=np.int32))
    dl = be.upload(np.ones(B, dtype=np.int32))
    do = be.alloc(B * hq * d * 4)
    with pytest.raises(VexelError, match="fixed area holds"):
        be.sdpa_paged_decode_ragged_noalloc(dq, dpool, True, dmat, dl, do, B, mb, bs, hq, hk, d, 0.1, mb * bs)
    need, cap = be.sdpa_paged_decode_ragged_noalloc_bytes(B, hq, hk, d, mb * bs)
    assert cap == 8 << 20 and need == B * hq * 16 * (d + 2) * 4
    # a float32 pool has no streaming kernel: refused rather than sent to the allocating path
    with pytest.raises(VexelError, match="streaming kernel"):
        be.sdpa_paged_decode_ragged_noalloc(dq, dpool, False, dmat, dl, do, 2, mb, bs, hq, hk, d, 0.1, 64)
    with pytest.raises(VexelError, match="null pointer"):
        be.sdpa_paged_decode_ragged_noalloc(dq, dpool, True, dmat, dl, None, 2, mb, bs, hq, hk, d, 0.1, 64)
    be.reset_pool()


def test_noalloc_grouped_queries_at_the_limit_of_the_area(be):
    """Grouped queries run on splits of 256 tokens (128 for small batches), so they need two to four times the
    partial sums of one query head per KV head: the query function gives the exact figure, a call just inside the
    area runs and matches the allocating entry point bit for bit, the 8B shape at 32 x 4096 tokens is refused."""
    from vexel_amd.backend import VexelError
    rng = np.random.default_rng(79)
    hq, hk, d, bs = 32, 8, 128, 16
    need, cap = be.sdpa_paged_decode_ragged_noalloc_bytes(32, hq, hk, d, 4096)
    assert need == 32 * hq * 16 * (d + 2) * 4 and need > cap          # 16 splits of 256 tokens: 8.5 MB
    # the largest batch of 3800-token tables that fits: 15 splits of 256 tokens
    B = cap // (hq * 15 * (d + 2) * 4)
    mb = 3800 // bs + 1
    need, _ = be.sdpa_paged_decode_ragged_noalloc_bytes(B, hq, hk, d, mb * bs)
    assert need <= cap < be.sdpa_paged_decode_ragged_noalloc_bytes(B + 1, hq, hk, d, mb * bs)[0]
    lens = [int(x) for x in rng.integers(1, 3800, B)]
    lens[0], lens[1] = 3800, 256
    nblocks = sum((L + bs - 1) // bs for L in lens) + 4
    pool = nx.f32_to_f16_array(rng.standard_normal(nblocks * 2 * bs * hk * d).astype(np.float32))
    dpool = be.upload(pool)
    _case(rng, be, lens, hq, hk, d, nblocks, dpool, pool, mb=mb)
    dq = be.upload(np.zeros((32, hq, d), dtype=np.float32))
    dmat = be.upload(np.zeros((32, 256), dtype=np.int32))
    dl = be.upload(np.ones(32, dtype=np.int32))
    do = be.alloc(32 * hq * d * 4)
    with pytest.raises(VexelError, match="fixed area holds"):
        be.sdpa_paged_decode_ragged_noalloc(dq, dpool, True, dmat, dl, do, 32, 256, bs, hq, hk, d, 0.1, 4096)
    be.reset_pool()
