"""GPU parity of the decode-batch GEMM over load-time packed matrices of the six block formats (vx_qweight_pack): the packed
copy dequantises to the reference's values bit for bit, the products match the CPU oracle's MatMulQ4_0 / Q8_0 / Q4_K / Q6_K / Q5_0 / Q5_K
(backend/cpu/cpu.go:842-911) to float32 summation order on every cut of the matrix the planner makes, a row's bits
do not depend on the batch it sits in (2 .. 32 rows; 33 .. 64 rows), and the fused decode blocks give the oracle's
layer with packed weights."""
import numpy as np
import pytest

from oracle import numerics as nx
from oracle import quantize as qz

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def be():
    from vexel_amd.backend import HipBackend
    b = HipBackend(0)
    yield b
    b.close()


def _close(got, want, rtol, atol, what=""):
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    lim = atol + rtol * np.abs(want.astype(np.float64))
    assert np.all(err <= lim), "%s: max err %.3e (limit %.3e at worst element)" % (
        what, err.max(), lim.reshape(-1)[err.argmax()])


FMTS = [nx.FMT_Q4_0, nx.FMT_Q8_0, nx.FMT_Q6_K, nx.FMT_Q4_K, nx.FMT_Q5_0, nx.FMT_Q5_K]


def _packed(be, w, n, k, fmt=nx.FMT_Q4_0):
    dw = be.upload(w, permanent=True)
    qw = be.qweight(fmt, dw, n, k)
    assert be.qweight_pack(qw)
    assert be.qweight_is_packed(qw)
    return dw, qw


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("n,k", [(16, 256), (48, 1024), (1040, 512)])
def test_packed_copy_dequantises_bit_exact(be, n, k, fmt):
    rng = np.random.default_rng(n + k)
    w = qz.random_quant(fmt, rng, n, k)
    if fmt == nx.FMT_Q5_0:
        w.reshape(-1)[2:22] = rng.integers(0, 256, 20, dtype=np.uint8)     # arbitrary fifth bits and nibbles in one block
    elif fmt == nx.FMT_Q5_K:
        w.reshape(-1)[4:176] = rng.integers(0, 256, 172, dtype=np.uint8)   # arbitrary scale / min fields, fifth bits and nibbles
    elif fmt == nx.FMT_Q4_K:
        w.reshape(-1)[4:144] = rng.integers(0, 256, 140, dtype=np.uint8)   # arbitrary scale / min fields and codes in one super-block
    elif fmt == nx.FMT_Q6_K:
        w.reshape(-1)[0:208] = rng.integers(0, 256, 208, dtype=np.uint8)   # arbitrary codes and scale bytes in one super-block
    else:
        w.reshape(-1)[2:34] = rng.integers(0, 256, 32, dtype=np.uint8)   # every code position carries arbitrary codes
    dw, qw = _packed(be, w, n, k, fmt)
    dst = be.alloc(n * k * 4)
    be.dequantize_packed(qw, dst)
    got = be.download(dst, (n * k,), np.float32)
    want = nx.dequantize(fmt, w, n * k)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    be.free(dw)
    assert not be.qweight_is_packed(qw)                          # the copy goes with the matrix
    be.reset_pool()


def test_pack_refuses_other_formats_and_shapes(be):
    rng = np.random.default_rng(0)
    w = qz.random_quant(nx.FMT_BF16, rng, 32, 256)
    dw = be.upload(w, permanent=True)
    assert not be.qweight_pack(be.qweight(nx.FMT_BF16, dw, 32, 256))
    assert not be.qweight_pack(be.qweight(nx.FMT_Q4_0, dw, 24, 256))     # rows not a multiple of 16
    assert not be.qweight_pack(be.qweight(nx.FMT_Q4_0, dw, 32, 128))     # K not a multiple of 256
    be.free(dw)


# (n, k): one tile; K slices of one and two half chunks per wave; slices with an odd share of half chunks;
# more tiles than workgroups in a slice; a 7B down-projection's K
@pytest.mark.parametrize("n,k", [(16, 256), (80, 1024), (96, 2048), (1040, 2304), (4112, 512), (64, 4352), (208, 11008)])
@pytest.mark.parametrize("m", [2, 5, 16, 17, 32, 33, 48, 64])
@pytest.mark.parametrize("fmt", FMTS)
def test_matmul_packed_vs_oracle(be, n, k, m, fmt):
    rng = np.random.default_rng(n * 7 + k + m)
    w = qz.random_quant(fmt, rng, n, k)
    a = (rng.standard_normal((m, k)) * (1.0 + 3.0 * (rng.random((1, k)) < 0.1))).astype(np.float32)
    want = nx.matmul_quant(fmt, a, w, m, n, k)
    dw, qw = _packed(be, w, n, k, fmt)
    da = be.upload(a)
    dout = be.alloc(m * n * 4)
    be.matmul_quant(fmt, da, dw, dout, None, m, n, k)
    got = be.download(dout, (m, n), np.float32)
    scale = np.abs(want).max()
    _close(got, want, 2e-5, 2e-6 * scale + 1e-7, "packed matmul %dx%dx%d" % (m, n, k))
    # the unpacked path on the same inputs: float32 summation order apart
    be.qweight_unpack(qw)
    be.matmul_quant(fmt, da, dw, dout, None, m, n, k)
    plain = be.download(dout, (m, n), np.float32)
    _close(got, plain, 0, 3e-6 * scale + 1e-7, "packed vs unpacked")
    be.free(dw)
    be.reset_pool()


# more than 64 rows: the kernel whose waves own weight tiles and share the activation through LDS
# (n, k): fewer tiles than a workgroup's waves own; tiles not a multiple of a wave's; many K slices; a long K
@pytest.mark.parametrize("n,k", [(16, 256), (80, 1024), (1040, 2304), (4112, 512), (208, 11008)])
@pytest.mark.parametrize("m", [65, 96, 130, 256])
@pytest.mark.parametrize("fmt", FMTS)
def test_matmul_packed_many_rows_vs_oracle(be, n, k, m, fmt):
    rng = np.random.default_rng(n * 5 + k + m)
    w = qz.random_quant(fmt, rng, n, k)
    a = (rng.standard_normal((m, k)) * (1.0 + 3.0 * (rng.random((1, k)) < 0.1))).astype(np.float32)
    want = nx.matmul_quant(fmt, a, w, m, n, k)
    dw, qw = _packed(be, w, n, k, fmt)
    da = be.upload(a)
    dout = be.alloc(m * n * 4)
    be.matmul_quant(fmt, da, dw, dout, None, m, n, k)
    got = be.download(dout, (m, n), np.float32)
    scale = np.abs(want).max()
    _close(got, want, 2e-5, 2e-6 * scale + 1e-7, "packed matmul %dx%dx%d" % (m, n, k))
    res = rng.standard_normal((m, n)).astype(np.float32)
    dres = be.upload(res)
    be.matmul_quant(fmt, da, dw, dout, dres, m, n, k)
    assert np.array_equal(be.download(dout, (m, n), np.float32).view(np.uint32), (res + got).view(np.uint32))
    be.qweight_unpack(qw)
    be.matmul_quant(fmt, da, dw, dout, None, m, n, k)
    plain = be.download(dout, (m, n), np.float32)
    _close(got, plain, 0, 3e-6 * scale + 1e-7, "packed vs unpacked")
    be.free(dw)
    be.reset_pool()


@pytest.mark.parametrize("fmt", FMTS)
def test_matmul_packed_many_rows_independent_of_batch(be, fmt):
    """A row has the same bits in any batch with the same number of 64-row groups (the K slicing depends on that
    number beside the matrix' shape): 65 .. 128 rows here."""
    rng = np.random.default_rng(12)
    n, k = 208, 4096
    w = qz.random_quant(fmt, rng, n, k)
    a = rng.standard_normal((128, k)).astype(np.float32)
    dw, qw = _packed(be, w, n, k, fmt)
    da = be.upload(a)

    def batch(first, rows):
        d = be.alloc(rows * n * 4)
        be.matmul_quant(fmt, da + first * k * 4, dw, d, None, rows, n, k)
        return be.download(d, (rows, n), np.float32)

    full = batch(0, 128)
    for first, rows in ((0, 65), (11, 90), (40, 88), (1, 127)):
        part = batch(first, rows)
        assert np.array_equal(part.view(np.uint32), full[first:first + rows].view(np.uint32)), (first, rows)
    be.free(dw)
    be.reset_pool()


@pytest.mark.parametrize("fmt", FMTS)
def test_matmul_packed_rows_independent_of_batch(be, fmt):
    """A row has the same bits in a batch of 2, of 16, of 17 and of 32 rows (the cut of the matrix depends on its
    shape and the device only; 16 rows and fewer run the one-tile form of the kernel), and in a batch of 33, of 40
    and of 64 rows (four activation tiles a step: K is cut into narrower slices there)."""
    rng = np.random.default_rng(11)
    n, k = 208, 4096
    w = qz.random_quant(fmt, rng, n, k)
    a = rng.standard_normal((64, k)).astype(np.float32)
    dw, qw = _packed(be, w, n, k, fmt)
    da = be.upload(a)

    def batch(first, rows):
        d = be.alloc(rows * n * 4)
        be.matmul_quant(fmt, da + first * k * 4, dw, d, None, rows, n, k)
        return be.download(d, (rows, n), np.float32)

    full = batch(0, 32)
    for first, rows in ((0, 2), (5, 2), (30, 2), (0, 16), (3, 17), (16, 16), (9, 7)):
        part = batch(first, rows)
        assert np.array_equal(part.view(np.uint32), full[first:first + rows].view(np.uint32)), (first, rows)
    full64 = batch(0, 64)
    for first, rows in ((0, 33), (20, 40), (31, 33), (7, 57)):
        part = batch(first, rows)
        assert np.array_equal(part.view(np.uint32), full64[first:first + rows].view(np.uint32)), (first, rows)
    scale = np.abs(full).max()
    _close(full64[:32], full, 0, 3e-6 * scale, "a row in 64 against the same row in 32")
    res = rng.standard_normal((32, n)).astype(np.float32)
    dres, d = be.upload(res), be.alloc(32 * n * 4)
    be.matmul_quant(fmt, da, dw, d, dres, 32, n, k)
    assert np.array_equal(be.download(d, (32, n), np.float32).view(np.uint32), (res + full).view(np.uint32))
    be.free(dw)
    be.reset_pool()


def test_default_configuration_takes_the_kernels_the_benchmark_reports(be):
    """With no environment switch set, a packed matrix runs the streaming kernel at 2 .. 64 rows and the many-rows
    kernel beyond, one row the matrix-vector kernel, and an unpacked matrix the kernels over the GGUF rows: the paths
    bench.py times are the paths a default process takes."""
    import os
    if [k for k in os.environ if k.startswith("VEXEL_HIP_")]:
        pytest.skip("a VEXEL_HIP_* switch is set: this is not the default configuration")
    rng = np.random.default_rng(21)
    n, k = 256, 4096
    w = qz.random_quant(nx.FMT_Q4_0, rng, n, k)
    a = rng.standard_normal((256, k)).astype(np.float32)
    dw, qw = _packed(be, w, n, k)
    da, dout = be.upload(a), be.alloc(256 * n * 4)
    for m, want in ((1, "qmatvec_kernel"), (2, "qstream_kernel"), (32, "qstream_kernel"), (64, "qstream_kernel"),
                    (65, "qtiles_kernel"), (256, "qtiles_kernel")):
        be.matmul_quant(nx.FMT_Q4_0, da, dw, dout, None, m, n, k)
        assert be.last_matmul_kernel() == want, (m, be.last_matmul_kernel())
    be.qweight_unpack(qw)
    for m, want in ((1, "qmatvec_kernel"), (32, "qgemm_wave_kernel"), (256, "qgemm_kernel")):
        be.matmul_quant(nx.FMT_Q4_0, da, dw, dout, None, m, n, k)
        assert be.last_matmul_kernel() == want, (m, be.last_matmul_kernel())
    be.free(dw)
    be.reset_pool()


def test_rewriting_the_matrix_drops_the_packed_copy(be):
    rng = np.random.default_rng(5)
    n, k, m = 64, 512, 8
    w1, w2 = qz.random_quant(nx.FMT_Q4_0, rng, n, k), qz.random_quant(nx.FMT_Q4_0, rng, n, k)
    a = rng.standard_normal((m, k)).astype(np.float32)
    dw, qw = _packed(be, w1, n, k)
    da, dout = be.upload(a), be.alloc(m * n * 4)
    be.to_device(dw, w2)                                         # new rows under the same address
    assert not be.qweight_is_packed(qw)
    be.matmul_q4_0(da, dw, dout, m, n, k)
    want = nx.matmul_quant(nx.FMT_Q4_0, a, w2, m, n, k)
    _close(be.download(dout, (m, n), np.float32), want, 2e-5, 2e-6 * np.abs(want).max() + 1e-7, "after rewrite")
    be.free(dw)
    be.reset_pool()


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("rows", [2, 7, 32, 64])
@pytest.mark.parametrize("hq,hk,d,hidden,ffn", [(8, 8, 64, 512, 1024), (8, 2, 128, 1024, 2816), (32, 32, 128, 4096, 1024)])
def test_fused_decode_blocks_with_packed_weights(be, rows, hq, hk, d, hidden, ffn, fmt):
    """RMSNorm -> Q|K|V -> RoPE -> KV store (one launch with the table of angles) and Wo -> residual -> RMSNorm ->
    gate|up -> SiLU*up -> down -> residual on packed weights against the oracle's operators."""
    rng = np.random.default_rng(rows + hq + hidden)
    bs, nblocks, theta, eps = 16, 8, 10000.0, 1e-5
    qd, kvd = hq * d, hk * d
    quant = {nx.FMT_Q4_0: qz.quantize_q4_0, nx.FMT_Q8_0: qz.quantize_q8_0, nx.FMT_Q5_0: qz.quantize_q5_0}.get(fmt)
    if fmt in (nx.FMT_Q6_K, nx.FMT_Q4_K, nx.FMT_Q5_K):
        mk = lambda n, k: qz.random_quant(fmt, rng, n, k, std=0.05).reshape(-1)
    else:
        mk = lambda n, k: quant((rng.standard_normal((n, k)) * 0.05).astype(np.float32)).reshape(-1)
    raw = {"wq": (mk(qd, hidden), qd, hidden), "wk": (mk(kvd, hidden), kvd, hidden), "wv": (mk(kvd, hidden), kvd, hidden),
           "wo": (mk(hidden, qd), hidden, qd), "w1": (mk(ffn, hidden), ffn, hidden), "w3": (mk(ffn, hidden), ffn, hidden),
           "w2": (mk(hidden, ffn), hidden, ffn)}
    dev, qws = {}, {}
    for name, (w, n, k) in raw.items():
        dev[name], qws[name] = _packed(be, w, n, k, fmt)
    x = rng.standard_normal((rows, hidden)).astype(np.float32)
    nw_attn = (1.0 + 0.1 * rng.standard_normal(hidden)).astype(np.float32)
    nw_ffn = (1.0 + 0.1 * rng.standard_normal(hidden)).astype(np.float32)
    positions = rng.integers(0, 100, rows).astype(np.int32)
    slots = rng.permutation(nblocks * bs)[:rows].astype(np.int32)
    per_block = 2 * bs * kvd
    pool0 = nx.f32_to_f16_array(rng.standard_normal(nblocks * per_block).astype(np.float32))

    # oracle
    h = nx.rmsnorm(x, nw_attn, rows, hidden, eps)
    q = nx.matmul_quant(fmt, h, raw["wq"][0], rows, qd, hidden)
    kk = nx.matmul_quant(fmt, h, raw["wk"][0], rows, kvd, hidden)
    vv = nx.matmul_quant(fmt, h, raw["wv"][0], rows, kvd, hidden)
    want_q, want_k = nx.rope_positions(q, kk, d, hq, hk, positions, d, theta, False)
    attn = rng.standard_normal((rows, qd)).astype(np.float32)
    x1 = nx.add(x, nx.matmul_quant(fmt, attn, raw["wo"][0], rows, hidden, qd))
    h2 = nx.rmsnorm(x1, nw_ffn, rows, hidden, eps)
    g = nx.matmul_quant(fmt, h2, raw["w1"][0], rows, ffn, hidden)
    u = nx.matmul_quant(fmt, h2, raw["w3"][0], rows, ffn, hidden)
    want_x = nx.add(x1, nx.matmul_quant(fmt, nx.silu_mul(g, u), raw["w2"][0], rows, hidden, ffn))

    # GPU
    dx, dnw, dnf = be.upload(x, permanent=True), be.upload(nw_attn, permanent=True), be.upload(nw_ffn, permanent=True)
    dpos, dslots = be.upload(positions, permanent=True), be.upload(slots, permanent=True)
    dpool, dq = be.upload(pool0, permanent=True), be.alloc_permanent(rows * qd * 4)
    be.rope_table_prepare(dpos, rows, d, theta)
    be.decode_attn_qkv(dx, dnw, eps, False, qws["wq"], qws["wk"], qws["wv"], rows, dpos, dslots, dpool, True, hq, hk, d, bs,
                       theta, dq)
    got_q = be.download(dq, (rows, qd), np.float32)
    _close(got_q, want_q, 2e-4, 2e-5 * np.abs(want_q).max(), "Q")
    pool = nx.f16_to_f32_array(be.download(dpool, (nblocks * per_block,), np.uint16))
    for r in range(rows):
        blk, off = divmod(int(slots[r]), bs)
        gk = pool[blk * per_block + off * kvd: blk * per_block + (off + 1) * kvd]
        gv = pool[blk * per_block + bs * kvd + off * kvd: blk * per_block + bs * kvd + (off + 1) * kvd]
        _close(gk, nx.f16_to_f32_array(nx.f32_to_f16_array(want_k[r])), 2e-3, 2e-3 * np.abs(want_k).max(), "K row %d" % r)
        _close(gv, nx.f16_to_f32_array(nx.f32_to_f16_array(vv[r])), 2e-3, 2e-3 * np.abs(vv).max(), "V row %d" % r)
    dattn = be.upload(attn, permanent=True)
    be.decode_ffn(dattn, dx, qws["wo"], dnf, eps, qws["w1"], qws["w3"], qws["w2"], rows)
    got_x = be.download(dx, (rows, hidden), np.float32)
    _close(got_x, want_x, 2e-4, 2e-5 * np.abs(want_x).max(), "layer output")
    for p in list(dev.values()) + [dx, dnw, dnf, dpos, dslots, dpool, dq, dattn]:
        be.free(p)
    be.reset_pool()


@pytest.mark.parametrize("fqk", [nx.FMT_Q4_K, nx.FMT_Q5_K])
@pytest.mark.parametrize("rows", [2, 7, 17, 32, 40])
@pytest.mark.parametrize("hq,hk,d,hidden", [(8, 2, 128, 1024), (32, 32, 128, 4096), (32, 8, 128, 4096), (24, 1, 64, 2048)])
def test_fused_qkv_with_packed_v_in_q6_k(be, rows, hq, hk, d, hidden, fqk):
    """attn_q and attn_k in Q4_K or Q5_K beside attn_v in Q6_K, as the K-quant mixes of GGUF files hold them, all
    three packed: up to 32 rows one launch computes the three (row groups shared out between the two formats),
    beyond that V takes a launch of its own; either way RMSNorm -> Q|K|V -> RoPE -> KV store gives what the oracle's
    operators give."""
    import os
    rng = np.random.default_rng(rows * 31 + hq + hidden + fqk)
    bs, nblocks, theta, eps = 16, 8, 10000.0, 1e-5
    qd, kvd = hq * d, hk * d
    fm = {"wq": fqk, "wk": fqk, "wv": nx.FMT_Q6_K}
    shapes = {"wq": (qd, hidden), "wk": (kvd, hidden), "wv": (kvd, hidden)}
    raw = {n: qz.random_quant(fm[n], rng, *shapes[n], std=0.05).reshape(-1) for n in shapes}
    dev, qws = {}, {}
    for name in shapes:
        dev[name], qws[name] = _packed(be, raw[name], *shapes[name], fm[name])
    x = rng.standard_normal((rows, hidden)).astype(np.float32)
    nw = (1.0 + 0.1 * rng.standard_normal(hidden)).astype(np.float32)
    positions = rng.integers(0, 100, rows).astype(np.int32)
    slots = rng.permutation(nblocks * bs)[:rows].astype(np.int32)
    per_block = 2 * bs * kvd
    pool0 = nx.f32_to_f16_array(rng.standard_normal(nblocks * per_block).astype(np.float32))

    h = nx.rmsnorm(x, nw, rows, hidden, eps)
    q = nx.matmul_quant(fqk, h, raw["wq"], rows, qd, hidden)
    kk = nx.matmul_quant(fqk, h, raw["wk"], rows, kvd, hidden)
    vv = nx.matmul_quant(nx.FMT_Q6_K, h, raw["wv"], rows, kvd, hidden)
    want_q, want_k = nx.rope_positions(q, kk, d, hq, hk, positions, d, theta, False)

    dx, dnw = be.upload(x, permanent=True), be.upload(nw, permanent=True)
    dpos, dslots = be.upload(positions, permanent=True), be.upload(slots, permanent=True)
    dpool, dq = be.upload(pool0, permanent=True), be.alloc_permanent(rows * qd * 4)
    be.rope_table_prepare(dpos, rows, d, theta)
    be.decode_attn_qkv(dx, dnw, eps, False, qws["wq"], qws["wk"], qws["wv"], rows, dpos, dslots, dpool, True, hq, hk, d, bs,
                       theta, dq)
    if not [k for k in os.environ if k.startswith("VEXEL_HIP_")] and rows <= 32 and hidden % 1024 == 0:
        assert be.last_matmul_kernel() == "qstream_mixed_kernel", be.last_matmul_kernel()
    got_q = be.download(dq, (rows, qd), np.float32)
    _close(got_q, want_q, 2e-4, 2e-5 * np.abs(want_q).max(), "Q")
    pool = nx.f16_to_f32_array(be.download(dpool, (nblocks * per_block,), np.uint16))
    untouched = np.ones(nblocks * per_block, dtype=bool)
    for r in range(rows):
        blk, off = divmod(int(slots[r]), bs)
        ko, vo = blk * per_block + off * kvd, blk * per_block + bs * kvd + off * kvd
        untouched[ko:ko + kvd] = False
        untouched[vo:vo + kvd] = False
        _close(pool[ko:ko + kvd], nx.f16_to_f32_array(nx.f32_to_f16_array(want_k[r])), 2e-3, 2e-3 * np.abs(want_k).max(), "K row %d" % r)
        _close(pool[vo:vo + kvd], nx.f16_to_f32_array(nx.f32_to_f16_array(vv[r])), 2e-3, 2e-3 * np.abs(vv).max(), "V row %d" % r)
    assert np.array_equal(pool[untouched], nx.f16_to_f32_array(pool0)[untouched])
    for p in list(dev.values()) + [dx, dnw, dpos, dslots, dpool, dq]:
        be.free(p)
    be.reset_pool()
