"""GPU parity: every C-ABI compute entry point against the CPU oracle on the same seeded
inputs. Integer/byte results (dequantised weights, scatter layout, argmax, packing) are
compared bit-exactly; floating point within the stated tolerances."""
import math

import numpy as np
import pytest

from oracle import numerics as nx
from oracle import quantize as qz
from oracle import host_logic as hl

pytestmark = pytest.mark.gpu

FMTS = [nx.FMT_Q4_0, nx.FMT_Q8_0, nx.FMT_Q4_K, nx.FMT_Q6_K]
FMTS_MFMA = FMTS + [nx.FMT_Q5_0, nx.FMT_Q5_K]      # the formats with matrix-vector and MFMA kernels


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


# ------------------------------------------------------------------ dequant: bit exact
@pytest.mark.parametrize("fmt", FMTS)
def test_dequantize_bit_exact(be, fmt):
    rng = np.random.default_rng(100 + fmt)
    n, k = 37, 1024
    w = qz.random_quant(fmt, rng, n, k)
    # adversarial header bits: random f16 scales including subnormals and negative values
    raw = w.reshape(-1).copy()
    want = nx.dequantize(fmt, raw, n * k)
    dw = be.upload(raw)
    dout = be.alloc(n * k * 4)
    be.dequantize(fmt, dw, dout, n * k)
    got = be.download(dout, (n * k,), np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    be.reset_pool()


@pytest.mark.parametrize("fmt", FMTS)
def test_dequantize_all_byte_patterns(be, fmt):
    """Blocks filled with every byte value, finite random scales: covers every code."""
    rng = np.random.default_rng(7)
    bb, be_ = nx.BLOCK_BYTES[fmt], nx.BLOCK_ELEMS[fmt]
    nblk = 512
    raw = rng.integers(0, 256, size=(nblk, bb), dtype=np.uint8)
    # keep f16 headers finite (exponent != 31) so NaN payload rules do not enter
    def fix(col):
        hi = raw[:, col + 1]
        bad = (hi & 0x7C) == 0x7C
        raw[bad, col + 1] = hi[bad] & 0xBF
    if fmt in (nx.FMT_Q4_0, nx.FMT_Q8_0):
        fix(0)
    elif fmt == nx.FMT_Q4_K:
        fix(0); fix(2)
    else:
        fix(208)
    want = nx.dequantize(fmt, raw.reshape(-1), nblk * be_)
    d = be.upload(raw)
    o = be.alloc(nblk * be_ * 4)
    be.dequantize(fmt, d, o, nblk * be_)
    got = be.download(o, (nblk * be_,), np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    be.reset_pool()


@pytest.mark.parametrize("fmt", [nx.FMT_Q5_0, nx.FMT_Q5_K, nx.FMT_BF16])
def test_dequantize_other_formats_bit_exact(be, fmt):
    """Q5_0, Q5_K, BF16 (pkg/gguf/dequant.go:100-145, 423-500, 215-228): random weights, then blocks of random
    bytes with finite f16 headers (every code, every fifth-bit position)."""
    rng = np.random.default_rng(300 + fmt)
    n, k = 11, 1024
    raw = qz.random_quant(fmt, rng, n, k).reshape(-1).copy()
    bb, be_ = nx.BLOCK_BYTES[fmt], nx.BLOCK_ELEMS[fmt]
    rnd = rng.integers(0, 256, size=(2048 // be_ * 8, bb), dtype=np.uint8)
    if fmt == nx.FMT_BF16:
        rnd[(rnd[:, 1] & 0x7F) == 0x7F, 1] &= 0xBF          # no NaN / Inf patterns
    else:
        for col in ((0,) if fmt == nx.FMT_Q5_0 else (0, 2)):
            hi = rnd[:, col + 1]
            bad = (hi & 0x7C) == 0x7C
            rnd[bad, col + 1] = hi[bad] & 0xBF
    for data in (raw, rnd.reshape(-1)):
        cnt = data.size // bb * be_
        want = nx.dequantize(fmt, data, cnt)
        d = be.upload(data)
        o = be.alloc(cnt * 4)
        be.dequantize(fmt, d, o, cnt)
        got = be.download(o, (cnt,), np.float32)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    be.reset_pool()


@pytest.mark.parametrize("fmt", [nx.FMT_Q5_0, nx.FMT_Q5_K, nx.FMT_BF16])
@pytest.mark.parametrize("m", [1, 3, 8, 9, 32])
def test_matmul_other_formats_vs_oracle(be, fmt, m):
    """MatMulQ5_0 / MatMulQ5_K / MatMulBF16 (backend.go:65-80) against Dequantize + the naive product."""
    rng = np.random.default_rng(fmt * 100 + m)
    n, k = 70, 1536
    w = qz.random_quant(fmt, rng, n, k)
    a = rng.standard_normal((m, k)).astype(np.float32)
    want = nx.matmul_quant(fmt, a, w, m, n, k)
    da, dw = be.upload(a), be.upload(w)
    dout = be.alloc(m * n * 4)
    {nx.FMT_Q5_0: be.matmul_q5_0, nx.FMT_Q5_K: be.matmul_q5_k, nx.FMT_BF16: be.matmul_bf16}[fmt](da, dw, dout, m, n, k)
    got = be.download(dout, (m, n), np.float32)
    _close(got, want, 2e-5, 2e-6 * np.abs(want).max() + 1e-7, "matmul fmt %d m %d" % (fmt, m))
    # an activation that is not 16-byte aligned takes the element-wise path: same values to rounding
    if m == 3:
        big = be.alloc((m * k + 1) * 4)
        be.copy_buffer(da, 0, big, 4, m * k * 4)
        be.matmul_quant(fmt, big + 4, dw, dout, None, m, n, k)
        _close(be.download(dout, (m, n), np.float32), want, 2e-5, 2e-6 * np.abs(want).max() + 1e-7, "unaligned")
    be.reset_pool()


@pytest.mark.parametrize("m,n,k", [(2, 64, 256), (32, 256, 2048), (40, 512, 1024), (7, 1040, 512), (100, 96, 768),
                                   (1, 71, 4096), (1, 256, 11008), (1, 3, 8)])
def test_matmul_bf16_fast_paths(be, m, n, k):
    """MatMulBF16 (backend.go:80) where the matrix-core kernel (two rows and more, K a multiple of 256, N of 16:
    the bf16 weights become f16 exactly) and the streaming matrix-vector kernel (one row) take it; with and without
    the residual; weights down to f16's smallest normal magnitudes."""
    rng = np.random.default_rng(m * 7 + n + k)
    fmt = nx.FMT_BF16
    w = qz.random_quant(fmt, rng, n, k)
    a = rng.standard_normal((m, k)).astype(np.float32)
    res = rng.standard_normal((m, n)).astype(np.float32)
    want = nx.matmul_quant(fmt, a, w, m, n, k)
    da, dw, dres = be.upload(a), be.upload(w), be.upload(res)
    dout = be.alloc(m * n * 4)
    scale = np.abs(want).max()
    be.matmul_quant(fmt, da, dw, dout, None, m, n, k)
    _close(be.download(dout, (m, n), np.float32), want, 2e-5, 3e-6 * scale + 1e-7, "bf16 %dx%dx%d" % (m, n, k))
    be.matmul_quant(fmt, da, dw, dout, dres, m, n, k)
    _close(be.download(dout, (m, n), np.float32), want + res, 2e-5, 3e-6 * scale + 1e-6, "bf16 + residual")
    # small weights: 2^-14 .. 2^-10 (f16 keeps all eight bits of a bf16 there)
    wf = (rng.standard_normal(n * k) * 2.0 ** -12).astype(np.float32)
    ws = (wf.view(np.uint32) >> 16).astype(np.uint16)
    want2 = a.astype(np.float64) @ (ws.astype(np.uint32) << 16).view(np.float32).reshape(n, k).astype(np.float64).T
    be.matmul_quant(fmt, da, be.upload(ws), dout, None, m, n, k)
    got2 = be.download(dout, (m, n), np.float32)
    assert np.all(np.abs(got2 - want2) <= 2e-5 * np.abs(want2) + 3e-6 * np.abs(want2).max())
    be.reset_pool()


# ------------------------------------------------------------------ quantized matmul
@pytest.mark.parametrize("fmt", FMTS_MFMA)
@pytest.mark.parametrize("m", [1, 3, 8, 16, 17, 32, 40])
def test_matmul_quant_vs_oracle(be, fmt, m):
    rng = np.random.default_rng(fmt * 100 + m)
    n, k = 80, 1024
    w = qz.random_quant(fmt, rng, n, k)
    a = rng.standard_normal((m, k)).astype(np.float32)
    want = nx.matmul_quant(fmt, a, w, m, n, k)
    da, dw = be.upload(a), be.upload(w)
    dout = be.alloc(m * n * 4)
    name = {nx.FMT_Q4_0: be.matmul_q4_0, nx.FMT_Q8_0: be.matmul_q8_0, nx.FMT_Q4_K: be.matmul_q4_k,
            nx.FMT_Q6_K: be.matmul_q6_k, nx.FMT_Q5_0: be.matmul_q5_0, nx.FMT_Q5_K: be.matmul_q5_k}[fmt]
    name(da, dw, dout, m, n, k)
    got = be.download(dout, (m, n), np.float32)
    # float32 summation-order level: far inside the 1e-2 abs / 1e-3 rel logits budget
    scale = np.abs(want).max()
    _close(got, want, 2e-5, 2e-6 * scale + 1e-7, "matmul fmt %d m %d" % (fmt, m))
    be.reset_pool()


@pytest.mark.parametrize("fmt", FMTS_MFMA)
def test_matmul_rows_independent_of_batch(be, fmt):
    """A row has the same bits in a batch of 2 and of 32, in a batch of 40 and of 64, and in a batch of 72 and of
    90: the k-slices and the order their sums are added in depend on the matrix, the device and the kernel only, and
    the kernel (or its cut of the matrix) changes at 32 and at 64 rows (cf. the reference's loop of M=1 kernels,
    backend/metal/backend.go:777-779). Across those boundaries, and for a single row (M = 1, the matrix-vector
    kernel), rows agree to rounding, not bit for bit."""
    rng = np.random.default_rng(9)
    m, n, k = 32, 96, 2048
    w = qz.random_quant(fmt, rng, n, k)
    big = rng.standard_normal((90, k)).astype(np.float32)
    a = big[:m]
    da, dw = be.upload(big), be.upload(w)

    def batch(rows):
        d = be.alloc(rows * n * 4)
        be.matmul_quant(fmt, da, dw, d, None, rows, n, k)
        return be.download(d, (rows, n), np.float32)

    full, many = batch(m), batch(90)
    assert np.array_equal(many[:72].view(np.uint32), batch(72).view(np.uint32))
    mid = batch(64)
    assert np.array_equal(mid[:40].view(np.uint32), batch(40).view(np.uint32))
    want = nx.matmul_quant(fmt, big, w, 90, n, k)
    _close(many, want, 2e-5, 3e-6 * np.abs(want).max() + 1e-7, "90-row batch")
    _close(mid, want[:64], 2e-5, 3e-6 * np.abs(want).max() + 1e-7, "64-row batch")
    assert np.all(np.abs(many[:m] - full) <= 2e-6 * np.abs(full).max() + 1e-7)
    assert np.all(np.abs(mid[:m] - full) <= 2e-6 * np.abs(full).max() + 1e-7)
    for r in (0, 5, 30):
        d2 = be.alloc(2 * n * 4)
        be.matmul_quant(fmt, da + r * k * 4, dw, d2, None, 2, n, k)
        two = be.download(d2, (2, n), np.float32)
        assert np.array_equal(two.view(np.uint32), full[r:r + 2].view(np.uint32))
        d1 = be.alloc(n * 4)
        be.matmul_quant(fmt, da + r * k * 4, dw, d1, None, 1, n, k)
        one = be.download(d1, (n,), np.float32)
        assert np.all(np.abs(one - full[r]) <= 2e-6 * np.abs(full[r]).max() + 1e-7)
    be.reset_pool()


@pytest.mark.parametrize("fmt", FMTS_MFMA)
@pytest.mark.parametrize("n,k", [(80, 1024), (33, 256), (7, 4096), (96, 11008), (40, 14336)])
def test_matvec_single_row(be, fmt, n, k):
    """M = 1 (the reference's decode call): segments that start at odd 16-byte phases, rows that are not a
    multiple of 16 bytes (Q6_K at K = 11008), row groups running past N, with and without the residual. Shapes
    the matrix-vector kernel declines (a matrix that is not a multiple of 16 bytes long) fall to the other paths
    and must give the same answer."""
    rng = np.random.default_rng(fmt * 1000 + n + k)
    w = qz.random_quant(fmt, rng, n, k)
    a = rng.standard_normal((1, k)).astype(np.float32)
    res = rng.standard_normal((1, n)).astype(np.float32)
    want = nx.matmul_quant(fmt, a, w, 1, n, k)
    da, dw, dres = be.upload(a), be.upload(w), be.upload(res)
    dout = be.alloc(n * 4)
    scale = np.abs(want).max()
    be.matmul_quant(fmt, da, dw, dout, None, 1, n, k)
    _close(be.download(dout, (1, n), np.float32), want, 2e-5, 3e-6 * scale + 1e-7, "matvec fmt %d %dx%d" % (fmt, n, k))
    be.matmul_quant(fmt, da, dw, dout, dres, 1, n, k)
    _close(be.download(dout, (1, n), np.float32), want + res, 2e-5, 3e-6 * scale + 1e-6, "matvec + residual")
    be.reset_pool()


@pytest.mark.parametrize("fmt", [nx.FMT_Q4_0, nx.FMT_Q8_0, nx.FMT_Q4_K])
@pytest.mark.parametrize("m,n,k", [(33, 4112, 512), (48, 12304, 256), (64, 96, 4096), (50, 1040, 2048)])
def test_matmul_33_to_64_rows(be, fmt, m, n, k):
    """Batches of 33 to 64 rows (four activation tiles a step in the kernel whose waves split K): a matrix tall
    enough for several rounds of workgroups, heights that leave the last workgroup overlapping its neighbour, several
    K slices, rows of padding in the last tile; with and without the residual."""
    rng = np.random.default_rng(m + n + k + fmt)
    w = qz.random_quant(fmt, rng, n, k)
    a = rng.standard_normal((m, k)).astype(np.float32)
    res = rng.standard_normal((m, n)).astype(np.float32)
    want = nx.matmul_quant(fmt, a, w, m, n, k)
    da, dw, dres = be.upload(a), be.upload(w), be.upload(res)
    dout = be.alloc(m * n * 4)
    scale = np.abs(want).max()
    be.matmul_quant(fmt, da, dw, dout, None, m, n, k)
    _close(be.download(dout, (m, n), np.float32), want, 2e-5, 3e-6 * scale + 1e-7, "%dx%dx%d" % (m, n, k))
    be.matmul_quant(fmt, da, dw, dout, dres, m, n, k)
    _close(be.download(dout, (m, n), np.float32), want + res, 2e-5, 3e-6 * scale + 1e-6, "with the residual")
    be.reset_pool()


@pytest.mark.parametrize("fmt", [nx.FMT_Q4_0, nx.FMT_Q6_K])
def test_matmul_rows_independent_at_prefill_size(be, fmt):
    """1024 rows against a 2048-row matrix: enough (row group, activation group) pairs that one workgroup walks
    the k-slices in order instead of one workgroup per slice. Rows keep the bits they have in a batch of 70."""
    rng = np.random.default_rng(19)
    m, n, k = 1024, 2048, 512
    w = qz.random_quant(fmt, rng, n, k)
    a = rng.standard_normal((m, k)).astype(np.float32)
    da, dw = be.upload(a), be.upload(w)
    dout = be.alloc(m * n * 4)
    be.matmul_quant(fmt, da, dw, dout, None, m, n, k)
    full = be.download(dout, (m, n), np.float32)
    for r in (0, 517, 954):
        d2 = be.alloc(70 * n * 4)
        be.matmul_quant(fmt, da + r * k * 4, dw, d2, None, 70, n, k)
        assert np.array_equal(be.download(d2, (70, n), np.float32).view(np.uint32), full[r:r + 70].view(np.uint32))
    want = nx.matmul_quant(fmt, a[:64], w, 64, n, k)
    _close(full[:64], want, 2e-5, 3e-6 * np.abs(want).max() + 1e-7, "1024-row batch")
    be.reset_pool()


@pytest.mark.parametrize("m,n,k", [(100, 208, 512), (256, 1024, 2048), (130, 4096, 256), (97, 48, 1024)])
def test_matmul_many_rows_q8_0(be, m, n, k):
    """Q8_0 with more than 96 rows (prompt chunks): the kernel whose waves split the weight rows. Heights that
    leave waves and whole workgroups past the matrix' end, one and several K slices, a last group of activation
    rows that is partly padding; with and without the residual."""
    rng = np.random.default_rng(m + n + k)
    fmt = nx.FMT_Q8_0
    w = qz.random_quant(fmt, rng, n, k)
    a = rng.standard_normal((m, k)).astype(np.float32)
    res = rng.standard_normal((m, n)).astype(np.float32)
    want = nx.matmul_quant(fmt, a, w, m, n, k)
    da, dw, dres = be.upload(a), be.upload(w), be.upload(res)
    dout = be.alloc(m * n * 4)
    scale = np.abs(want).max()
    be.matmul_quant(fmt, da, dw, dout, None, m, n, k)
    got = be.download(dout, (m, n), np.float32)
    _close(got, want, 2e-5, 3e-6 * scale + 1e-7, "many rows %dx%dx%d" % (m, n, k))
    be.matmul_quant(fmt, da, dw, dout, dres, m, n, k)
    _close(be.download(dout, (m, n), np.float32), want + res, 2e-5, 3e-6 * scale + 1e-6, "many rows + residual")
    # (this kernel's K slices depend on how many groups of 64 rows the batch has: a row keeps its bits between
    # batches of the same number of groups, and agrees to rounding otherwise)
    m2 = min(m + 20, (m + 63) // 64 * 64)
    if m2 > m:
        a2 = np.concatenate([a, rng.standard_normal((m2 - m, k)).astype(np.float32)])
        d2 = be.alloc(m2 * n * 4)
        be.matmul_quant(fmt, be.upload(a2), dw, d2, None, m2, n, k)
        assert np.array_equal(be.download(d2, (m2, n), np.float32)[:m].view(np.uint32), got.view(np.uint32))
    be.reset_pool()


@pytest.mark.parametrize("fmt", FMTS_MFMA)
@pytest.mark.parametrize("m,n,k", [(5, 96, 11008), (32, 40, 14336), (16, 7, 4096), (33, 200, 256)])
def test_matmul_batched_shapes(be, fmt, m, n, k):
    """M >= 2 at the 7B / 8B reduction lengths: Q6_K rows of 9030 bytes (every even 16-byte phase), row groups
    running past N, one-chunk reductions, M just past a tile boundary; with and without the residual."""
    rng = np.random.default_rng(fmt * 77 + m + n)
    w = qz.random_quant(fmt, rng, n, k)
    a = rng.standard_normal((m, k)).astype(np.float32)
    res = rng.standard_normal((m, n)).astype(np.float32)
    want = nx.matmul_quant(fmt, a, w, m, n, k)
    da, dw, dres = be.upload(a), be.upload(w), be.upload(res)
    dout = be.alloc(m * n * 4)
    scale = np.abs(want).max()
    be.matmul_quant(fmt, da, dw, dout, None, m, n, k)
    _close(be.download(dout, (m, n), np.float32), want, 2e-5, 3e-6 * scale + 1e-7, "matmul fmt %d %dx%dx%d" % (fmt, m, n, k))
    be.matmul_quant(fmt, da, dw, dout, dres, m, n, k)
    _close(be.download(dout, (m, n), np.float32), want + res, 2e-5, 3e-6 * scale + 1e-6, "matmul + residual")
    be.reset_pool()


def test_prepared_activation_paths(be):
    """prepare-once / multiply-many equals the one-shot entry point bit for bit, and the fused
    RMSNorm / SiLU*up prepares equal the separate ops."""
    rng = np.random.default_rng(14)
    m, n, k = 32, 160, 2048
    a = (rng.standard_normal((m, k)) * 3).astype(np.float32)
    wn = rng.standard_normal(k).astype(np.float32)
    ws = {f: qz.random_quant(f, rng, n, k) for f in (nx.FMT_Q4_0, nx.FMT_Q8_0, nx.FMT_Q4_K)}
    da, dwn = be.upload(a), be.upload(wn)
    dws = {f: be.upload(w) for f, w in ws.items()}
    d1, d2, dnorm = be.alloc(m * n * 4), be.alloc(m * n * 4), be.alloc(m * k * 4)
    # plain prepare, three formats from one prepared activation
    be.prepare_act(da, m, k)
    for f in ws:
        be.matmul_quant_prepared(f, dws[f], d1, None, m, n, k)
        one = be.download(d1, (m, n), np.float32)
        be.matmul_quant(f, da, dws[f], d2, None, m, n, k)
        be.prepare_act(da, m, k)      # the one-shot call re-filled the slot; prepare again for the next format
        assert np.array_equal(one.view(np.uint32), be.download(d2, (m, n), np.float32).view(np.uint32))
    # fused rmsnorm + prepare
    be.rmsnorm_prepare(da, dwn, dnorm, m, k, 1e-5)
    want_norm = nx.rmsnorm(a, wn, m, k, 1e-5)
    got_norm = be.download(dnorm, (m, k), np.float32)
    _close(got_norm, want_norm, 2e-6, 1e-7, "rmsnorm_prepare f32 output")
    be.matmul_quant_prepared(nx.FMT_Q4_0, dws[nx.FMT_Q4_0], d1, None, m, n, k)
    got = be.download(d1, (m, n), np.float32)
    want = nx.matmul_q4_0(want_norm, ws[nx.FMT_Q4_0], m, n, k)
    _close(got, want, 3e-5, 3e-6 * np.abs(want).max(), "rmsnorm_prepare + matmul")
    be.rmsnorm_prepare(da, dwn, None, m, k, 1e-5)     # no f32 copy: same prepared values
    be.matmul_quant_prepared(nx.FMT_Q4_0, dws[nx.FMT_Q4_0], d2, None, m, n, k)
    assert np.array_equal(got.view(np.uint32), be.download(d2, (m, n), np.float32).view(np.uint32))
    # fused silu*up + prepare (staged and recomputing variants)
    for kk in (2048, 14336):
        g = (rng.standard_normal((3, kk)) * 2).astype(np.float32)
        u = rng.standard_normal((3, kk)).astype(np.float32)
        w2 = qz.random_quant(nx.FMT_Q4_0, rng, 48, kk)
        dg, du, dw2 = be.upload(g), be.upload(u), be.upload(w2)
        dact, do = be.alloc(3 * kk * 4), be.alloc(3 * 48 * 4)
        be.silu_mul_prepare(dg, du, dact, 3, kk)
        act = nx.silu_mul(g, u)
        _close(be.download(dact, (3, kk), np.float32), act, 1e-6, 1e-9, "silu_mul_prepare f32 output")
        be.matmul_quant_prepared(nx.FMT_Q4_0, dw2, do, None, 3, 48, kk)
        want = nx.matmul_q4_0(act, w2, 3, 48, kk)
        _close(be.download(do, (3, 48), np.float32), want, 3e-5, 3e-6 * np.abs(want).max(), "silu_mul_prepare + matmul")
        # the GeGLU form of the same launch: the bits of the separate GELU * up kernel
        be.gelu_mul_prepare(dg, du, dact, 3, kk)
        act = nx.gelu_mul(g, u)
        got_act = be.download(dact, (3, kk), np.float32)
        _close(got_act, act, 1e-6, 1e-9, "gelu_mul_prepare f32 output")
        dsep = be.alloc(3 * kk * 4)
        be.gelu_mul(dg, du, dsep, 3 * kk)
        assert np.array_equal(got_act.view(np.uint32), be.download(dsep, (3, kk), np.float32).view(np.uint32))
        be.matmul_quant_prepared(nx.FMT_Q4_0, dw2, do, None, 3, 48, kk)
        want = nx.matmul_q4_0(act, w2, 3, 48, kk)
        _close(be.download(do, (3, 48), np.float32), want, 3e-5, 3e-6 * np.abs(want).max(), "gelu_mul_prepare + matmul")
        # GELU alone (the GELU MLP's fc1 output as fc2's operand): the bits of vx_gelu
        be.gelu_prepare(dg, dact, 3, kk)
        got_act = be.download(dact, (3, kk), np.float32)
        be.gelu(dg, dsep, 3 * kk)
        assert np.array_equal(got_act.view(np.uint32), be.download(dsep, (3, kk), np.float32).view(np.uint32))
        _close(got_act, nx.gelu(g), 1e-6, 1e-9, "gelu_prepare f32 output")
        be.matmul_quant_prepared(nx.FMT_Q4_0, dw2, do, None, 3, 48, kk)
        want = nx.matmul_q4_0(nx.gelu(g), w2, 3, 48, kk)
        _close(be.download(do, (3, 48), np.float32), want, 3e-5, 3e-6 * np.abs(want).max(), "gelu_prepare + matmul")
    # shape mismatch is an error, not a wrong answer
    from vexel_amd.backend import VexelError
    with pytest.raises(VexelError):
        be.matmul_quant_prepared(nx.FMT_Q4_0, dws[nx.FMT_Q4_0], d1, None, m, n, 4096)
    be.reset_pool()


@pytest.mark.parametrize("fmt,rows,hidden,ffn", [(nx.FMT_Q4_0, 1, 512, 1024), (nx.FMT_Q4_0, 32, 512, 14336),
                                                 (nx.FMT_Q8_0, 5, 512, 1024), (nx.FMT_Q4_K, 40, 1024, 2048),
                                                 (nx.FMT_Q6_K, 32, 512, 2816), (nx.FMT_Q6_K, 3, 1024, 1024),
                                                 (nx.FMT_Q8_0, 1, 512, 1024), (nx.FMT_Q4_K, 1, 1024, 2048),
                                                 (nx.FMT_Q6_K, 1, 1024, 2816), (nx.FMT_Q4_0, 1, 4096, 11008),
                                                 (nx.FMT_Q4_0, 100, 512, 1024), (nx.FMT_Q6_K, 256, 512, 1024),
                                                 (nx.FMT_Q8_0, 300, 512, 2816), (nx.FMT_Q4_0, 512, 1024, 1024)])
def test_fused_decode_blocks_equal_the_unfused_sequence(be, fmt, rows, hidden, ffn):
    """vx_decode_attn_qkv / vx_decode_ffn give what the one-call-per-operation sequence of
    runtime/block.go:834-1077 gives (float32 activations, F16 and F32 pools; one row goes through the
    matrix-vector kernel with RMSNorm, SiLU*up and the residual adds folded in), including the chained
    prepared activation for the next block. A fused projection group is one launch over the summed
    width, so its split-K slices differ from the separate launches': values agree to float32 summation
    order (1e-5 of the row magnitude), not bit for bit; a chained call equals a fresh one exactly."""
    rng = np.random.default_rng(77 + rows)
    hq, hk, d, bs, eps, theta = hidden // 64, 2, 64, 16, 1e-5, 10000.0
    nblocks = max(24, (rows + bs - 1) // bs + 8)      # (a slot for every row)
    assert nblocks * bs >= rows
    kvd = hk * d
    W = {name: qz.random_quant(fmt, rng, n, k) for name, (n, k) in
         dict(wq=(hidden, hidden), wk=(kvd, hidden), wv=(kvd, hidden), wo=(hidden, hidden), w1=(ffn, hidden),
              w3=(ffn, hidden), w2=(hidden, ffn)).items()}
    dims = dict(wq=(hidden, hidden), wk=(kvd, hidden), wv=(kvd, hidden), wo=(hidden, hidden), w1=(ffn, hidden),
                w3=(ffn, hidden), w2=(hidden, ffn))
    dW = {n: be.upload(w) for n, w in W.items()}
    qw = {n: be.qweight(fmt, dW[n], *dims[n]) for n in W}
    assert be.decode_attn_qkv_supported(qw["wq"], qw["wk"], qw["wv"], d)
    assert be.decode_ffn_supported(qw["wo"], qw["w1"], qw["w3"], qw["w2"])
    x = (rng.standard_normal((rows, hidden)) * 2).astype(np.float32)
    n1, n2, n3 = (rng.standard_normal(hidden).astype(np.float32) for _ in range(3))
    pos = rng.integers(0, 3000, rows).astype(np.int32)
    slots = rng.permutation(nblocks * bs)[:rows].astype(np.int32)
    dn1, dn2, dn3, dpos, dslots = (be.upload(a) for a in (n1, n2, n3, pos, slots))
    f4 = lambda *shape: be.alloc(int(np.prod(shape)) * 4)
    bits = lambda a: a.view(np.uint32) if a.dtype == np.float32 else a.view(np.uint16)

    def near(got, want, what):
        if got.dtype == np.uint16:   # F16 pool: the float32 values differ in the last bits, so allow the f16 neighbour
            g, w = nx.f16_to_f32_array(got), nx.f16_to_f32_array(want)
            assert np.all(np.abs(g - w) <= np.abs(w) * 2.0 ** -10 + 1e-4), what
            assert np.mean(got != want) < 2e-2, what
        else:
            assert np.all(np.abs(got - want) <= 2e-5 * np.abs(want).max() + 1e-6), \
                "%s: %g" % (what, np.abs(got - want).max())
    for f16 in (True, False):
        pool = _make_pool(rng, f16, nblocks, bs, hk, d)
        # ---- unfused
        dx, dpool = be.upload(x), be.upload(pool)
        dq, dk, dv, dg, du = f4(rows, hidden), f4(rows, kvd), f4(rows, kvd), f4(rows, ffn), f4(rows, ffn)
        be.rmsnorm_prepare(dx, dn1, None, rows, hidden, eps)
        for name, out in (("wq", dq), ("wk", dk), ("wv", dv)):
            be.matmul_quant_prepared(fmt, dW[name], out, None, rows, dims[name][0], hidden)
        be.rope_store_paged(dq, dk, dv, dpos, dslots, dpool, f16, rows, hq, hk, d, bs, theta)
        q_ref = be.download(dq, (rows, hidden), np.float32)
        pool_ref = be.download(dpool, pool.shape, pool.dtype)
        attn = (rng.standard_normal((rows, hidden))).astype(np.float32)   # stands in for the attention output
        dattn = be.upload(attn)
        be.matmul_quant(fmt, dattn, dW["wo"], dx, dx, rows, hidden, hidden)
        be.rmsnorm_prepare(dx, dn2, None, rows, hidden, eps)
        be.matmul_quant_prepared(fmt, dW["w1"], dg, None, rows, ffn, hidden)
        be.matmul_quant_prepared(fmt, dW["w3"], du, None, rows, ffn, hidden)
        be.silu_mul_prepare(dg, du, None, rows, ffn)
        be.matmul_quant_prepared(fmt, dW["w2"], dx, dx, rows, hidden, ffn)
        x_ref = be.download(dx, (rows, hidden), np.float32)
        be.rmsnorm_prepare(dx, dn3, None, rows, hidden, eps)
        be.matmul_quant_prepared(fmt, dW["wk"], dk, None, rows, kvd, hidden)
        next_ref = be.download(dk, (rows, kvd), np.float32)
        # ---- fused, without and with the chained prepare
        for chain in (False, True):
            dx2, dpool2, dq2 = be.upload(x), be.upload(pool), f4(rows, hidden)
            be.decode_attn_qkv(dx2, dn1, eps, False, qw["wq"], qw["wk"], qw["wv"], rows, dpos, dslots, dpool2, f16,
                               hq, hk, d, bs, theta, dq2)
            near(be.download(dq2, (rows, hidden), np.float32), q_ref, "q")
            near(be.download(dpool2, pool.shape, pool.dtype), pool_ref, "pool")
            be.decode_ffn(dattn, dx2, qw["wo"], dn2, eps, qw["w1"], qw["w3"], qw["w2"], rows, dn3 if chain else None)
            near(be.download(dx2, (rows, hidden), np.float32), x_ref, "x after the block")
            if chain:
                be.matmul_quant_prepared(fmt, dW["wk"], dk, None, rows, kvd, hidden)
                near(be.download(dk, (rows, kvd), np.float32), next_ref, "projection of the chained activation")
                # and the next block's attention half accepts the chained activation
                be.decode_ffn(dattn, dx2, qw["wo"], dn2, eps, qw["w1"], qw["w3"], qw["w2"], rows, dn1)
                dx3 = be.upload(be.download(dx2, (rows, hidden), np.float32))
                dq3, dq4, dpool3, dpool4 = f4(rows, hidden), f4(rows, hidden), be.upload(pool), be.upload(pool)
                be.decode_attn_qkv(0, 0, eps, True, qw["wq"], qw["wk"], qw["wv"], rows, dpos, dslots, dpool3, f16,
                                   hq, hk, d, bs, theta, dq3)
                be.decode_attn_qkv(dx3, dn1, eps, False, qw["wq"], qw["wk"], qw["wv"], rows, dpos, dslots, dpool4, f16,
                                   hq, hk, d, bs, theta, dq4)
                # (the chained activation is prepared per 256-column chunk with 1/rms applied to the products,
                # the fresh one per row with x/rms prepared: same values up to float32 rounding)
                near(be.download(dq3, (rows, hidden), np.float32), be.download(dq4, (rows, hidden), np.float32),
                     "q from the chained activation")
                near(be.download(dpool3, pool.shape, pool.dtype), be.download(dpool4, pool.shape, pool.dtype),
                     "pool from the chained activation")
            else:
                from vexel_amd.backend import VexelError
                with pytest.raises(VexelError):   # nothing was left prepared
                    be.decode_attn_qkv(0, 0, eps, True, qw["wq"], qw["wk"], qw["wv"], rows, dpos, dslots, dpool2, f16,
                                       hq, hk, d, bs, theta, dq2)
        # ---- with the step's table of RoPE angles the projection launch finishes its own rows where it can (one
        # K slice, up to 32 rows; a single row: the matrix-vector kernel's epilogue): same Q and pool
        if rows <= 64:
            dx5, dpool5, dq5 = be.upload(x), be.upload(pool), f4(rows, hidden)
            be.rope_table_prepare(dpos, rows, d, theta)   # (after the uploads: writes to device memory drop the table)
            be.decode_attn_qkv(dx5, dn1, eps, False, qw["wq"], qw["wk"], qw["wv"], rows, dpos, dslots, dpool5, f16,
                               hq, hk, d, bs, theta, dq5)
            near(be.download(dq5, (rows, hidden), np.float32), q_ref, "q with the angle table")
            near(be.download(dpool5, pool.shape, pool.dtype), pool_ref, "pool with the angle table")
    # mixed formats inside a group are refused, not mis-computed
    other = be.qweight(nx.FMT_Q8_0 if fmt != nx.FMT_Q8_0 else nx.FMT_Q4_0, dW["wk"], kvd, hidden)
    assert not be.decode_attn_qkv_supported(qw["wq"], other, qw["wv"], d)
    be.reset_pool()


@pytest.mark.parametrize("rows", [1, 5, 32, 40])
@pytest.mark.parametrize("fqk,fv", [(nx.FMT_Q4_K, nx.FMT_Q6_K), (nx.FMT_Q4_0, nx.FMT_Q8_0)])
def test_decode_attn_qkv_with_v_in_another_format(be, rows, fqk, fv):
    """The Q4_K_M mixes keep attn_v in Q6_K beside Q4_K attn_q / attn_k: the fused attention half takes V as a launch
    of its own between the shared prepare and the shared RoPE + store, and gives what the one-call-per-operation
    sequence gives (runtime/block.go:834-905)."""
    rng = np.random.default_rng(300 + rows)
    hidden, hq, hk, d, bs, nblocks, eps, theta = 1024, 16, 4, 64, 16, 24, 1e-5, 10000.0
    kvd = hk * d
    dims = dict(wq=(hidden, hidden), wk=(kvd, hidden), wv=(kvd, hidden))
    fm = dict(wq=fqk, wk=fqk, wv=fv)
    dW = {n: be.upload(qz.random_quant(fm[n], rng, *dims[n])) for n in dims}
    qw = {n: be.qweight(fm[n], dW[n], *dims[n]) for n in dims}
    assert be.decode_attn_qkv_supported(qw["wq"], qw["wk"], qw["wv"], d)
    x = (rng.standard_normal((rows, hidden)) * 2).astype(np.float32)
    n1 = rng.standard_normal(hidden).astype(np.float32)
    pos = rng.integers(0, 3000, rows).astype(np.int32)
    slots = rng.permutation(nblocks * bs)[:rows].astype(np.int32)
    pool = _make_pool(rng, True, nblocks, bs, hk, d)
    dn1, dpos, dslots = be.upload(n1), be.upload(pos), be.upload(slots)
    f4 = lambda *shape: be.alloc(int(np.prod(shape)) * 4)
    dx, dpool = be.upload(x), be.upload(pool)
    dq, dk, dv = f4(rows, hidden), f4(rows, kvd), f4(rows, kvd)
    be.rmsnorm_prepare(dx, dn1, None, rows, hidden, eps)
    for name, out in (("wq", dq), ("wk", dk), ("wv", dv)):
        be.matmul_quant_prepared(fm[name], dW[name], out, None, rows, dims[name][0], hidden)
    be.rope_store_paged(dq, dk, dv, dpos, dslots, dpool, True, rows, hq, hk, d, bs, theta)
    q_ref = be.download(dq, (rows, hidden), np.float32)
    pool_ref = nx.f16_to_f32_array(be.download(dpool, pool.shape, pool.dtype))
    dx2, dpool2, dq2 = be.upload(x), be.upload(pool), f4(rows, hidden)
    be.decode_attn_qkv(dx2, dn1, eps, False, qw["wq"], qw["wk"], qw["wv"], rows, dpos, dslots, dpool2, True,
                       hq, hk, d, bs, theta, dq2)
    q = be.download(dq2, (rows, hidden), np.float32)
    assert np.all(np.abs(q - q_ref) <= 2e-5 * np.abs(q_ref).max() + 1e-6)
    got = nx.f16_to_f32_array(be.download(dpool2, pool.shape, pool.dtype))
    assert np.all(np.abs(got - pool_ref) <= np.abs(pool_ref) * 2.0 ** -10 + 1e-4)
    be.reset_pool()


# (query heads, kv heads, head size): a workgroup's columns are one 256-column chunk, a quarter or half of one,
# four of them, one and a half (two KV heads make three chunks: merged in the kernel), three and a half and five
# sixteenths (7 chunks per two KV heads, 5 per sixteen heads of 80: more than a workgroup merges at once, the
# prepare kernel does it)
@pytest.mark.parametrize("hq,hk,d", [(8, 2, 64), (8, 8, 64), (4, 4, 128), (8, 1, 128), (6, 2, 128), (28, 4, 128),
                                     (16, 16, 80)])
def test_decode_ffn_merges_split_attention(be, hq, hk, d):
    """vx_sdpa_paged_decode_ragged(out = NULL) + vx_decode_ffn(attn = NULL) equals the merged attention output
    fed to vx_decode_ffn (the split-KV partials are merged by the same formula, by the attention kernel's last
    workgroup of each chunk or by the prepare kernel)."""
    rng = np.random.default_rng(91)
    fmt, rows, hidden, ffn = nx.FMT_Q4_0, 5, 512, 1024
    bs, nblocks, eps = 16, 160, 1e-5
    dims = dict(wo=(hidden, hq * d), w1=(ffn, hidden), w3=(ffn, hidden), w2=(hidden, ffn))
    dW = {n: be.upload(qz.random_quant(fmt, rng, *dims[n])) for n in dims}
    qw = {n: be.qweight(fmt, dW[n], *dims[n]) for n in dims}
    assert be.lib_call("vx_sdpa_paged_decode_split_supported", 1, bs, hq, hk, d) == 1
    lens = np.array([1, 16, 700, 513, 37], dtype=np.int32)          # several splits, block boundaries
    max_blocks = 48
    perm = rng.permutation(nblocks).astype(np.int32)
    tables = np.zeros((rows, max_blocks), dtype=np.int32)
    off = 0
    for i, L in enumerate(lens):
        nb = (L + bs - 1) // bs
        tables[i, :nb] = perm[off:off + nb]
        off += nb
    pool = _make_pool(rng, True, nblocks, bs, hk, d)
    q = rng.standard_normal((rows, hq * d)).astype(np.float32)
    x = rng.standard_normal((rows, hidden)).astype(np.float32)
    nw = rng.standard_normal(hidden).astype(np.float32)
    dpool, dq, dt, dl, dnw = be.upload(pool), be.upload(q), be.upload(tables), be.upload(lens), be.upload(nw)
    scale = 1.0 / math.sqrt(d)
    dattn = be.alloc(rows * hq * d * 4)
    # twice, the second time with other lengths (fewer splits, one sequence without tokens: zeros): whatever the
    # first call counted is gone
    for lens_i in (lens, np.array([300, 0, 512, 40, 31], dtype=np.int32)):
        dl = be.upload(lens_i)
        be.sdpa_paged_decode_ragged(dq, dpool, True, dt, dl, dattn, rows, max_blocks, bs, hq, hk, d, scale, max_blocks * bs)
        dx1 = be.upload(x)
        be.decode_ffn(dattn, dx1, qw["wo"], dnw, eps, qw["w1"], qw["w3"], qw["w2"], rows, None)
        want_i = be.download(dx1, (rows, hidden), np.float32)
        dx2 = be.upload(x)
        be.sdpa_paged_decode_ragged(dq, dpool, True, dt, dl, None, rows, max_blocks, bs, hq, hk, d, scale, max_blocks * bs)
        be.decode_ffn(None, dx2, qw["wo"], dnw, eps, qw["w1"], qw["w3"], qw["w2"], rows, None)
        got = be.download(dx2, (rows, hidden), np.float32)
        assert np.all(np.abs(got - want_i) <= 1e-5 * np.abs(want_i).max())
        if lens_i is lens:
            want = want_i
    # one row (the matrix-vector path merges the partials while it reads its activation): sequence 2, 700 tokens
    one = slice(2, 3)
    dq1, dt1, dl1 = be.upload(q[one]), be.upload(tables[one]), be.upload(lens[one])
    dx3 = be.upload(x[one])
    be.sdpa_paged_decode_ragged(dq1, dpool, True, dt1, dl1, None, 1, max_blocks, bs, hq, hk, d, scale, max_blocks * bs)
    be.decode_ffn(None, dx3, qw["wo"], dnw, eps, qw["w1"], qw["w3"], qw["w2"], 1, None)
    got1 = be.download(dx3, (1, hidden), np.float32)
    assert np.all(np.abs(got1 - want[one]) <= 2e-5 * np.abs(want).max())
    from vexel_amd.backend import VexelError
    with pytest.raises(VexelError):      # the pending split result was consumed
        be.decode_ffn(None, dx2, qw["wo"], dnw, eps, qw["w1"], qw["w3"], qw["w2"], rows, None)
    dpool32 = be.upload(_make_pool(rng, False, nblocks, bs, hk, d))
    with pytest.raises(VexelError):      # no split form for an F32 pool
        be.sdpa_paged_decode_ragged(dq, dpool32, False, dt, dl, None, rows, max_blocks, bs, hq, hk, d, scale, max_blocks * bs)
    be.reset_pool()


def test_matmul_quant_residual_and_shapes(be):
    rng = np.random.default_rng(11)
    for (m, n, k) in [(2, 33, 512), (32, 4096, 4096), (5, 100, 11008)]:
        w = qz.random_quant(nx.FMT_Q4_0, rng, n, k)
        a = rng.standard_normal((m, k)).astype(np.float32)
        res = rng.standard_normal((m, n)).astype(np.float32)
        want = nx.add(res, nx.matmul_q4_0(a, w, m, n, k))
        da, dw, dr = be.upload(a), be.upload(w), be.upload(res)
        be.matmul_quant(nx.FMT_Q4_0, da, dw, dr, dr, m, n, k)   # in place on the residual
        got = be.download(dr, (m, n), np.float32)
        _close(got, want, 2e-5, 1e-5, "residual %s" % ((m, n, k),))
        be.reset_pool()


def test_matmul_quant_unaligned_k_uses_fallback(be):
    rng = np.random.default_rng(12)
    m, n, k = 3, 20, 96   # K not a multiple of 256
    w = qz.random_quant(nx.FMT_Q4_0, rng, n, k)
    a = rng.standard_normal((m, k)).astype(np.float32)
    da, dw = be.upload(a), be.upload(w)
    dout = be.alloc(m * n * 4)
    be.matmul_q4_0(da, dw, dout, m, n, k)
    _close(be.download(dout, (m, n), np.float32), nx.matmul_q4_0(a, w, m, n, k), 1e-5, 1e-6, "fallback")
    be.reset_pool()


def test_unknown_format_and_bad_shape_report(be):
    from vexel_amd.backend import VexelError
    d = be.alloc(4096)
    with pytest.raises(VexelError) as e:
        be.matmul_quant(9, d, d, d, None, 1, 4, 32)          # no such format
    assert e.value.code == 4
    with pytest.raises(VexelError) as e:
        be.matmul_q5_k(d, d, d, 1, 4, 128)                   # K is not a whole number of 256-element blocks
    assert e.value.code == 1
    with pytest.raises(VexelError) as e:
        be.matmul_q5_0(0, 0, 0, 1, 32, 32)
    assert e.value.code == 1
    be.reset_pool()


def test_matmul_f32(be):
    rng = np.random.default_rng(13)
    m, n, k = 7, 45, 100
    a = rng.standard_normal((m, k)).astype(np.float32)
    b = rng.standard_normal((n, k)).astype(np.float32)
    da, db = be.upload(a), be.upload(b)
    do = be.alloc(m * n * 4)
    be.matmul_transposed(da, db, do, m, n, k)
    _close(be.download(do, (m, n), np.float32), nx.matmul_t_f32(a, b, m, n, k), 1e-5, 1e-5, "matmul_t")
    dbt = be.upload(np.ascontiguousarray(b.T))
    be.matmul(da, dbt, do, m, n, k)
    _close(be.download(do, (m, n), np.float32), nx.matmul_f32(a, b.T.copy(), m, n, k), 1e-5, 1e-5, "matmul")
    be.reset_pool()


# ------------------------------------------------------------------ elementwise
def test_rmsnorm_rope_silu_add_softmax_embedding_argmax(be):
    rng = np.random.default_rng(20)
    rows, cols = 5, 2048
    x = (rng.standard_normal((rows, cols)) * 2).astype(np.float32)
    w = rng.standard_normal(cols).astype(np.float32)
    dx, dw = be.upload(x), be.upload(w)
    do = be.alloc(x.nbytes)
    be.rmsnorm(dx, dw, do, rows, cols, 1e-5)
    _close(be.download(do, x.shape, np.float32), nx.rmsnorm(x, w, rows, cols, 1e-5), 2e-6, 1e-7, "rmsnorm")

    hq, hk, d, s = 8, 2, 64, 6
    q = rng.standard_normal((s, hq, d)).astype(np.float32)
    k = rng.standard_normal((s, hk, d)).astype(np.float32)
    for neox, rd in ((False, 0), (True, 0), (False, 32)):
        dq, dk = be.upload(q), be.upload(k)
        be.rope(dq, dk, d, hq, hk, s, 1234, rd, 10000.0, neox)
        wq, wk = nx.rope(q, k, d, hq, hk, s, 1234, rd, 10000.0, neox)
        _close(be.download(dq, q.shape, np.float32), wq.reshape(q.shape), 0, 1e-6, "rope q")
        _close(be.download(dk, k.shape, np.float32), wk.reshape(k.shape), 0, 1e-6, "rope k")
    dq = be.upload(q)
    be.rope(dq, 0, d, hq, 0, s, 0, 0, 500000.0, False)   # k = nil is allowed (cpu.go:269)
    wq, _ = nx.rope(q, None, d, hq, 0, s, 0, 0, 500000.0, False)
    _close(be.download(dq, q.shape, np.float32), wq.reshape(q.shape), 0, 1e-6, "rope q only")

    n = 11008 * 3
    g = (rng.standard_normal(n) * 3).astype(np.float32)
    u = rng.standard_normal(n).astype(np.float32)
    dg, du = be.upload(g), be.upload(u)
    dn = be.alloc(n * 4)
    be.silu_mul(dg, du, dn, n)
    _close(be.download(dn, (n,), np.float32), nx.silu_mul(g, u), 1e-6, 1e-9, "silu_mul")
    be.silu(dg, dn, n)
    _close(be.download(dn, (n,), np.float32), nx.silu(g), 1e-6, 1e-9, "silu")
    be.add(dg, du, dn, n)
    assert np.array_equal(be.download(dn, (n,), np.float32), nx.add(g, u))
    be.mul(dg, du, dn, n)
    assert np.array_equal(be.download(dn, (n,), np.float32), nx.mul(g, u))

    sm = (rng.standard_normal((4, 333)) * 5).astype(np.float32)
    ds = be.upload(sm)
    dso = be.alloc(sm.nbytes)
    be.softmax(ds, dso, 4, 333)
    _close(be.download(dso, sm.shape, np.float32), nx.softmax(sm, 4, 333), 2e-6, 1e-9, "softmax")

    table = rng.standard_normal((50, 64)).astype(np.float32)
    ids = np.array([3, 49, -1, 50, 0], dtype=np.int32)
    dt, di = be.upload(table), be.upload(ids)
    init = np.full((5, 64), 7.0, dtype=np.float32)
    de = be.upload(init)
    be.embedding(di, 5, dt, de, 50, 64)
    assert np.array_equal(be.download(de, (5, 64), np.float32), nx.embedding(ids, table, 50, 64, out=init.copy()))

    lg = rng.standard_normal((6, 32000)).astype(np.float32)
    lg[1, 777] = lg[1, 20000] = 50.0          # tie -> lowest index
    lg[2, :] = -np.inf                         # all -inf -> 0
    lg[3, 5] = np.nan; lg[3, 9] = 60.0         # NaN never wins
    lg[4, 31999] = 99.0
    dl = be.upload(lg)
    di = be.alloc(6 * 4)
    be.argmax_rows(dl, 6, 32000, di)
    got = be.download(di, (6,), np.int32)
    assert list(got) == [nx.argmax(lg[r]) for r in range(6)]
    assert be.argmax(dl + 4 * 32000 * 4, 32000) == 31999
    # ties between the columns one thread scans (4 t .. 4 t + 3, then 4096 further on), and rows that the vector
    # scan does not take (a width that is no multiple of four: every second row also starts off a 16-byte boundary)
    lg2 = rng.standard_normal((4, 8200)).astype(np.float32)
    lg2[0, 9] = lg2[0, 4105] = lg2[0, 8] = 40.0
    lg2[1, 4106] = lg2[1, 11] = 40.0
    lg2[2, 8199] = lg2[2, 4103] = 40.0
    lg2[3, 8196] = 40.0
    d2, di2 = be.upload(lg2), be.alloc(4 * 4)
    be.argmax_rows(d2, 4, 8200, di2)
    assert list(be.download(di2, (4,), np.int32)) == [8, 11, 4103, 8196]
    lg3 = rng.standard_normal((3, 333)).astype(np.float32)
    lg3[1, 332] = lg3[1, 7] = 30.0
    d3, di3 = be.upload(lg3), be.alloc(3 * 4)
    be.argmax_rows(d3, 3, 333, di3)
    assert list(be.download(di3, (3,), np.int32)) == [nx.argmax(lg3[r]) for r in range(3)]
    be.reset_pool()


# ------------------------------------------------------------------ attention
def test_sdpa_and_prefill(be):
    rng = np.random.default_rng(30)
    for (hq, hk, d, L, stride) in [(1, 1, 4, 1, 1), (8, 2, 64, 300, 512), (4, 4, 128, 1500, 1500), (2, 1, 2, 3, 3)]:
        q = rng.standard_normal((hq, d)).astype(np.float32)
        k = rng.standard_normal((hk, stride, d)).astype(np.float32)
        v = rng.standard_normal((hk, stride, d)).astype(np.float32)
        sc = np.float32(1 / math.sqrt(d))
        dq, dk, dv = be.upload(q), be.upload(k), be.upload(v)
        do = be.alloc(q.nbytes)
        be.sdpa(dq, dk, dv, do, L, hq, hk, d, sc, stride * d)
        _close(be.download(do, q.shape, np.float32), nx.sdpa(q, k, v, L, hq, hk, d, sc, stride * d), 1e-5, 2e-6, "sdpa")
        be.reset_pool()
    # causal prefill: the tiled matrix-core kernel (head_dim 64 / 128; one query, ragged tile ends, exact tile
    # multiples, GQA) and the generic kernel (other head sizes)
    for (s, hq, hk, d) in [(70, 4, 2, 64), (1, 2, 2, 128), (33, 4, 1, 128), (64, 2, 2, 64), (129, 8, 2, 128),
                           (200, 2, 1, 64), (40, 2, 2, 32)]:
        q = rng.standard_normal((s, hq, d)).astype(np.float32)
        k = rng.standard_normal((s, hk, d)).astype(np.float32)
        v = rng.standard_normal((s, hk, d)).astype(np.float32)
        sc = np.float32(1 / math.sqrt(d))
        dq, dk, dv = be.upload(q), be.upload(k), be.upload(v)
        do = be.alloc(q.nbytes)
        be.sdpa_prefill(dq, dk, dv, do, s, hq, hk, d, sc)
        _close(be.download(do, q.shape, np.float32), nx.sdpa_prefill(q, k, v, s, hq, hk, d, sc), 1e-5, 3e-6,
               "prefill s=%d hq=%d hk=%d d=%d" % (s, hq, hk, d))
        be.reset_pool()


def _make_pool(rng, f16, nblocks, bs, hk, d):
    elems = nblocks * 2 * bs * hk * d
    vals = rng.standard_normal(elems).astype(np.float32)
    return nx.f32_to_f16_array(vals) if f16 else vals


@pytest.mark.parametrize("f16", [False, True])
def test_reshape_paged_kv_exact_layout(be, f16):
    """inference/backend/metal/paged_test.go:10-128: exact equality of the scattered layout."""
    rng = np.random.default_rng(31)
    bs, hk, d, nblocks, t = 16, 4, 64, 12, 21
    src = (rng.standard_normal((t, hk, d)) * 3).astype(np.float32)
    bi = rng.integers(0, nblocks, t).astype(np.int32)
    bo = rng.integers(0, bs, t).astype(np.int32)
    # distinct (block, offset) pairs so the result does not depend on write order
    pairs = set()
    for i in range(t):
        while (int(bi[i]), int(bo[i])) in pairs:
            bo[i] = (bo[i] + 1) % bs
            if bo[i] == 0:
                bi[i] = (bi[i] + 1) % nblocks
        pairs.add((int(bi[i]), int(bo[i])))
    pool = _make_pool(rng, f16, nblocks, bs, hk, d)
    want = pool.copy()
    dpool, dsrc, dbi, dbo = be.upload(pool), be.upload(src), be.upload(bi), be.upload(bo)
    fn = be.reshape_paged_kv_f16 if f16 else be.reshape_paged_kv
    for isv in (False, True):
        fn(dsrc, dpool, dbi, dbo, t, hk, d, bs, isv)
        nx.reshape_paged_kv(src, want, bi, bo, hk, d, bs, isv)
    got = be.download(dpool, pool.shape, pool.dtype)
    assert np.array_equal(got, want)
    be.reset_pool()


@pytest.mark.parametrize("f16", [False, True])
@pytest.mark.parametrize("shape", [(32, 4, 64), (32, 32, 128), (8, 8, 128), (4, 2, 32), (28, 4, 128), (24, 8, 128),
                                   (12, 2, 64), (10, 2, 128), (14, 2, 64), (8, 4, 256), (4, 4, 256), (32, 32, 80), (6, 6, 96),
                                   (32, 2, 128), (24, 2, 128)])
def test_paged_decode_single_batched_ragged(be, f16, shape):
    hq, hk, d = shape
    rng = np.random.default_rng(32 + hq + d)
    bs, nblocks = 16, 200
    pool = _make_pool(rng, f16, nblocks, bs, hk, d)
    dpool = be.upload(pool)
    sc = np.float32(1 / math.sqrt(d))
    lens = [1, 15, 16, 17, 513, 700, 1024, 37]
    perm = rng.permutation(nblocks)
    tables, off = [], 0
    for L in lens:
        nb = (L + bs - 1) // bs
        tables.append(perm[off:off + nb].astype(np.int32)); off += nb
    B = len(lens)
    q = rng.standard_normal((B, hq, d)).astype(np.float32)
    dq = be.upload(q)
    want = np.stack([nx.sdpa_paged_decode(q[i], pool, tables[i], len(tables[i]), bs, hq, hk, d, sc,
                                          lens[i] - (len(tables[i]) - 1) * bs) for i in range(B)])
    # single-sequence entry points
    single = be.sdpa_paged_decode_f16 if f16 else be.sdpa_paged_decode
    for i in (0, 3, 5):
        dbt = be.upload(tables[i])
        do = be.alloc(hq * d * 4)
        single(dq + i * hq * d * 4, dpool, dbt, do, len(tables[i]), bs, hq, hk, d, sc,
               lens[i] - (len(tables[i]) - 1) * bs)
        _close(be.download(do, (hq, d), np.float32), want[i], 1e-5, 3e-6, "paged single %d" % i)
    # Go-style batched (host arrays of device pointers)
    ptrs = [be.upload(t) for t in tables]
    mb = max(len(t) for t in tables)
    do = be.alloc(q.nbytes)
    be.sdpa_paged_decode_batched(dq, dpool, ptrs, do, B, mb, bs, hq, hk, d, sc, lens, pool_is_f16=f16)
    _close(be.download(do, q.shape, np.float32), want, 1e-5, 3e-6, "paged batched")
    # ragged (device matrix + device lengths)
    mat = np.full((B, mb), -1, dtype=np.int32)
    for i, t in enumerate(tables):
        mat[i, :len(t)] = t
    mat[mat < 0] = 0
    dmat, dl = be.upload(mat), be.upload(np.array(lens, dtype=np.int32))
    do2 = be.alloc(q.nbytes)
    be.sdpa_paged_decode_ragged(dq, dpool, f16, dmat, dl, do2, B, mb, bs, hq, hk, d, sc, max(lens))
    _close(be.download(do2, q.shape, np.float32), want, 1e-5, 3e-6, "paged ragged")
    be.reset_pool()


@pytest.mark.parametrize("hq,hk,d", [(8, 2, 128), (16, 2, 64), (6, 2, 128)])
def test_paged_decode_grouped_queries_value_ranges(be, hq, hk, d):
    """The grouped-query kernel scales every query row by a power of two before it splits it into two f16 halves and
    carries the softmax weights times 2^10: rows of very large and very small magnitude, a zero row, a row with one
    dominant element, scores peaked on one token with a long tail of small weights, contexts that end inside a
    block and on a split boundary."""
    rng = np.random.default_rng(77 + hq + d)
    bs, nblocks = 16, 200
    pool = _make_pool(rng, True, nblocks, bs, hk, d)
    dpool = be.upload(pool)
    sc = np.float32(1 / math.sqrt(d))
    lens = [700, 37, 513, 16, 1024, 256, 300]
    B, mb = len(lens), 64
    perm = rng.permutation(nblocks)
    mat = np.zeros((B, mb), dtype=np.int32)
    tables, off = [], 0
    for i, L in enumerate(lens):
        nb = (L + bs - 1) // bs
        mat[i, :nb] = perm[off:off + nb]
        tables.append(mat[i, :nb].copy()); off += nb
    q = rng.standard_normal((B, hq, d)).astype(np.float32)
    q[0] *= 1e3
    q[1] *= 1e-6
    q[2, 1] = 0.0
    q[3, :, 5] = 4000.0
    q[4] *= 30.0                       # peaked: one token takes nearly all the weight, a thousand share the rest
    q[5, 0] *= 1e-20
    q[6, ::2] *= 200.0
    want = np.stack([nx.sdpa_paged_decode(q[i], pool, tables[i], len(tables[i]), bs, hq, hk, d, sc,
                                          lens[i] - (len(tables[i]) - 1) * bs) for i in range(B)])
    dq, dmat, dl = be.upload(q), be.upload(mat), be.upload(np.array(lens, dtype=np.int32))
    do = be.alloc(q.nbytes)
    be.sdpa_paged_decode_ragged(dq, dpool, True, dmat, dl, do, B, mb, bs, hq, hk, d, sc, mb * bs)
    got = be.download(do, q.shape, np.float32)
    assert np.isfinite(got).all()
    # A query row enters with 22 significant bits relative to its largest element, so a score s carries an error of
    # about 2^-22 |s| (float32 dot products: 2^-24 |s| and their own rounding); where the scores reach into the
    # hundreds that shows in the weights, and the bar widens with the largest score of the sequence.
    errs = []
    for i in range(B):
        smax = float(np.abs(q[i]).max() * 6.0 * math.sqrt(d) * sc * math.sqrt(2.0)) if lens[i] > 16 else 0.0
        tol = 3e-6 + 2.0 ** -21 * min(smax, 64.0)
        e = np.abs(got[i].astype(np.float64) - want[i]) - 1e-5 * np.abs(want[i])
        errs.append((i, float(e.max()), tol))
    assert all(e <= t for _, e, t in errs), errs
    be.reset_pool()


def test_attention_work_list_from_pack_batch(be):
    """vx_pack_batch leaves a work list for the ragged decode attention (full 512-token items first, partial last
    items from the longest down). The attention call that passes the packed kv_lens array and row indices takes the list; a call
    with a copy of the same lengths in another array walks the (split, sequence) grid. Both give the same bits,
    and match the oracle; writing the lengths through the library drops the list."""
    rng = np.random.default_rng(36)
    bs, hq, hk, d, nblocks = 16, 8, 2, 128, 400
    pool = _make_pool(rng, True, nblocks, bs, hk, d)
    dpool = be.upload(pool)
    sc = np.float32(1 / math.sqrt(d))
    pos = np.array([0, 511, 512, 700, 1023, 1536, 40, 1100, 255], dtype=np.int32)   # kv_len = pos + 1
    B, mb = pos.size, 100
    perm = rng.permutation(nblocks)
    tables = np.zeros((B, mb), dtype=np.int32)
    nblk = np.zeros(B, dtype=np.int32)
    off = 0
    for i, p_ in enumerate(pos):
        nb = (int(p_) + 1 + bs - 1) // bs          # blocks already there, the new token's included
        tables[i, :nb] = perm[off:off + nb]; nblk[i] = nb; off += nb
    free = perm[off:].astype(np.int32)
    d_t, d_n, d_f, d_c = be.upload(tables), be.upload(nblk), be.upload(free), be.upload(np.array([free.size], np.int32))
    d_s, d_p = be.upload(np.arange(B, dtype=np.int32)), be.upload(pos)
    cu, tp, sm, kl, st = be.alloc((B + 1) * 4), be.alloc(B * 4), be.alloc(B * 4), be.alloc(B * 4), be.alloc(4)
    be.pack_batch(d_s, d_p, 0, B, B, d_t, mb, d_n, d_f, d_c, bs, cu, tp, sm, kl, st)
    assert be.download(st, (1,), np.int32)[0] == 0
    lens = be.download(kl, (B,), np.int32)
    assert list(lens) == [int(p_) + 1 for p_ in pos]
    q = rng.standard_normal((B, hq, d)).astype(np.float32)
    dq = be.upload(q)
    want = np.stack([nx.sdpa_paged_decode(q[i], pool, tables[i, :nblk[i]], int(nblk[i]), bs, hq, hk, d, sc,
                                          int(lens[i]) - (int(nblk[i]) - 1) * bs) for i in range(B)])
    o_list, o_grid, o_after = be.alloc(q.nbytes), be.alloc(q.nbytes), be.alloc(q.nbytes)
    be.sdpa_paged_decode_ragged(dq, dpool, True, d_t, kl, o_list, B, mb, bs, hq, hk, d, sc, mb * bs, table_rows=d_s)
    kl2 = be.alloc(B * 4)
    be.copy_buffer(kl, 0, kl2, 0, B * 4)
    be.sdpa_paged_decode_ragged(dq, dpool, True, d_t, kl2, o_grid, B, mb, bs, hq, hk, d, sc, mb * bs)
    got = be.download(o_list, q.shape, np.float32)
    assert np.array_equal(got.view(np.uint32), be.download(o_grid, q.shape, np.float32).view(np.uint32))
    _close(got, want, 1e-5, 3e-6, "attention over the packed work list")
    # shorter lengths written into the packed array: the stale list must not be used
    short = np.maximum(lens // 2, 1).astype(np.int32)
    be.to_device(kl, short)
    be.sdpa_paged_decode_ragged(dq, dpool, True, d_t, kl, o_after, B, mb, bs, hq, hk, d, sc, mb * bs, table_rows=d_s)
    want2 = np.stack([nx.sdpa_paged_decode(q[i], pool, tables[i, :nblk[i]], (int(short[i]) + bs - 1) // bs, bs, hq, hk, d, sc,
                                           int(short[i]) - ((int(short[i]) + bs - 1) // bs - 1) * bs) for i in range(B)])
    _close(be.download(o_after, q.shape, np.float32), want2, 1e-5, 3e-6, "attention after the lengths were rewritten")
    be.reset_pool()


def test_paged_multiquery_and_tree(be):
    rng = np.random.default_rng(34)
    bs, hq, hk, d, nblocks = 16, 8, 2, 64, 40
    for f16 in (False, True):
        pool = _make_pool(rng, f16, nblocks, bs, hk, d)
        dpool = be.upload(pool)
        bt = rng.permutation(nblocks)[:20].astype(np.int32)
        dbt = be.upload(bt)
        sc = np.float32(1 / math.sqrt(d))
        qn = 6
        q = rng.standard_normal((qn, hq, d)).astype(np.float32)
        dq = be.upload(q)
        kvl = np.array([100 + i + 1 for i in range(qn)], dtype=np.int32)   # block.go:884-887
        dk = be.upload(kvl)
        do = be.alloc(q.nbytes)
        be.sdpa_paged_decode_multiquery(dq, dpool, dbt, do, dk, len(bt), bs, hq, hk, d, sc, qn, pool_is_f16=f16)
        want = nx.sdpa_paged_multiquery(q, pool, bt, kvl, bs, hq, hk, d, sc)
        _close(be.download(do, q.shape, np.float32), want, 1e-5, 3e-6, "multiquery")
        parent = [-1, -1, 0, 0, 1, 1]
        mask = np.array(hl.build_tree_attention_mask(6, parent), dtype=np.uint8)
        dm = be.upload(mask)
        be.sdpa_paged_tree(dq, dpool, f16, dbt, do, dm, 200, bs, hq, hk, d, sc, qn)
        want = nx.sdpa_paged_multiquery(q, pool, bt, None, bs, hq, hk, d, sc, tree_mask=mask, tree_base=200)
        _close(be.download(do, q.shape, np.float32), want, 1e-5, 3e-6, "tree")
        be.reset_pool()


@pytest.mark.parametrize("hq,hk,d,qn,start,bs", [(8, 2, 128, 200, 137, 16), (8, 8, 64, 70, 0, 16), (4, 1, 128, 16, 500, 16),
                                                 (32, 8, 128, 65, 40, 16), (28, 4, 128, 50, 77, 16), (4, 4, 128, 100, 300, 16),
                                                 (8, 2, 128, 200, 137, 32), (8, 8, 64, 70, 0, 8)])
def test_paged_multiquery_tiled(be, hq, hk, d, qn, start, bs):
    """SDPAPagedDecodeMultiquery on the matrix-core kernels (F16 pool, 16 or more query rows): the later chunk of a
    prompt (row i sees start + i + 1 keys, runtime/block.go:884-887), with the chunk's rows crossing tile boundaries,
    against the oracle's per-row attention. 16-token blocks: the kernel that walks the blocks per wave; other block
    sizes: the one that stages 32-key tiles in LDS."""
    rng = np.random.default_rng(340 + qn)
    nblocks = 960 // bs
    pool = _make_pool(rng, True, nblocks, bs, hk, d)
    dpool = be.upload(pool)
    bt = rng.permutation(nblocks)[:(start + qn + bs - 1) // bs + 1].astype(np.int32)
    sc = np.float32(1 / math.sqrt(d))
    q = rng.standard_normal((qn, hq, d)).astype(np.float32)
    kvl = np.array([start + i + 1 for i in range(qn)], dtype=np.int32)
    dq, dbt, dk, do = be.upload(q), be.upload(bt), be.upload(kvl), be.alloc(q.nbytes)
    be.sdpa_paged_decode_multiquery(dq, dpool, dbt, do, dk, len(bt), bs, hq, hk, d, sc, qn, pool_is_f16=True)
    want = nx.sdpa_paged_multiquery(q, pool, bt, kvl, bs, hq, hk, d, sc)
    _close(be.download(do, q.shape, np.float32), want, 1e-5, 3e-6, "tiled multiquery, causal chunk")
    # lengths in no order, some rows seeing a single key, one row none at all (its output is zero)
    kvl2 = rng.integers(1, start + qn + 1, qn).astype(np.int32)
    kvl2[3], kvl2[qn - 1] = 1, start + qn
    be.to_device(dk, kvl2)
    be.sdpa_paged_decode_multiquery(dq, dpool, dbt, do, dk, len(bt), bs, hq, hk, d, sc, qn, pool_is_f16=True)
    want = nx.sdpa_paged_multiquery(q, pool, bt, kvl2, bs, hq, hk, d, sc)
    _close(be.download(do, q.shape, np.float32), want, 1e-5, 3e-6, "tiled multiquery, ragged lengths")
    kvl2[5] = 0
    be.to_device(dk, kvl2)
    be.sdpa_paged_decode_multiquery(dq, dpool, dbt, do, dk, len(bt), bs, hq, hk, d, sc, qn, pool_is_f16=True)
    got = be.download(do, q.shape, np.float32)
    assert not got[5].any()
    keep = [i for i in range(qn) if i != 5]
    _close(got[keep], want[keep], 1e-5, 3e-6, "tiled multiquery, one empty row")
    be.reset_pool()


@pytest.mark.parametrize("hq,hk,d,half", [(8, 8, 128, False), (8, 8, 128, True), (8, 2, 64, False), (8, 2, 64, True),
                                          (16, 2, 128, False), (16, 2, 128, True), (6, 2, 128, False), (10, 2, 64, False),
                                          (14, 2, 128, True)])
def test_paged_tree_batched(be, hq, hk, d, half):
    """Every tree of a batch in two launches: against the oracle's masked multi-query attention per sequence and,
    to rounding, the per-sequence entry point. Ragged contexts (one empty, one a multiple of the 512-token split),
    trees of different sizes, entries padded with repeated rows; entries of 16 / G rows and, where that is even, of
    half as many."""
    rng = np.random.default_rng(37)
    bs, nblocks = 16, 160
    rg = be._lib.vx_sdpa_paged_tree_rows_per_entry(1, bs, hq, hk, d)
    assert rg == 16 // (hq // hk)
    if half:
        assert rg % 2 == 0
        rg //= 2
    pool = _make_pool(rng, True, nblocks, bs, hk, d)
    dpool = be.upload(pool)
    starts = [0, 37, 512, 700]
    parents = [[-1, -1, 0, 0, 1, 1, 2, 2, 3, 3, 4, 4, 5, 5, 6], [-1, 0, 1], [-1, -1, -1, 0, 1, 2, 3, 3, 3, 8], [-1]]
    mb = (max(starts) + 16 + bs - 1) // bs + 1
    perm = rng.permutation(nblocks)
    tables = np.zeros((len(starts), mb), dtype=np.int32)
    off = 0
    for i, st in enumerate(starts):
        nb = (st + len(parents[i]) + bs - 1) // bs
        tables[i, :nb] = perm[off:off + nb]
        off += nb
    sc = np.float32(1 / math.sqrt(d))
    qs, masks, info, moff, ent_rows, ent_lens, row0 = [], [], [], [], [], [], []
    mask_bytes = 0
    for i, par in enumerate(parents):
        n = len(par)
        pad = (n + rg - 1) // rg * rg
        q = rng.standard_normal((n, hq, d)).astype(np.float32)
        mask = np.array(hl.build_tree_attention_mask(n, par), dtype=np.uint8)
        row0.append(sum(x.shape[0] for x in qs))
        qs.append(np.concatenate([q, np.repeat(q[-1:], pad - n, axis=0)]))
        for r in range(pad):
            info.append([i, starts[i], min(r, n - 1), n])
            moff.append(mask_bytes)
        masks.append(mask)
        mask_bytes += mask.size
        ent_rows += [i] * (pad // rg)
        ent_lens += [starts[i]] * (pad // rg)
    qall = np.concatenate(qs)
    rows = qall.shape[0]
    dq, dt = be.upload(qall), be.upload(tables)
    dm = be.upload(np.concatenate(masks))
    do = be.alloc(qall.nbytes)
    be.call("vx_sdpa_paged_tree_batched", dq, dpool, dt, mb, be.upload(np.array(ent_rows, dtype=np.int32)),
            be.upload(np.array(ent_lens, dtype=np.int32)), len(ent_rows), be.upload(np.array(info, dtype=np.int32)), dm,
            be.upload(np.array(moff, dtype=np.int32)), do, rows, max(len(p) for p in parents), hq, hk, d, sc, max(starts))
    got = be.download(do, qall.shape, np.float32)
    for i, par in enumerate(parents):
        n = len(par)
        want = nx.sdpa_paged_multiquery(qs[i][:n], pool, tables[i], None, bs, hq, hk, d, sc, tree_mask=masks[i],
                                        tree_base=starts[i])
        _close(got[row0[i]:row0[i] + n], want, 1e-5, 3e-6, "batched tree, sequence %d" % i)
        one = be.alloc(n * hq * d * 4)
        be.sdpa_paged_tree(dq + row0[i] * hq * d * 4, dpool, True, dt + i * mb * 4, one, be.upload(masks[i]), starts[i], bs,
                           hq, hk, d, sc, n)
        _close(got[row0[i]:row0[i] + n], be.download(one, (n, hq, d), np.float32), 1e-5, 3e-6, "against the per-sequence call")
    be.reset_pool()


def test_sample_rows_matches_the_reference_sampler(be):
    """Sampler.Sample (pkg/sampler/sampler.go:48-204) on the device against its restatement with the same uniform
    draws: greedy rows, plain temperature sampling, top-k, top-p and both, flat and peaked distributions, draws at
    both ends of [0, 1), equal probabilities at the cut-offs, a vocabulary that is not a power of two."""
    rng = np.random.default_rng(38)
    n = 3001
    cases = []
    for temp, k, p in [(0.0, 0, 0.0), (1.0, 0, 0.0), (0.7, 40, 0.0), (0.7, 0, 0.9), (1.3, 50, 0.95), (0.5, 1, 0.0),
                       (1.0, n, 1.0), (1.0, 5, 0.5), (2.0, 0, 0.999), (0.1, 0, 0.3), (1.0, 300, 0.2)]:
        for r in (float(rng.random()), 0.0, 0.99999994):
            cases.append((temp, k, p, r))
    rows = len(cases)
    logits = (rng.standard_normal((rows, n)) * rng.choice([0.2, 1.0, 4.0], size=(rows, 1))).astype(np.float32)
    logits[3, 100:140] = logits[3, 100]                     # runs of equal logits: ties at the top-k / top-p cuts
    logits[9, :] = 0.25
    logits[12, 7] = logits[12, 2000] = logits[12].max() + 1
    logits[20, 500:2500] = logits[20, 499]
    temp = np.array([c[0] for c in cases], dtype=np.float32)
    topk = np.array([c[1] for c in cases], dtype=np.int32)
    topp = np.array([c[2] for c in cases], dtype=np.float32)
    uni = np.array([c[3] for c in cases], dtype=np.float32)
    out = be.alloc(rows * 4)
    be.sample_rows(be.upload(logits), rows, n, be.upload(temp), be.upload(topk), be.upload(topp), be.upload(uni), out)
    got = be.download(out, (rows,), np.int32)
    want = [hl.sampler_sample(logits[i], float(temp[i]), int(topk[i]), float(topp[i]), float(uni[i])) for i in range(rows)]
    assert got.tolist() == want
    assert len(set(want)) > rows // 3                        # the cases do pick different tokens
    # tiny and odd vocabularies, one row and many
    for n2, rows2 in ((1, 1), (5, 3), (257, 40), (4096, 2)):
        lg = rng.standard_normal((rows2, n2)).astype(np.float32)
        t2 = rng.choice([0.0, 0.6, 1.0], rows2).astype(np.float32)
        k2 = rng.integers(0, n2 + 2, rows2).astype(np.int32)
        p2 = rng.choice([0.0, 0.5, 0.9, 1.0], rows2).astype(np.float32)
        u2 = rng.random(rows2).astype(np.float32)
        o2 = be.alloc(rows2 * 4)
        be.sample_rows(be.upload(lg), rows2, n2, be.upload(t2), be.upload(k2), be.upload(p2), be.upload(u2), o2)
        w2 = [hl.sampler_sample(lg[i], float(t2[i]), int(k2[i]), float(p2[i]), float(u2[i])) for i in range(rows2)]
        assert be.download(o2, (rows2,), np.int32).tolist() == w2, (n2, rows2)
    be.reset_pool()


def test_paged_kv_move_chains(be):
    """Rows move inside the pool in chain order: a later move of a chain reads what an earlier one wrote."""
    rng = np.random.default_rng(36)
    bs, hk, d, nblocks = 16, 2, 64, 12
    for f16 in (False, True):
        pool = _make_pool(rng, f16, nblocks, bs, hk, d)
        dpool = be.upload(pool)
        # chain 0: the accepted path of a tree (rows 3, 8, 9 move up to 1, 2, 3: row 3 is read, then overwritten);
        # chain 1: a move across blocks; chain 2: a swap-like pair that depends on the order
        base0, base1 = 5 * bs + 2, 7 * bs + 14
        chains = [[(base0 + 3, base0 + 1), (base0 + 8, base0 + 2), (base0 + 9, base0 + 3)],
                  [(base1 + 5, base1 + 1)],
                  [(20, 21), (21, 22)]]
        off = np.cumsum([0] + [len(c) for c in chains]).astype(np.int32)
        src = np.array([m[0] for c in chains for m in c], dtype=np.int32)
        dst = np.array([m[1] for c in chains for m in c], dtype=np.int32)
        be.paged_kv_move(dpool, f16, be.upload(off), be.upload(src), be.upload(dst), len(chains), hk, d, bs)
        want = pool.copy()
        row = hk * d
        for c in chains:
            for sl, dl in c:
                for half in (0, 1):
                    so = (sl // bs) * 2 * bs * row + half * bs * row + (sl % bs) * row
                    do = (dl // bs) * 2 * bs * row + half * bs * row + (dl % bs) * row
                    want[do:do + row] = want[so:so + row].copy()
        got = be.download(dpool, pool.shape, pool.dtype)
        assert np.array_equal(got.view(np.uint16 if f16 else np.uint32), want.view(np.uint16 if f16 else np.uint32))
        be.reset_pool()


def test_rope_shift(be):
    """RoPEShift (backend/cpu/backend.go:244-276) against the oracle (to the last bits of the float64 cos / sin, as
    for RoPE itself); shift 0 leaves the buffer alone."""
    rng = np.random.default_rng(39)
    hd, hk, toks = 128, 4, 37
    k = rng.standard_normal(toks * hk * hd).astype(np.float32)
    dk = be.upload(k)
    be.rope_shift(dk, hd, hk, toks, 0, 10000.0)
    assert np.array_equal(be.download(dk, k.shape, np.float32), k)
    for shift, theta in ((3, 10000.0), (4095, 500000.0)):
        dk = be.upload(k)
        be.rope_shift(dk, hd, hk, toks, shift, theta)
        want = nx.rope_shift(k, hd, hk, toks, shift, theta)
        _close(be.download(dk, k.shape, np.float32), want, 0, 1e-6, "rope shift %d" % shift)
    be.reset_pool()


@pytest.mark.parametrize("rope_dim,neox,d", [(0, False, 64), (0, True, 64), (32, True, 80), (32, False, 64), (128, True, 128)])
def test_rope_store_paged(be, rope_dim, neox, d):
    """Interleaved whole-head RoPE (LLaMA) and the ropeDim / ropeNeox forms of Backend.RoPE (Phi-2: 32 of 80
    dimensions, split pairs; Qwen / Gemma: the whole head, split pairs), fused with the paged store."""
    rng = np.random.default_rng(35)
    rows, hq, hk, bs, nblocks = 9, 8, 2, 16, 30
    q = rng.standard_normal((rows, hq, d)).astype(np.float32)
    k = rng.standard_normal((rows, hk, d)).astype(np.float32)
    v = rng.standard_normal((rows, hk, d)).astype(np.float32)
    pos = rng.integers(0, 4000, rows).astype(np.int32)
    slots = rng.permutation(nblocks * bs)[:rows].astype(np.int32)
    for f16 in (False, True):
        pool = _make_pool(rng, f16, nblocks, bs, hk, d)
        want_pool = pool.copy()
        wq, wk = nx.rope_positions(q, k, d, hq, hk, pos, rope_dim, 10000.0, neox)
        nx.reshape_paged_kv(wk, want_pool, slots // bs, slots % bs, hk, d, bs, False)
        nx.reshape_paged_kv(v, want_pool, slots // bs, slots % bs, hk, d, bs, True)
        dq, dk, dv = be.upload(q), be.upload(k), be.upload(v)
        dpool, dp, ds = be.upload(pool), be.upload(pos), be.upload(slots)
        be.rope_store_paged(dq, dk, dv, dp, ds, dpool, f16, rows, hq, hk, d, bs, 10000.0, rope_dim, neox)
        _close(be.download(dq, q.shape, np.float32), wq.reshape(q.shape), 0, 1e-6, "rope_store q")
        got = be.download(dpool, pool.shape, pool.dtype)
        if f16:
            # K is rotated in float32 then rounded: allow the f16 neighbour where the f32 values differ in the last bit
            diff = np.abs(nx.f16_to_f32_array(got) - nx.f16_to_f32_array(want_pool))
            tol = np.abs(nx.f16_to_f32_array(want_pool)) * 2.0 ** -10 + 1e-7
            assert np.all(diff <= tol)
            assert np.mean(got != want_pool) < 1e-3
        else:
            _close(got, want_pool, 0, 1e-6, "rope_store pool")
        be.reset_pool()


# ------------------------------------------------------------------ packing: bit exact
def test_pack_batch_bit_exact(be):
    rng = np.random.default_rng(40)
    bs, max_blocks, nslots, pool_blocks = 16, 20, 12, 150
    for trial in range(6):
        ref = hl.GPUBlockPool(1, 1, 8, bs, pool_blocks)
        tables = np.zeros((nslots, max_blocks), dtype=np.int32)
        nblk = np.zeros(nslots, dtype=np.int32)
        ctx = rng.integers(0, 200, nslots)
        for s in range(nslots):
            ref.create_sequence(s)
            if ctx[s] > 0:
                ref.store_kv_slots(0, s, 0, int(ctx[s]))
            bt = ref.seqs[s].block_tables[0]
            tables[s, :len(bt)] = bt; nblk[s] = len(bt)
        free = np.zeros(pool_blocks, dtype=np.int32)
        fl = ref.free_lists[0]
        free[:len(fl)] = fl
        free_count0 = len(fl)
        batch_slots = rng.permutation(nslots)[:rng.integers(1, nslots + 1)].astype(np.int32)
        qlens = (rng.integers(1, 40, batch_slots.size) if trial % 2 else np.ones(batch_slots.size)).astype(np.int32)
        pos = np.array([ctx[s] for s in batch_slots], dtype=np.int32)
        T = int(qlens.sum())
        want = hl.pack_batch(ref, 0, [int(s) for s in batch_slots], [int(p) for p in pos], [int(x) for x in qlens])
        d = {k: be.upload(v) for k, v in dict(slots=batch_slots, pos=pos, ql=qlens, tables=tables, nblk=nblk,
                                              free=free, fc=np.array([free_count0], dtype=np.int32)).items()}
        B = batch_slots.size
        cu, tp, sm, kl, st = (be.alloc((B + 1) * 4), be.alloc(T * 4), be.alloc(T * 4), be.alloc(B * 4), be.alloc(4))
        be.pack_batch(d["slots"], d["pos"], d["ql"] if trial % 2 else 0, B, T, d["tables"], max_blocks, d["nblk"],
                      d["free"], d["fc"], bs, cu, tp, sm, kl, st)
        assert be.download(st, (1,), np.int32)[0] == 0
        assert list(be.download(cu, (B + 1,), np.int32)) == want["cu_seqlens"]
        assert list(be.download(tp, (T,), np.int32)) == want["token_pos"]
        assert list(be.download(sm, (T,), np.int32)) == want["slot_mapping"]
        assert list(be.download(kl, (B,), np.int32)) == want["kv_lens"]
        got_tables = be.download(d["tables"], tables.shape, np.int32)
        got_nblk = be.download(d["nblk"], nblk.shape, np.int32)
        for s in range(nslots):
            bt = ref.seqs[s].block_tables[0]
            assert got_nblk[s] == len(bt) and list(got_tables[s, :len(bt)]) == bt
        assert be.download(d["fc"], (1,), np.int32)[0] == len(ref.free_lists[0])
        be.reset_pool()
    # exhaustion: status 1 and nothing changed
    tables = np.zeros((1, 4), dtype=np.int32); nblk = np.zeros(1, dtype=np.int32)
    free = np.arange(2, dtype=np.int32)
    d_t, d_n, d_f, d_c = be.upload(tables), be.upload(nblk), be.upload(free), be.upload(np.array([2], dtype=np.int32))
    d_s, d_p, d_q = be.upload(np.zeros(1, np.int32)), be.upload(np.zeros(1, np.int32)), be.upload(np.array([48], np.int32))
    cu, tp, sm, kl, st = be.alloc(8), be.alloc(48 * 4), be.alloc(48 * 4), be.alloc(4), be.alloc(4)
    be.pack_batch(d_s, d_p, d_q, 1, 48, d_t, 4, d_n, d_f, d_c, 16, cu, tp, sm, kl, st)
    assert be.download(st, (1,), np.int32)[0] == 1
    assert be.download(d_c, (1,), np.int32)[0] == 2 and be.download(d_n, (1,), np.int32)[0] == 0
    be.reset_pool()


def test_pool_alloc_reset_and_copy(be):
    a = be.alloc(1000); b = be.alloc(1000)
    assert a and b and a != b and a % 256 == 0
    be.reset_pool()
    assert be.alloc(1000) == a            # recycled after ResetPool
    p = be.alloc_permanent(4096)
    be.reset_pool()
    x = np.arange(1024, dtype=np.float32)
    be.to_device(p, x)
    q = be.alloc_permanent(4096)
    be.copy_buffer(p, 1024, q, 2048, 1024)
    got = be.download(q + 2048, (256,), np.float32)
    assert np.array_equal(got, x[256:512])
    be.free(p); be.free(q)
    be.begin_batch(); be.memory_barrier(); be.end_batch()


def test_graph_capture_replays_match_eager(be):
    rng = np.random.default_rng(50)
    m, n, k = 4, 256, 1024
    w = qz.random_quant(nx.FMT_Q4_0, rng, n, k)
    dw = be.upload(w, permanent=True)
    da = be.alloc_permanent(m * k * 4); do = be.alloc_permanent(m * n * 4); dn = be.alloc_permanent(m * n * 4)
    nw = be.upload(np.ones(n, dtype=np.float32), permanent=True)
    a = rng.standard_normal((m, k)).astype(np.float32)
    be.to_device(da, a)
    be.matmul_q4_0(da, dw, do, m, n, k)           # warm-up sizes the scratch
    be.graph_begin_capture()
    be.matmul_q4_0(da, dw, do, m, n, k)
    be.rmsnorm(do, nw, dn, m, n, 1e-5)
    g = be.graph_end_capture()
    for it in range(4):
        a = rng.standard_normal((m, k)).astype(np.float32)
        be.to_device(da, a)
        be.graph_launch(g)
        got = be.download(dn, (m, n), np.float32)
        be.matmul_q4_0(da, dw, do, m, n, k)
        be.rmsnorm(do, nw, dn, m, n, 1e-5)
        eager = be.download(dn, (m, n), np.float32)
        assert np.array_equal(got, eager)
    be.graph_destroy(g)
    for p in (dw, da, do, dn, nw):
        be.free(p)


# ------------------------------------------------------------------ optional interfaces of other architectures
def test_layernorm_gelu_bias_scale(be):
    """LayerNormOps, GELUOps, BiasOps, ScaleOps (backend.go:205-263) against the oracle's restatement of the CPU
    backend. The element-wise ones follow the reference's float32 operation order and are compared bit for bit."""
    rng = np.random.default_rng(61)
    for rows, cols in ((5, 2560), (3, 80), (1, 1)):
        x = (rng.standard_normal((rows, cols)) * 2 + 0.5).astype(np.float32)
        w = rng.standard_normal(cols).astype(np.float32)
        b = rng.standard_normal(cols).astype(np.float32)
        dx, dw, db = be.upload(x), be.upload(w), be.upload(b)
        do = be.alloc(x.nbytes)
        be.layernorm(dx, dw, db, do, rows, cols, 1e-5)
        _close(be.download(do, x.shape, np.float32), nx.layernorm(x, w, b, rows, cols, 1e-5), 1e-5, 2e-6, "layernorm")
        be.add_bias(dx, db, do, rows, cols)
        assert np.array_equal(be.download(do, x.shape, np.float32), nx.add_bias(x, b, rows, cols))
        be.add_bias(dx, db, dx, rows, cols)                          # in place
        assert np.array_equal(be.download(dx, x.shape, np.float32), nx.add_bias(x, b, rows, cols))
    n = 100003
    g = np.concatenate([(rng.standard_normal(n - 6) * 3), [0.0, -0.0, 40.0, -40.0, 1e-20, 9.5]]).astype(np.float32)
    u = rng.standard_normal(n).astype(np.float32)
    dg, du = be.upload(g), be.upload(u)
    do = be.alloc(n * 4)
    be.gelu(dg, do, n)
    got, want = be.download(do, (n,), np.float32), nx.gelu(g)
    _close(got, want, 2e-7, 1e-9, "gelu")
    assert np.mean(got.view(np.uint32) == want.view(np.uint32)) > 0.999
    be.gelu_mul(dg, du, do, n)
    _close(be.download(do, (n,), np.float32), nx.gelu_mul(g, u), 2e-7, 1e-9, "gelu_mul")
    be.scale_buffer(du, float(np.float32(math.sqrt(2304.0))), n)
    assert np.array_equal(be.download(du, (n,), np.float32), nx.scale_buffer(u, np.float32(math.sqrt(2304.0))))
    be.gelu(dg, do, 0)                                              # nothing to do
    # ApplyFinalLogitSoftCap (model.go:336-350): float64 tanh, bit for bit but for the device's tanh
    lg = np.concatenate([rng.standard_normal(n - 4) * 40, [0.0, 1e30, -1e30, 1e-8]]).astype(np.float32)
    dl = be.upload(lg)
    be.logit_softcap(dl, n, 30.0)
    got, want = be.download(dl, (n,), np.float32), nx.logit_softcap(lg, 30.0)
    _close(got, want, 2e-7, 1e-9, "logit_softcap")
    assert np.mean(got.view(np.uint32) == want.view(np.uint32)) > 0.999
    be.logit_softcap(dl, n, 0.0)                                    # disabled: unchanged
    assert np.array_equal(be.download(dl, (n,), np.float32), got)
    be.reset_pool()


@pytest.mark.parametrize("hq,hk,d,n,cap", [(8, 4, 256, 300, 30.0), (1, 1, 4, 4, 5.0), (32, 8, 128, 1500, 50.0),
                                            (4, 4, 80, 33, 0.0)])
def test_sdpa_softcap(be, hq, hk, d, n, cap):
    """SDPASoftCap (backend.go:235, cpu.go:705-765): Gemma 2's geometry (heads of 256, cap 30), the reference
    test's 4-key case, a context longer than one chunk of the kernel, and cap 0 = plain SDPA."""
    rng = np.random.default_rng(62 + n)
    q = (rng.standard_normal((hq, d)) * 3).astype(np.float32)
    k = (rng.standard_normal((hk, n, d)) * 3).astype(np.float32)
    v = rng.standard_normal((hk, n, d)).astype(np.float32)
    sc = float(np.float32(1 / math.sqrt(d)))
    dq, dk, dv = be.upload(q), be.upload(k), be.upload(v)
    do = be.alloc(q.nbytes)
    be.sdpa_softcap(dq, dk, dv, do, n, hq, hk, d, sc, cap, n * d)
    want = nx.sdpa_softcap(q, k, v, n, hq, hk, d, sc, cap, n * d)
    _close(be.download(do, q.shape, np.float32), want, 1e-5, 3e-6, "sdpa_softcap")
    if cap > 0:
        assert np.abs(want - nx.sdpa(q, k, v, n, hq, hk, d, sc, n * d)).max() > 1e-3   # the cap mattered
    be.reset_pool()


@pytest.mark.parametrize("hq,hk,d,s,cap", [(4, 2, 128, 70, 50.0), (8, 4, 64, 33, 30.0), (8, 4, 256, 40, 50.0),
                                            (4, 2, 128, 70, 0.0)])
def test_sdpa_prefill_softcap(be, hq, hk, d, s, cap):
    """SDPAPrefillSoftCap (backend.go:239, cpu.go:770-841) on the MFMA kernel (heads of 64 / 128) and the generic
    one (256), with scores well into the curved part of the cap."""
    rng = np.random.default_rng(63 + s + d)
    q = (rng.standard_normal((s, hq, d)) * 3).astype(np.float32)
    k = (rng.standard_normal((s, hk, d)) * 3).astype(np.float32)
    v = rng.standard_normal((s, hk, d)).astype(np.float32)
    sc = float(np.float32(1 / math.sqrt(d)))
    dq, dk, dv = be.upload(q), be.upload(k), be.upload(v)
    do = be.alloc(q.nbytes)
    be.sdpa_prefill_softcap(dq, dk, dv, do, s, hq, hk, d, sc, cap)
    want = nx.sdpa_prefill_softcap(q, k, v, s, hq, hk, d, sc, cap)
    # scores reach tens here (inputs scaled by 3): a float32 rounding of a score of 30 moves its weight by 2e-6
    _close(be.download(do, q.shape, np.float32), want, 5e-5, 2e-5, "sdpa_prefill_softcap")
    if cap > 0:
        assert np.abs(want - nx.sdpa_prefill(q, k, v, s, hq, hk, d, sc)).max() > 1e-3
    be.reset_pool()


@pytest.mark.parametrize("neox", [False, True])
def test_rope_with_freqs(be, neox):
    """ScaledRoPEOps.RoPEWithFreqs (backend.go:247-249, cpu.go:308-375) with frequencies that no theta gives
    (scaled_rope_test.go:134-138), with and without K."""
    rng = np.random.default_rng(64)
    d, hq, hk, s, start = 64, 8, 4, 5, 1000
    freqs = (0.01 * np.arange(1, d // 2 + 1)).astype(np.float32)
    q = rng.standard_normal((s, hq, d)).astype(np.float32)
    k = rng.standard_normal((s, hk, d)).astype(np.float32)
    wq, wk = nx.rope_with_freqs(q, k, freqs, d, hq, hk, s, start, neox)
    dq, dk, df = be.upload(q), be.upload(k), be.upload(freqs)
    be.rope_with_freqs(dq, dk, df, d, hq, hk, s, start, neox)
    _close(be.download(dq, q.shape, np.float32), wq, 0, 1e-6, "rope_with_freqs q")
    _close(be.download(dk, k.shape, np.float32), wk, 0, 1e-6, "rope_with_freqs k")
    dq = be.upload(q)
    be.rope_with_freqs(dq, None, df, d, hq, hk, s, start, neox)
    _close(be.download(dq, q.shape, np.float32), wq, 0, 1e-6, "rope_with_freqs, no k")
    be.reset_pool()


# ------------------------------------------------------------------ Medusa heads
@pytest.mark.parametrize("rows,heads,h,v", [(1, 4, 64, 100), (1, 4, 512, 4000), (3, 2, 256, 1000), (8, 1, 128, 260),
                                             (5, 3, 100, 36)])
def test_medusa_forward(be, rows, heads, h, v):
    """Heads.ForwardAll (medusa/heads.go:83-128) for a few hidden states at once against the oracle's Forward per
    head and row; then the heads' top-k (heads.go:146-171) against the oracle's selection."""
    rng = np.random.default_rng(70 + rows + h)
    hidden = (rng.random((rows, h)) * 2 - 1).astype(np.float32)
    fc1 = ((rng.random((heads, h, h)) * 2 - 1) * math.sqrt(2.0 / h)).astype(np.float32)
    fc2 = ((rng.random((heads, h, v)) * 2 - 1) * math.sqrt(2.0 / h)).astype(np.float32)
    dh, d1, d2 = be.upload(hidden), be.upload(fc1), be.upload(fc2)
    di, dl = be.alloc(heads * rows * h * 4), be.alloc(heads * rows * v * 4)
    be.medusa_forward(dh, d1, d2, di, dl, rows, heads, h, v)
    got_i = be.download(di, (heads, rows, h), np.float32)
    got_l = be.download(dl, (heads, rows, v), np.float32)
    for hd in range(heads):
        for r in range(rows):
            wi, wl = nx.medusa_forward(hidden[r], fc1[hd], fc2[hd])
            _close(got_i[hd, r], wi, 1e-5, 2e-6, "medusa intermediate")
            _close(got_l[hd, r], wl, 1e-5, 5e-6, "medusa logits")
    k = 5
    dk, dv = be.alloc(heads * rows * k * 4), be.alloc(heads * rows * k * 4)
    be.topk_rows(dl, heads * rows, v, k, dk, dv)
    idx = be.download(dk, (heads * rows, k), np.int32)
    val = be.download(dv, (heads * rows, k), np.float32)
    flat = got_l.reshape(heads * rows, v)
    for r in range(heads * rows):
        assert idx[r].tolist() == hl.medusa_top_k(flat[r].tolist(), k)
        assert np.array_equal(val[r], flat[r][idx[r]])
    be.reset_pool()


def test_topk_rows_ties_and_unusable_values(be):
    x = np.array([[0.5, 2.0, 2.0, -1.0, 3.0, 2.0],
                  [-np.inf, 1.0, np.nan, -np.inf, -np.inf, np.nan],
                  [7.0, 7.0, 7.0, 7.0, 7.0, 7.0]], dtype=np.float32)
    dx = be.upload(x)
    dk, dv = be.alloc(3 * 6 * 4), be.alloc(3 * 6 * 4)
    be.topk_rows(dx, 3, 6, 6, dk, dv)
    idx = be.download(dk, (3, 6), np.int32)
    for r in range(3):
        assert idx[r].tolist() == hl.medusa_top_k(x[r].tolist(), 6)
    assert idx[0].tolist() == [4, 1, 2, 5, 0, 3] and idx[1].tolist() == [1, -1, -1, -1, -1, -1]
    big = np.random.default_rng(71).standard_normal((2, 128256)).astype(np.float32)
    big[1, 77] = big[1, 100000] = big[1].max() + 1                  # a tie at the top: the lower index first
    db = be.upload(big)
    dk = be.alloc(2 * 10 * 4)
    be.topk_rows(db, 2, 128256, 10, dk)
    idx = be.download(dk, (2, 10), np.int32)
    for r in range(2):
        assert idx[r].tolist() == np.argsort(-big[r].astype(np.float64), kind="stable")[:10].tolist()
    with pytest.raises(RuntimeError, match="exceeds the row length"):
        be.topk_rows(dx, 3, 6, 7, dk)
    with pytest.raises(RuntimeError, match="above 256"):
        be.topk_rows(db, 2, 128256, 257, dk)
    be.reset_pool()


@pytest.mark.parametrize("rows", [1, 5, 32])
@pytest.mark.parametrize("rope_dim,neox,bias,d", [(0, True, True, 64), (32, True, True, 128), (0, False, True, 64),
                                                  (64, False, False, 128)])
def test_decode_attn_qkv_with_bias_and_rope_forms(be, rows, rope_dim, neox, bias, d):
    """vx_decode_attn_qkv_ex: RMSNorm -> Q|K|V (+ biases) -> RoPE in the ropeDim / ropeNeox forms -> paged store, in
    its one-row (matrix-vector) and batched (MFMA) forms, against the oracle's operation sequence
    (block.go:834-868 with matMulTransposedWithBias and applyRoPE)."""
    rng = np.random.default_rng(80 + rows + d)
    hq, hk, hidden, bs, nblocks = 8, 2, 1024, 16, 40
    qd, kvd = hq * d, hk * d
    x = rng.standard_normal((rows, hidden)).astype(np.float32)
    nw = (1 + 0.1 * rng.standard_normal(hidden)).astype(np.float32)
    ws = [qz.random_quant(nx.FMT_Q4_0, rng, n, hidden) for n in (qd, kvd, kvd)]
    bs_ = [(0.1 * rng.standard_normal(n)).astype(np.float32) if bias else None for n in (qd, kvd, kvd)]
    pos = rng.integers(0, 3000, rows).astype(np.int32)
    slots = rng.permutation(nblocks * bs)[:rows].astype(np.int32)
    pool = _make_pool(rng, True, nblocks, bs, hk, d)
    norm = nx.rmsnorm(x, nw, rows, hidden, 1e-5)
    proj = [nx.matmul_quant(nx.FMT_Q4_0, norm, w, rows, n, hidden) for w, n in zip(ws, (qd, kvd, kvd))]
    if bias:
        proj = [nx.add_bias(p, b, rows, n) for p, b, n in zip(proj, bs_, (qd, kvd, kvd))]
    wq, wk = nx.rope_positions(proj[0], proj[1], d, hq, hk, pos, rope_dim, 10000.0, neox)
    want_pool = pool.copy()
    nx.reshape_paged_kv(wk, want_pool, slots // bs, slots % bs, hk, d, bs, False)
    nx.reshape_paged_kv(proj[2], want_pool, slots // bs, slots % bs, hk, d, bs, True)
    dx, dn = be.upload(x), be.upload(nw)
    dws = [be.qweight(nx.FMT_Q4_0, be.upload(w), n, hidden) for w, n in zip(ws, (qd, kvd, kvd))]
    dbs = [be.upload(b) if b is not None else None for b in bs_]
    dpool, dp, ds = be.upload(pool), be.upload(pos), be.upload(slots)
    dq = be.alloc(rows * qd * 4)
    be.decode_attn_qkv_ex(dx, dn, 1e-5, False, dws[0], dws[1], dws[2], dbs[0], dbs[1], dbs[2], rows, dp, ds, dpool, True,
                          hq, hk, d, bs, 10000.0, rope_dim, neox, dq)
    got_q = be.download(dq, (rows, qd), np.float32)
    scale = np.abs(wq).max()
    _close(got_q, wq.reshape(rows, qd), 2e-5, 3e-6 * scale + 1e-7, "fused q")
    got = nx.f16_to_f32_array(be.download(dpool, pool.shape, pool.dtype))
    ref = nx.f16_to_f32_array(want_pool)
    assert np.all(np.abs(got - ref) <= np.abs(ref) * 2.0 ** -9 + 1e-5)        # f16 neighbours where f32 differs in its last bits
    untouched = np.ones(pool.shape, dtype=bool)
    per_blk = 2 * bs * hk * d
    for sl in slots:
        b, o = sl // bs, sl % bs
        untouched[b * per_blk + o * hk * d: b * per_blk + (o + 1) * hk * d] = False
        untouched[b * per_blk + bs * hk * d + o * hk * d: b * per_blk + bs * hk * d + (o + 1) * hk * d] = False
    assert np.array_equal(be.download(dpool, pool.shape, pool.dtype)[untouched], pool[untouched])
    be.reset_pool()


@pytest.mark.parametrize("fmt", [nx.FMT_Q4_0, nx.FMT_Q6_K])
@pytest.mark.parametrize("rows,f16,general", [(1, True, False), (5, True, False), (40, False, True), (130, True, False),
                                              (130, False, False), (200, True, True)])
def test_prefill_attn_qkv_leaves_dense_k_and_v(be, fmt, rows, f16, general):
    """vx_prefill_attn_qkv (a prompt's first chunk, block.go:834-868 + 891-895): Q and the pool as
    vx_decode_attn_qkv_ex leaves them, bit for bit, and the rotated K rows and the V rows as dense floats - the values
    the pool holds (exactly for a float pool, rounded to f16 for an f16 pool) -, against the oracle's operation
    sequence; both RoPE + store kernels (the interleaved whole-head form, and the general one with biases and a
    partial NeoX rotation)."""
    rng = np.random.default_rng(500 + rows + fmt)
    hq, hk, d, hidden, bs, nblocks = 8, 2, 64, 1024, 16, 40
    qd, kvd = hq * d, hk * d
    rope_dim, neox = (32, True) if general else (0, False)
    x = rng.standard_normal((rows, hidden)).astype(np.float32)
    nw = (1 + 0.1 * rng.standard_normal(hidden)).astype(np.float32)
    ws = [qz.random_quant(fmt, rng, n, hidden) for n in (qd, kvd, kvd)]
    bs_ = [(0.1 * rng.standard_normal(n)).astype(np.float32) if general else None for n in (qd, kvd, kvd)]
    pos = np.arange(rows, dtype=np.int32)
    slots = rng.permutation(nblocks * bs)[:rows].astype(np.int32)
    pool = _make_pool(rng, f16, nblocks, bs, hk, d)
    norm = nx.rmsnorm(x, nw, rows, hidden, 1e-5)
    proj = [nx.matmul_quant(fmt, norm, w, rows, n, hidden) for w, n in zip(ws, (qd, kvd, kvd))]
    if general:
        proj = [nx.add_bias(p, b, rows, n) for p, b, n in zip(proj, bs_, (qd, kvd, kvd))]
    want_q, want_k = nx.rope_positions(proj[0], proj[1], d, hq, hk, pos, rope_dim if rope_dim else d, 10000.0, neox)
    dx, dn = be.upload(x), be.upload(nw)
    dws = [be.qweight(fmt, be.upload(w), n, hidden) for w, n in zip(ws, (qd, kvd, kvd))]
    dbs = [be.upload(b) if b is not None else None for b in bs_]
    dp, ds = be.upload(pos), be.upload(slots)
    dpool1, dpool2 = be.upload(pool), be.upload(pool)
    dq1, dq2, dk, dv = be.alloc(rows * qd * 4), be.alloc(rows * qd * 4), be.alloc(rows * kvd * 4), be.alloc(rows * kvd * 4)
    be.decode_attn_qkv_ex(dx, dn, 1e-5, False, dws[0], dws[1], dws[2], dbs[0], dbs[1], dbs[2], rows, dp, ds, dpool1, f16,
                          hq, hk, d, bs, 10000.0, rope_dim, neox, dq1)
    be.prefill_attn_qkv(dx, dn, 1e-5, False, dws[0], dws[1], dws[2], dbs[0], dbs[1], dbs[2], rows, dp, ds, dpool2, f16,
                        hq, hk, d, bs, 10000.0, rope_dim, neox, dq2, dk, dv)
    q1, q2 = be.download(dq1, (rows, qd), np.float32), be.download(dq2, (rows, qd), np.float32)
    p1, p2 = be.download(dpool1, pool.shape, pool.dtype), be.download(dpool2, pool.shape, pool.dtype)
    k, v = be.download(dk, (rows, kvd), np.float32), be.download(dv, (rows, kvd), np.float32)
    if rows > 1:   # (one row: the decode entry point takes the matrix-vector kernels, whose sums are added in another order)
        assert np.array_equal(q1.view(np.uint32), q2.view(np.uint32))
        assert np.array_equal(p1, p2)
    scale = np.abs(want_q).max()
    _close(q2, want_q.reshape(rows, qd), 2e-5, 3e-6 * scale + 1e-7, "q")
    _close(k, want_k.reshape(rows, kvd), 2e-5, 3e-6 * np.abs(want_k).max() + 1e-7, "dense k")
    _close(v, proj[2].reshape(rows, kvd), 2e-5, 3e-6 * np.abs(proj[2]).max() + 1e-7, "dense v")
    per_blk = 2 * bs * kvd
    for r, sl in enumerate(slots):
        b, o = int(sl) // bs, int(sl) % bs
        pk = p2[b * per_blk + o * kvd: b * per_blk + (o + 1) * kvd]
        pv_ = p2[b * per_blk + bs * kvd + o * kvd: b * per_blk + bs * kvd + (o + 1) * kvd]
        if f16:
            assert np.array_equal(pk, nx.f32_to_f16_array(k[r])) and np.array_equal(pv_, nx.f32_to_f16_array(v[r])), r
        else:
            assert np.array_equal(pk.view(np.uint32), k[r].view(np.uint32)), r
            assert np.array_equal(pv_.view(np.uint32), v[r].view(np.uint32)), r
    be.reset_pool()


@pytest.mark.parametrize("hq,hk,d,hidden", [(32, 32, 128, 4096), (32, 8, 128, 4096), (24, 8, 128, 3072)])
def test_in_kernel_merge_equals_the_separate_merge_and_the_oracle(be, hq, hk, d, hidden):
    """The attention kernel's own merge of its splits (vx_backend_set_attn_merge, the default) against the merge left
    to vx_decode_ffn, at the north-star head geometry and two grouped-query ones: over 24 launches with changing
    ragged lengths (up to nine splits per sequence, sequences without tokens, lengths on split boundaries) the
    layer outputs of the two forms are the same bits, launch after launch; and the first launch's attention output,
    merged in the kernel and fed through Wo, matches the oracle's paged attention and MatMulQ4_0."""
    rng = np.random.default_rng(hq * 7 + hk)
    fmt, rows, ffn = nx.FMT_Q4_0, 32, 1024
    bs, eps = 16, 1e-5
    max_blocks = 290
    nblocks = 32 * 140
    dims = dict(wo=(hidden, hq * d), w1=(ffn, hidden), w3=(ffn, hidden), w2=(hidden, ffn))
    raw = {n: qz.random_quant(fmt, rng, *dims[n]) for n in dims}
    dW = {n: be.upload(raw[n], permanent=True) for n in dims}
    qw = {n: be.qweight(fmt, dW[n], *dims[n]) for n in dims}
    pool = _make_pool(rng, True, nblocks, bs, hk, d)
    q = rng.standard_normal((rows, hq * d)).astype(np.float32)
    x = rng.standard_normal((rows, hidden)).astype(np.float32)
    nw = (1.0 + 0.1 * rng.standard_normal(hidden)).astype(np.float32)
    dpool, dq, dnw = be.upload(pool, permanent=True), be.upload(q, permanent=True), be.upload(nw, permanent=True)
    scale = np.float32(1.0 / math.sqrt(d))
    dl, dt = be.alloc_permanent(rows * 4), be.alloc_permanent(rows * max_blocks * 4)
    dx = be.alloc_permanent(rows * hidden * 4)
    try:
        for launch in range(24):
            lens = np.clip(np.exp(rng.normal(math.log(600), 0.9, rows)), 1, max_blocks * bs).astype(np.int32)
            lens[launch % rows] = 0
            lens[(launch + 3) % rows] = 512 * (1 + launch % 4)
            lens[(launch + 7) % rows] = 512 * (1 + launch % 3) + 1
            perm = rng.permutation(nblocks).astype(np.int32)
            tables = np.zeros((rows, max_blocks), dtype=np.int32)
            off = 0
            for i, L in enumerate(lens):
                nb = (int(L) + bs - 1) // bs
                tables[i, :nb] = perm[off:off + nb]
                off += nb
            be.to_device(dl, lens)
            be.to_device(dt, tables)
            outs = []
            for merge in (True, False):
                be.set_attn_merge(merge)
                be.to_device(dx, x)
                be.sdpa_paged_decode_ragged(dq, dpool, True, dt, dl, None, rows, max_blocks, bs, hq, hk, d, scale, max_blocks * bs)
                be.decode_ffn(None, dx, qw["wo"], dnw, eps, qw["w1"], qw["w3"], qw["w2"], rows, None)
                outs.append(be.download(dx, (rows, hidden), np.float32))
            assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32)), "launch %d" % launch
            if launch == 0:
                attn = nx.sdpa_paged_decode_batched(q.reshape(rows, hq, d), pool, tables, bs, hq, hk, d, scale, lens)
                attn = np.where((lens > 0)[:, None], attn.reshape(rows, hq * d), 0.0).astype(np.float32)
                x1 = nx.add(x, nx.matmul_quant(fmt, attn, raw["wo"], rows, hidden, hq * d))
                h2 = nx.rmsnorm(x1, nw, rows, hidden, eps)
                g = nx.matmul_quant(fmt, h2, raw["w1"], rows, ffn, hidden)
                u = nx.matmul_quant(fmt, h2, raw["w3"], rows, ffn, hidden)
                want = nx.add(x1, nx.matmul_quant(fmt, nx.silu_mul(g, u), raw["w2"], rows, hidden, ffn))
                _close(outs[0], want, 2e-4, 2e-5 * np.abs(want).max(), "merged in the kernel, against the oracle")
    finally:
        be.set_attn_merge(True)
        for p in list(dW.values()) + [dpool, dq, dnw, dl, dt, dx]:
            be.free(p)
        be.reset_pool()
