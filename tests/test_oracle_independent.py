"""Pins the oracle where the reference's own vectors leave it open: exhaustive code
sweeps against independent implementations (numpy.float16, float64 arithmetic, naive
list models), closed forms and invariants chosen so a plausible slip (wrong nibble,
dropped term, transposed index, wrong sign) fails."""
import math

import numpy as np
import pytest

from oracle import numerics as nx
from oracle import quantize as qz
from oracle import host_logic as hl


# ----------------------------------------------------------------- half precision
def test_f16_to_f32_all_65536_patterns():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = nx.f16_to_f32_array(bits)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    # the cpu.go twin agrees on every non-NaN pattern
    got_cpu = np.array([nx.f16_to_f32_cpu(int(b)) for b in bits[::7]], dtype=np.float32)
    w7 = want[::7]
    ok = ~np.isnan(w7)
    assert np.array_equal(got_cpu[ok].view(np.uint32), w7[ok].view(np.uint32))


def test_f32_to_f16_rne_against_numpy():
    rng = np.random.default_rng(0)
    xs = [rng.standard_normal(200000).astype(np.float32),
          (rng.standard_normal(50000) * 1e-6).astype(np.float32),     # subnormal halves
          (rng.standard_normal(50000) * 3e4).astype(np.float32),      # near overflow
          rng.integers(0, 2**32, 200000, dtype=np.uint64).astype(np.uint32).view(np.float32)]
    # every half value, its neighbours' midpoints (ties) and one ulp around them
    h = np.arange(0x7C00, dtype=np.uint16).view(np.float16).astype(np.float64)
    mids = ((h[:-1] + h[1:]) / 2).astype(np.float32)
    xs += [h.astype(np.float32), mids, np.nextafter(mids, np.float32(np.inf)),
           np.nextafter(mids, np.float32(-np.inf)), -mids,
           np.array([65504, 65519.996, 65520, 65536, 1e30, np.inf, -np.inf, 0.0, -0.0,
                     2.0**-25, np.nextafter(np.float32(2.0**-25), np.float32(1)), 2.0**-24], dtype=np.float32)]
    x = np.concatenate(xs)
    with np.errstate(over="ignore", invalid="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = nx.f32_to_f16_array(x)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all((got[nan] & 0x7C00) == 0x7C00) and np.all((got[nan] & 0x3FF) != 0)


# ----------------------------------------------------------------- dequant closed forms
def _f16(v):
    return np.float32(np.float16(v))


def test_q4_0_exhaustive_codes_and_positions():
    for scale in (1.0, 0.5, -0.0123, 3.1e-5):
        for shift in range(16):
            vals = [(i + shift) % 16 for i in range(32)]
            blk = qz.encode_q4_0_block(scale, vals)
            r = nx.dequantize(nx.FMT_Q4_0, blk, 32)
            want = np.array([_f16(scale) * np.float32(v - 8) for v in vals], dtype=np.float32)
            assert np.array_equal(r, want)


def test_q8_0_exhaustive_codes():
    for scale in (1.0, 0.0371, -2.5):
        for base in range(0, 256, 32):
            vals = np.arange(base, base + 32).astype(np.uint8).view(np.int8)
            blk = qz.encode_q8_0_block(scale, vals)
            r = nx.dequantize(nx.FMT_Q8_0, blk, 32)
            want = np.array([_f16(scale) * np.float32(int(v)) for v in vals], dtype=np.float32)
            assert np.array_equal(r, want)


def test_get_scale_min_k4_all_6bit_values():
    rng = np.random.default_rng(3)
    for _ in range(200):
        sc = rng.integers(0, 64, 8)
        mn = rng.integers(0, 64, 8)
        packed = qz.pack_q4_k_scales(sc, mn)
        for j in range(8):
            assert nx.get_scale_min_k4(j, packed) == (int(sc[j]), int(mn[j]))
    for j in range(8):  # every 6-bit value in every slot
        for v in range(64):
            sc = np.zeros(8, dtype=int); mn = np.zeros(8, dtype=int)
            sc[j] = v; mn[j] = 63 - v
            assert nx.get_scale_min_k4(j, qz.pack_q4_k_scales(sc, mn)) == (v, 63 - v)


def test_q4_k_closed_form():
    """element = (d*sc)*q - (dmin*m), each product rounded to float32 first."""
    rng = np.random.default_rng(4)
    for _ in range(20):
        d, dmin = float(rng.uniform(1e-4, 0.1)), float(rng.uniform(1e-4, 0.1))
        sc = rng.integers(0, 64, 8); mn = rng.integers(0, 64, 8)
        vals = rng.integers(0, 16, 256)
        blk = qz.encode_q4_k_block(d, dmin, sc, mn, vals)
        r = nx.dequantize(nx.FMT_Q4_K, blk, 256)
        df, dmf = _f16(d), _f16(dmin)
        want = np.empty(256, dtype=np.float32)
        for i in range(256):
            sb = i // 32
            d1 = np.float32(df * np.float32(sc[sb]))
            dm1 = np.float32(dmf * np.float32(mn[sb]))
            want[i] = np.float32(np.float32(d1 * np.float32(vals[i])) - dm1)
        assert np.array_equal(r, want)


def test_q6_k_closed_form():
    """element = (d*sc)*q with q in [-32,31] and int8 scales per 16 elements."""
    rng = np.random.default_rng(5)
    for _ in range(20):
        d = float(rng.uniform(1e-5, 0.01)) * (1 if rng.random() < 0.5 else -1)
        sc = rng.integers(-128, 128, 16)
        vals = rng.integers(-32, 32, 256)
        blk = qz.encode_q6_k_block(d, sc, vals)
        r = nx.dequantize(nx.FMT_Q6_K, blk, 256)
        df = _f16(d)
        want = np.array([np.float32(np.float32(df * np.float32(sc[i // 16])) * np.float32(vals[i]))
                         for i in range(256)], dtype=np.float32)
        assert np.array_equal(r, want)
    # every 6-bit code in every position class
    for shift in range(64):
        vals = np.array([((i + shift) % 64) - 32 for i in range(256)])
        blk = qz.encode_q6_k_block(1.0, np.ones(16, dtype=int), vals)
        assert np.array_equal(nx.dequantize(nx.FMT_Q6_K, blk, 256), vals.astype(np.float32))


def test_q5_0_closed_form_every_code_in_every_position():
    """element = float32(q - 16) * d; the encoder states the layout on its own (bit i of qh = fifth bit of
    element i), so a swapped half or a wrong bit index fails."""
    rng = np.random.default_rng(7)
    for shift in range(32):
        vals = np.array([(i * 7 + shift) % 32 for i in range(32)])
        blk = qz.encode_q5_0_block(1.0, vals)
        assert np.array_equal(nx.dequantize(nx.FMT_Q5_0, blk, 32), (vals - 16).astype(np.float32))
    for _ in range(20):
        d = float(rng.uniform(1e-4, 0.1)) * (1 if rng.random() < 0.5 else -1)
        vals = rng.integers(0, 32, 32)
        r = nx.dequantize(nx.FMT_Q5_0, qz.encode_q5_0_block(d, vals), 32)
        want = np.array([np.float32(np.float32(v - 16) * _f16(d)) for v in vals], dtype=np.float32)
        assert np.array_equal(r, want)


def test_q5_k_closed_form():
    """element = (d*sc)*q - (dmin*m) with q in [0,31]: Q4_K's arithmetic with a fifth bit from qh."""
    rng = np.random.default_rng(8)
    # a single high bit set: exactly one element differs from the four-bit block
    for e in (0, 31, 32, 100, 223, 255):
        vals = np.zeros(256, dtype=int)
        vals[e] = 16
        blk = qz.encode_q5_k_block(1.0, 0.0, np.ones(8, dtype=int), np.zeros(8, dtype=int), vals)
        assert np.array_equal(nx.dequantize(nx.FMT_Q5_K, blk, 256), vals.astype(np.float32))
    for _ in range(20):
        d, dmin = float(rng.uniform(1e-4, 0.1)), float(rng.uniform(1e-4, 0.1))
        sc = rng.integers(0, 64, 8); mn = rng.integers(0, 64, 8)
        vals = rng.integers(0, 32, 256)
        r = nx.dequantize(nx.FMT_Q5_K, qz.encode_q5_k_block(d, dmin, sc, mn, vals), 256)
        df, dmf = _f16(d), _f16(dmin)
        want = np.empty(256, dtype=np.float32)
        for i in range(256):
            sb = i // 32
            d1 = np.float32(df * np.float32(sc[sb]))
            dm1 = np.float32(dmf * np.float32(mn[sb]))
            want[i] = np.float32(np.float32(d1 * np.float32(vals[i])) - dm1)
        assert np.array_equal(r, want)
    # with the fifth bits clear a Q5_K block decodes as the Q4_K block with the same header and nibbles
    vals = rng.integers(0, 16, 256)
    sc = rng.integers(0, 64, 8); mn = rng.integers(0, 64, 8)
    assert np.array_equal(nx.dequantize(nx.FMT_Q5_K, qz.encode_q5_k_block(0.01, 0.02, sc, mn, vals), 256),
                          nx.dequantize(nx.FMT_Q4_K, qz.encode_q4_k_block(0.01, 0.02, sc, mn, vals), 256))


def test_bf16_all_patterns_against_numpy():
    h = np.arange(65536, dtype=np.uint16)
    got = nx.dequantize(nx.FMT_BF16, h.view(np.uint8), 65536)
    want = (h.astype(np.uint32) << 16).view(np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # the synthetic-weight maker rounds to nearest even
    w = np.array([[1.0, 1.00390625, 1.005859375, -3.0e-5]], dtype=np.float32)
    back = nx.dequantize(nx.FMT_BF16, qz.quantize_bf16(w), 4)
    assert back[0] == 1.0 and back[1] == 1.0 and back[2] == np.float32(1.0078125)
    assert abs(back[3] + 3.0e-5) < 3.0e-5 * 2 ** -8


def test_multi_block_and_partial_count():
    rng = np.random.default_rng(6)
    w = rng.standard_normal((3, 128)).astype(np.float32)
    q = qz.quantize_q4_0(w)
    full = nx.dequantize(nx.FMT_Q4_0, q, 3 * 128)
    part = nx.dequantize(nx.FMT_Q4_0, q, 3 * 128 - 5)
    assert np.array_equal(full[:-5], part)
    assert np.max(np.abs(full.reshape(3, 128) - w)) < np.abs(w).max() / 7.0


# ----------------------------------------------------------------- matmul
@pytest.mark.parametrize("fmt", [nx.FMT_Q4_0, nx.FMT_Q8_0, nx.FMT_Q4_K, nx.FMT_Q6_K, nx.FMT_Q5_0, nx.FMT_Q5_K,
                                 nx.FMT_BF16])
def test_quant_matmul_vs_float64_of_exact_dequant(fmt):
    rng = np.random.default_rng(10 + fmt)
    m, n, k = 3, 5, 512
    w = qz.random_quant(fmt, rng, n, k)
    a = rng.standard_normal((m, k)).astype(np.float32)
    got = nx.matmul_quant(fmt, a, w, m, n, k)
    wd = nx.dequantize(fmt, w, n * k).reshape(n, k).astype(np.float64)
    want = a.astype(np.float64) @ wd.T
    assert np.allclose(got, want, rtol=0, atol=1e-5 * np.abs(want).max() + 1e-6)
    # row r of a batch equals the same row computed alone (sequential-loop semantics)
    for r in range(m):
        assert np.array_equal(nx.matmul_quant(fmt, a[r], w, 1, n, k)[0], got[r])


def test_matmul_q4_0_native_loop_order_differs_from_dequant_only_in_last_bits():
    rng = np.random.default_rng(20)
    n, k = 4, 256
    w = qz.random_quant(nx.FMT_Q4_0, rng, n, k)
    a = rng.standard_normal((2, k)).astype(np.float32)
    nat = nx.matmul_q4_0(a, w, 2, n, k)
    via = nx.matmul_quant_via_dequant(nx.FMT_Q4_0, a, w, 2, n, k)
    assert np.allclose(nat, via, rtol=1e-5, atol=1e-6)
    # explicit restatement of the native order for one output, element by element
    wd = nx.dequantize(nx.FMT_Q4_0, w, n * k).reshape(n, k)
    s = np.float32(0)
    for blk in range(k // 32):
        for i in range(16):
            s = np.float32(s + np.float32(a[0, blk * 32 + i] * wd[0, blk * 32 + i]))
            s = np.float32(s + np.float32(a[0, blk * 32 + i + 16] * wd[0, blk * 32 + i + 16]))
    assert s == nat[0, 0]


def test_matmul_f32_vs_numpy():
    rng = np.random.default_rng(21)
    a = rng.standard_normal((4, 37)).astype(np.float32)
    b = rng.standard_normal((6, 37)).astype(np.float32)
    assert np.allclose(nx.matmul_t_f32(a, b, 4, 6, 37), a.astype(np.float64) @ b.T.astype(np.float64), atol=1e-5)
    assert np.allclose(nx.matmul_f32(a, b.T.copy(), 4, 6, 37), a.astype(np.float64) @ b.T.astype(np.float64), atol=1e-5)


# ----------------------------------------------------------------- elementwise
def test_rmsnorm_vs_float64():
    rng = np.random.default_rng(30)
    x = rng.standard_normal((5, 300)).astype(np.float32) * 3
    w = rng.standard_normal(300).astype(np.float32)
    got = nx.rmsnorm(x, w, 5, 300, 1e-5)
    x64 = x.astype(np.float64)
    want = x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + 1e-5) * w
    assert np.allclose(got, want, rtol=2e-6, atol=1e-6)


def test_rope_closed_form_and_additivity():
    rng = np.random.default_rng(31)
    d, hq, hk, s = 64, 4, 2, 5
    q = rng.standard_normal((s, hq, d)).astype(np.float32)
    k = rng.standard_normal((s, hk, d)).astype(np.float32)
    q2, k2 = nx.rope(q, k, d, hq, hk, s, 7, 0, 10000.0, False)
    q2 = q2.reshape(s, hq, d); k2 = k2.reshape(s, hk, d)
    for t in range(s):
        pos = 7 + t
        for j in range(d // 2):
            ang = pos * (10000.0 ** (-2.0 * j / d))
            c, sn = math.cos(ang), math.sin(ang)
            want0 = q[t, :, 2 * j] * c - q[t, :, 2 * j + 1] * sn
            want1 = q[t, :, 2 * j] * sn + q[t, :, 2 * j + 1] * c
            assert np.allclose(q2[t, :, 2 * j], want0, atol=2e-5)
            assert np.allclose(q2[t, :, 2 * j + 1], want1, atol=2e-5)
            wk0 = k[t, :, 2 * j] * c - k[t, :, 2 * j + 1] * sn
            assert np.allclose(k2[t, :, 2 * j], wk0, atol=2e-5)
    # norms of pairs are preserved; rotating by a then b ~ rotating by a+b for the first pair (freq 1)
    assert np.allclose((q2 ** 2).sum(-1), (q ** 2).sum(-1), rtol=1e-5)
    # per-row positions == one-row calls
    pos = [3, 11, 0, 7, 4096]
    qp, kp = nx.rope_positions(q, k, d, hq, hk, pos, 0, 10000.0, False)
    for t, p in enumerate(pos):
        a, b = nx.rope(q[t], k[t], d, hq, hk, 1, p, 0, 10000.0, False)
        assert np.array_equal(qp.reshape(s, -1)[t], a.ravel()) and np.array_equal(kp.reshape(s, -1)[t], b.ravel())


def test_rope_neox_pairs():
    q = np.zeros(8, dtype=np.float32); q[1] = 1.0
    r, _ = nx.rope(q, None, 8, 1, 0, 1, 3, 0, 10000.0, True)
    ang = 3 * 10000.0 ** (-2.0 / 8)
    assert abs(r[1] - math.cos(ang)) < 1e-6 and abs(r[5] - math.sin(ang)) < 1e-6


def test_softmax_silu_vs_float64():
    rng = np.random.default_rng(32)
    x = rng.standard_normal((3, 50)).astype(np.float32) * 4
    e = np.exp(x.astype(np.float64) - x.max(axis=1, keepdims=True))
    assert np.allclose(nx.softmax(x, 3, 50), e / e.sum(axis=1, keepdims=True), rtol=1e-5, atol=1e-8)
    g = rng.standard_normal(100).astype(np.float32) * 3
    u = rng.standard_normal(100).astype(np.float32)
    want = g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64))) * u
    assert np.allclose(nx.silu_mul(g, u), want, rtol=1e-5, atol=1e-7)


# ----------------------------------------------------------------- attention
def _ref_attention64(q, K, V, scale):
    s = (K.astype(np.float64) @ q.astype(np.float64)) * scale
    e = np.exp(s - s.max())
    return (e / e.sum()) @ V.astype(np.float64)


def test_sdpa_vs_float64_gqa():
    rng = np.random.default_rng(40)
    hq, hk, d, L, stride = 8, 2, 16, 37, 64
    q = rng.standard_normal((hq, d)).astype(np.float32)
    k = rng.standard_normal((hk, stride, d)).astype(np.float32)
    v = rng.standard_normal((hk, stride, d)).astype(np.float32)
    sc = np.float32(1 / math.sqrt(d))
    out = nx.sdpa(q, k, v, L, hq, hk, d, sc, stride * d)
    for h in range(hq):
        want = _ref_attention64(q[h], k[h // 4, :L], v[h // 4, :L], float(sc))
        assert np.allclose(out[h], want, rtol=1e-5, atol=1e-6)


def test_sdpa_prefill_is_causal_sdpa():
    rng = np.random.default_rng(41)
    s, hq, hk, d = 9, 4, 2, 8
    q = rng.standard_normal((s, hq, d)).astype(np.float32)
    k = rng.standard_normal((s, hk, d)).astype(np.float32)
    v = rng.standard_normal((s, hk, d)).astype(np.float32)
    sc = np.float32(1 / math.sqrt(d))
    out = nx.sdpa_prefill(q, k, v, s, hq, hk, d, sc)
    khm = np.ascontiguousarray(k.transpose(1, 0, 2)); vhm = np.ascontiguousarray(v.transpose(1, 0, 2))
    for t in range(s):
        one = nx.sdpa(q[t], khm, vhm, t + 1, hq, hk, d, sc, s * d)
        assert np.array_equal(out[t], one)  # same loop body, same order -> bit equal


@pytest.mark.parametrize("f16", [False, True])
def test_paged_equals_contiguous(f16):
    """inference/backend/metal/paged_sdpa_test.go:16-335: paged == contiguous on the same
    K/V, incl. partial last block, GQA and a scattered physical mapping {5,2,7}."""
    rng = np.random.default_rng(42)
    bs, hq, hk, d = 4, 4, 2, 8
    L = 10  # 3 blocks, 2 tokens in the last
    phys = [5, 2, 7]
    k = rng.standard_normal((L, hk, d)).astype(np.float32)
    v = rng.standard_normal((L, hk, d)).astype(np.float32)
    q = rng.standard_normal((hq, d)).astype(np.float32)
    pool = np.zeros(8 * 2 * bs * hk * d, dtype=np.uint16 if f16 else np.float32)
    bi = [phys[p // bs] for p in range(L)]; bo = [p % bs for p in range(L)]
    nx.reshape_paged_kv(k, pool, bi, bo, hk, d, bs, False)
    nx.reshape_paged_kv(v, pool, bi, bo, hk, d, bs, True)
    if f16:
        k = nx.f16_to_f32_array(nx.f32_to_f16_array(k)); v = nx.f16_to_f32_array(nx.f32_to_f16_array(v))
    sc = np.float32(1 / math.sqrt(d))
    got = nx.sdpa_paged_decode(q, pool, phys, 3, bs, hq, hk, d, sc, 2)
    khm = np.ascontiguousarray(k.transpose(1, 0, 2)); vhm = np.ascontiguousarray(v.transpose(1, 0, 2))
    want = nx.sdpa(q, khm, vhm, L, hq, hk, d, sc, L * d)
    assert np.array_equal(got, want)
    # exact-layout check (paged_test.go:96-127): K of token 6 head 1 sits at block 2, offset 2
    part = bs * hk * d
    base = 2 * 2 * part + 2 * hk * d + 1 * d
    seg = pool[base:base + d]
    seg = nx.f16_to_f32_array(seg) if f16 else seg
    assert np.array_equal(seg, k[6, 1])
    vseg = pool[base + part:base + part + d]
    vseg = nx.f16_to_f32_array(vseg) if f16 else vseg
    assert np.array_equal(vseg, v[6, 1])
    # kvLen = 1 -> out = V of the mapped kv head (inference/runtime/paged_kv_test.go:161-175)
    one = nx.sdpa_paged_decode(q, pool, phys, 1, bs, hq, hk, d, sc, 1)
    for h in range(hq):
        assert np.allclose(one[h], v[0, h // 2], atol=1e-6)
    # batched == per sequence (paged_batched_test.go), and multiquery == per-query decode
    bts = np.array([[5, 2, 7], [5, 2, -1]], dtype=np.int32)
    qb = rng.standard_normal((2, hq, d)).astype(np.float32)
    outb = nx.sdpa_paged_decode_batched(qb, pool, bts, bs, hq, hk, d, sc, [10, 7])
    assert np.array_equal(outb[0], nx.sdpa_paged_decode(qb[0], pool, phys, 3, bs, hq, hk, d, sc, 2))
    assert np.array_equal(outb[1], nx.sdpa_paged_decode(qb[1], pool, phys, 2, bs, hq, hk, d, sc, 3))
    mq = nx.sdpa_paged_multiquery(qb, pool, phys, [7, 10], bs, hq, hk, d, sc)
    assert np.array_equal(mq[0], nx.sdpa_paged_decode(qb[0], pool, phys, 2, bs, hq, hk, d, sc, 3))
    assert np.array_equal(mq[1], nx.sdpa_paged_decode(qb[1], pool, phys, 3, bs, hq, hk, d, sc, 2))


def test_tree_mask_multiquery_equals_path_attention():
    """With the ancestor mask, node i must see exactly prefix + its root path: compare with
    an unmasked query over a pool that holds only that path."""
    rng = np.random.default_rng(43)
    bs, hq, hk, d, base = 4, 2, 1, 8, 5
    parent = [-1, -1, 0, 0, 1]
    n = len(parent)
    mask = np.array(hl.build_tree_attention_mask(n, parent), dtype=np.uint8)
    total = base + n
    k = rng.standard_normal((total, hk, d)).astype(np.float32)
    v = rng.standard_normal((total, hk, d)).astype(np.float32)
    q = rng.standard_normal((n, hq, d)).astype(np.float32)
    nblk = (total + bs - 1) // bs
    bt = list(range(nblk))
    pool = np.zeros(nblk * 2 * bs * hk * d, dtype=np.float32)
    nx.reshape_paged_kv(k, pool, [p // bs for p in range(total)], [p % bs for p in range(total)], hk, d, bs, False)
    nx.reshape_paged_kv(v, pool, [p // bs for p in range(total)], [p % bs for p in range(total)], hk, d, bs, True)
    sc = np.float32(1 / math.sqrt(d))
    got = nx.sdpa_paged_multiquery(q, pool, bt, None, bs, hq, hk, d, sc, tree_mask=mask, tree_base=base)
    for i in range(n):
        path = []
        j = i
        while j >= 0:
            path.append(j); j = parent[j]
        rows = list(range(base)) + [base + j for j in sorted(path)]
        K = np.ascontiguousarray(k[rows].transpose(1, 0, 2)); V = np.ascontiguousarray(v[rows].transpose(1, 0, 2))
        want = nx.sdpa(q[i], K, V, len(rows), hq, hk, d, sc, len(rows) * d)
        assert np.array_equal(got[i], want)


# ----------------------------------------------------------------- pool / packing
def test_block_pool_vs_naive_model_random_trace():
    """gpu_block_pool.go alloc/free order against an independent LIFO-stack model."""
    rng = np.random.default_rng(50)
    bs, maxb = 4, 24
    pool = hl.GPUBlockPool(2, 1, 8, bs, maxb)
    stack = list(range(maxb))           # naive model of one layer
    tables, lens = {}, {}
    next_id = 1
    for _ in range(400):
        op = rng.integers(0, 4)
        if op == 0 or not tables:
            pool.create_sequence(next_id); tables[next_id] = []; lens[next_id] = 0; next_id += 1
        elif op == 1:
            sid = int(rng.choice(list(tables)))
            n = int(rng.integers(1, 6))
            need = (lens[sid] + n - 1) // bs + 1 - len(tables[sid])
            if need > len(stack):
                with pytest.raises(hl.PoolError):
                    for layer in range(2):
                        pool.store_kv_slots(layer, sid, lens[sid], n)
                # the reference leaves partially allocated blocks in the table on failure
                for sid2 in tables:
                    tables[sid2] = list(pool.seqs[sid2].block_tables[0])
                stack = list(pool.free_lists[0])
                continue
            for layer in range(2):
                slots = pool.store_kv_slots(layer, sid, lens[sid], n)
            for _b in range(need):
                tables[sid].append(stack.pop())
            want = [(tables[sid][(lens[sid] + i) // bs], (lens[sid] + i) % bs) for i in range(n)]
            assert slots == want
            lens[sid] += n
        elif op == 2:
            sid = int(rng.choice(list(tables)))
            new = int(rng.integers(0, lens[sid] + 3))
            pool.truncate_sequence(sid, new)
            if new < lens[sid]:
                keep = 0 if new == 0 else (new - 1) // bs + 1
                for b in tables[sid][keep:]:
                    stack.append(b)
                tables[sid] = tables[sid][:keep]; lens[sid] = new
        else:
            sid = int(rng.choice(list(tables)))
            pool.delete_sequence(sid)
            for b in tables[sid]:
                stack.append(b)
            del tables[sid]; del lens[sid]
        for sid in tables:
            assert pool.seqs[sid].block_tables[0] == tables[sid] == pool.seqs[sid].block_tables[1]
            assert pool.seqs[sid].seq_len == lens[sid]
        assert pool.free_lists[0] == stack


def test_first_blocks_come_from_the_tail():
    pool = hl.GPUBlockPool(1, 1, 8, 16, 10)
    pool.create_sequence(7)
    pool.store_kv_slots(0, 7, 0, 33)
    assert pool.seqs[7].block_tables[0] == [9, 8, 7]      # gpu_block_pool.go:205-206
    bt, nb, til = pool.attention_args(0, 7)
    assert (nb, til) == (3, 1)
    bt, nb, til = pool.attention_args(0, 7, kv_len=16)
    assert (nb, til) == (1, 16)
    assert hl.int32_le_bytes([1, -1, 258]) == bytes([1, 0, 0, 0, 255, 255, 255, 255, 2, 1, 0, 0])


def test_slot_math_all_positions():
    for bs in (1, 4, 16):
        pool = hl.GPUBlockPool(1, 1, 8, bs, 64)
        pool.create_sequence(1)
        for pos in range(3 * bs + 2):
            (blk, off), = pool.store_kv_slots(0, 1, pos, 1)
            assert off == pos % bs and blk == 63 - pos // bs


def test_share_blocks_refcounts():
    pool = hl.GPUBlockPool(2, 1, 8, 4, 10)
    pool.create_sequence(1); pool.create_sequence(2)
    for layer in range(2):
        pool.store_kv_slots(layer, 1, 0, 9)
    pool.share_blocks(1, 2, 8)
    assert pool.seqs[2].block_tables[0] == pool.seqs[1].block_tables[0][:2]
    assert pool.block_stats() == (20, 14, 4)
    pool.delete_sequence(1)
    assert pool.block_stats() == (20, 16, 0)     # shared blocks survive with refcount 1
    pool.delete_sequence(2)
    assert pool.block_stats() == (20, 20, 0)
    with pytest.raises(hl.PoolError):
        pool.share_blocks(5, 2, 4)


def test_pack_batch_matches_sequential_calls():
    pool = hl.GPUBlockPool(1, 1, 8, 4, 32)
    ref = hl.GPUBlockPool(1, 1, 8, 4, 32)
    ctx = {3: 5, 4: 8, 9: 1}
    for p in (pool, ref):
        for sid, n in ctx.items():
            p.create_sequence(sid); p.store_kv_slots(0, sid, 0, n)
    ids = [3, 4, 9]
    pos = [ctx[s] for s in ids]
    pk = hl.pack_batch(pool, 0, ids, pos)
    assert pk["cu_seqlens"] == [0, 1, 2, 3] and pk["kv_lens"] == [6, 9, 2]
    want_slots = []
    for sid, p in zip(ids, pos):
        (blk, off), = ref.store_kv_slots(0, sid, p, 1)
        want_slots.append(blk * 4 + off)
    assert pk["slot_mapping"] == want_slots and pk["token_pos"] == pos
    assert pk["max_blocks"] == 3 and pk["block_tables"][2][1:] == [-1, -1]
    # a sequence at a block boundary takes the next tail block, in batch order
    assert pk["block_tables"][1][2] == ref.seqs[4].block_tables[0][2]


def test_sequence_next_input_token():
    s = hl.Sequence(kv_seq_id=5, prompt_tokens=[11, 12])
    assert s.next_input_token() == (11, 0, True)
    s.advance_position(); assert s.next_input_token() == (12, 1, True)
    s.advance_position(); assert s.next_input_token() == (0, 0, False)
    s.generated.append(77)
    assert s.next_input_token() == (77, 2, True)
    s2 = hl.Sequence(kv_seq_id=6, prompt_tokens=[1, 2, 3]); s2.set_prefill_complete(3); s2.generated.append(9)
    assert hl.pack_decode_inputs([s, s2]) == ([77, 9], [2, 3], [5, 6])
    assert hl.pack_decode_inputs([hl.Sequence(1, [])]) == ([1], [0], [1])


def test_greedy_tree_accept_equals_best_linear_path():
    tokens = [10, 11, 20, 21, 20, 21]
    parent = [-1, -1, 0, 0, 1, 1]
    # model wants 11 then 20 then 99
    acc, final = hl.greedy_tree_accept(tokens, parent, 11, [0, 20, 0, 0, 99, 0])
    assert acc == [1, 4] and final == 99
    assert hl.verify_tree_path([11, 20], [11, 20, 99]) == (2, 99)
    acc, final = hl.greedy_tree_accept(tokens, parent, 55, [0] * 6)
    assert acc == [] and final == 55


@pytest.mark.parametrize("fmt", [nx.FMT_Q4_0, nx.FMT_Q8_0, nx.FMT_Q6_K])
def test_row_sliced_matmul_has_the_same_bits(fmt):
    """set_row_threads() cuts the weight rows into slices computed side by side (long GPU parity runs use it to
    shorten the oracle's share): every output element is the same loop, so the result is bit-identical."""
    rng = np.random.default_rng(300 + fmt)
    m, n, k = 3, 1536, 1024
    w = qz.random_quant(fmt, rng, n, k)
    a = rng.standard_normal((m, k)).astype(np.float32)
    one = nx.matmul_quant(fmt, a, w, m, n, k)
    nx.set_row_threads(5)
    try:
        cut = nx.matmul_quant(fmt, a, w, m, n, k)
    finally:
        nx.set_row_threads(1)
    assert np.array_equal(one.view(np.uint32), cut.view(np.uint32))


# ----------------------------------------------------------------- named fragments
def test_fragment_cache_reference_counts_by_hand():
    """kv/fragment.go:36-89 and kv/paged_cache.go:285-343 on the pool's counters, worked by hand for a 4-block
    pool of block size 4: caching adds one reference per block and keeps the blocks alive after the sequence is
    gone; a second fragment of the same name releases the first; deleting the last holder frees the blocks."""
    p = hl.GPUBlockPool(num_layers=2, num_kv_heads=1, head_dim=2, block_size=4, max_blocks=4)
    p.create_sequence(1)
    p.store_kv_slots(0, 1, 0, 6), p.store_kv_slots(1, 1, 0, 6)       # two blocks per layer: 3 and 2 (tail first)
    assert p.seqs[1].block_tables == [[3, 2], [3, 2]]
    assert p.cache_content("sys", 1) == (6, [[3, 2], [3, 2]])
    assert p.ref_counts[0] == {3: 2, 2: 2} and p.block_stats() == (8, 4, 4)
    p.delete_sequence(1)                                             # the fragment still holds them
    assert p.ref_counts[0] == {3: 1, 2: 1} and p.block_stats() == (8, 4, 0)
    assert p.cache_content("nobody", 99) is None                     # an unknown sequence caches nothing
    p.create_sequence(2)
    p.store_kv_slots(0, 2, 0, 3), p.store_kv_slots(1, 2, 0, 3)       # block 1
    p.cache_content("sys", 2)                                        # same name: blocks 3 and 2 go back to the pool
    assert p.fragment("sys") == (3, [[1], [1]])
    assert p.free_lists[0] == [0, 3, 2] and p.ref_counts[0] == {1: 2}
    p.delete_fragment("sys")
    p.delete_sequence(2)
    assert p.free_lists[0] == [0, 3, 2, 1] and p.ref_counts == [{}, {}] and p.fragment("sys") is None


def test_fragment_inserted_at_p_holds_the_keys_of_positions_p_onward():
    """What the shift has to achieve, checked without the shift code: in layer 0 a token's K before RoPE depends on
    the token alone, so a fragment of tokens F cached from positions 0..n-1 and inserted at position p must leave,
    in layer 0, the K rows that a prefill of the same tokens at positions p..p+n-1 computes (to the half-precision
    rounding of rotating an already rounded row), and V rows that are bit-identical."""
    from oracle import model as om
    cfg = om.ModelConfig(num_layers=2, hidden=128, num_heads=4, num_kv_heads=2, head_dim=32, ffn=256, vocab=200)
    m = om.random_model(cfg, 17, nx.FMT_Q8_0, nx.FMT_Q8_0, max_blocks=24)
    rng = np.random.default_rng(18)
    frag, head = rng.integers(0, 200, 21).tolist(), rng.integers(0, 200, 11).tolist()
    m.pool.create_sequence(1)
    m.prefill_with_paged_kv(frag, 1, 0)
    m.pool.cache_content("doc", 1)
    m.pool.delete_sequence(1)
    m.pool.create_sequence(2)
    m.prefill_with_paged_kv(head, 2, 0)
    assert m.insert_fragment(2, "doc", 11) == 21 and m.pool.seqs[2].seq_len == 32
    assert m.insert_fragment(2, "no such name", 32) == 0
    m.pool.create_sequence(3)                                        # the same 32 tokens computed in place
    m.prefill_with_paged_kv(head + frag, 3, 0)
    row, bs = cfg.num_kv_heads * cfg.head_dim, cfg.block_size
    blk = 2 * bs * row

    def rows(seq, pos, v):
        bt = m.pool.seqs[seq].block_tables[0]
        o = bt[pos // bs] * blk + (bs * row if v else 0) + (pos % bs) * row
        return nx.f16_to_f32_array(m.kv[0][o:o + row])
    for pos in range(11, 32):
        assert np.array_equal(rows(2, pos, True), rows(3, pos, True))                 # V: position-free in layer 0
        k_ins, k_ref = rows(2, pos, False), rows(3, pos, False)
        assert np.abs(k_ins - k_ref).max() <= 2.5e-3 * np.abs(k_ref).max() + 1e-4    # two half-precision roundings
    # the rotation really happened: the unshifted rows are far from the reference
    m.pool.create_sequence(4)
    m.prefill_with_paged_kv(frag, 4, 0)
    far = max(np.abs(rows(4, t, False) - rows(3, 11 + t, False)).max() for t in range(21))
    assert far > 0.1 * max(np.abs(rows(3, 11 + t, False)).max() for t in range(21))
