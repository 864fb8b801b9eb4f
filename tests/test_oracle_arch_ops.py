"""The oracle's restatement of the reference's optional backend interfaces (backend.go:205-263: LayerNorm, GELU /
GELUMul, AddBias, ScaleBuffer, soft-capped SDPA, RoPE with given frequencies) against the vectors of the
reference's own tests (each cited) and against float64 closed forms written from the definitions, not from the
oracle's code."""
import math

import numpy as np
import pytest

from oracle import numerics as nx


# ---- backend/cpu/layernorm_test.go:10-58 and backend/metal/phi2_ops_test.go:10-55
def test_layernorm_kats():
    x = np.array([[1, 2, 3, 4], [-1, 0, 1, 2]], dtype=np.float32)
    got = nx.layernorm(x, np.ones(4), [0.1, 0.2, 0.3, 0.4], 2, 4, 1e-5)
    want0 = np.float32((1.0 - 2.5) / math.sqrt(1.25 + 1e-5) * 1.0 + 0.1)
    assert abs(got[0, 0] - want0) <= 1e-5 and abs(got[1, 0] - want0) <= 1e-5
    plain = nx.layernorm(x, np.ones(4), np.zeros(4), 2, 4, 1e-5)
    assert abs(plain[0, 0] - np.float32((1.0 - 2.5) / math.sqrt(1.25 + 1e-5))) <= 1e-6
    # both rows have the same spread about their mean
    assert np.array_equal(plain[0], plain[1])


def test_layernorm_against_float64_definition():
    rng = np.random.default_rng(31)
    rows, cols = 5, 320
    x = (rng.standard_normal((rows, cols)) * 3 + 1.5).astype(np.float32)
    w = rng.standard_normal(cols).astype(np.float32)
    b = rng.standard_normal(cols).astype(np.float32)
    got = nx.layernorm(x, w, b, rows, cols, 1e-5)
    x64 = x.astype(np.float64)
    mean = x64.mean(axis=1, keepdims=True)
    var = ((x64 - mean) ** 2).mean(axis=1, keepdims=True)          # the biased variance, divisor cols
    want = (x64 - mean) / np.sqrt(var + 1e-5) * w + b
    assert np.max(np.abs(got - want)) <= 2e-5
    # invariants of the definition: a shift of the row changes nothing; weight 0 leaves the bias
    shifted = nx.layernorm(x + np.float32(8.0), w, b, rows, cols, 1e-5)
    assert np.max(np.abs(shifted - got)) <= 5e-5
    assert np.array_equal(nx.layernorm(x, np.zeros(cols), b, rows, cols, 1e-5), np.broadcast_to(b, (rows, cols)))
    # a constant row: every element is the mean, the output is the bias whatever eps is
    const = nx.layernorm(np.full((1, 64), 3.25, dtype=np.float32), w[:64], b[:64], 1, 64, 1e-5)
    assert np.array_equal(const[0], b[:64])


# ---- backend/cpu/gelu_test.go:10-39, backend/metal/phi2_ops_test.go:57-88
def test_gelu_kats():
    got = nx.gelu([-2.0, -1.0, 0.0, 1.0, 2.0])
    assert got[2] == 0.0
    assert 1.9 < got[4] < 2.0 and abs(got[4] - 1.9546) < 1e-3
    assert abs(got[3] - 0.8413) < 1e-3                              # gelu_test.go:33 "GELU(1) ≈ 0.8413"


def test_gelu_against_float64_tanh_form():
    x = np.concatenate([np.linspace(-9, 9, 2001), [0.0, -0.0, 1e-20, 40.0, -40.0]]).astype(np.float32)
    got = nx.gelu(x)
    x64 = x.astype(np.float64)
    want = 0.5 * x64 * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (x64 + 0.044715 * x64 ** 3)))
    assert np.max(np.abs(got - want)) <= 2e-6 * np.maximum(1.0, np.abs(want)).max()
    # large arguments saturate: x and -0 (tanh rounds to +-1 in float32)
    assert got[-2] == np.float32(40.0) and got[-1] == 0.0
    # gelu(x) - gelu(-x) = x for the tanh form (tanh is odd)
    assert np.max(np.abs((nx.gelu(x) - nx.gelu(-x)) - x)) <= 2e-6 * 40


# ---- backend/metal/geglu_test.go:30-144: gelu(gate) * up, zero gates, zero ups
def test_gelu_mul_is_gelu_times_up():
    rng = np.random.default_rng(32)
    g = (rng.standard_normal(4099) * 2).astype(np.float32)
    u = rng.standard_normal(4099).astype(np.float32)
    got = nx.gelu_mul(g, u)
    assert np.array_equal(got.view(np.uint32), (nx.gelu(g) * u).view(np.uint32))
    assert np.all(nx.gelu_mul(np.zeros(8), u[:8]) == 0.0)
    assert np.all(nx.gelu_mul(g[:8], np.zeros(8)) == 0.0)
    assert np.array_equal(nx.gelu_mul(g, np.ones_like(g)), nx.gelu(g))


# ---- backend/cpu/bias_test.go:9-42, backend/metal/phi2_ops_test.go:143-
def test_add_bias_kat():
    got = nx.add_bias([[1, 2, 3], [4, 5, 6]], [0.1, 0.2, 0.3], 2, 3)
    want = np.array([[1.1, 2.2, 3.3], [4.1, 5.2, 6.3]], dtype=np.float32)
    assert np.max(np.abs(got - want)) <= 1e-5
    rng = np.random.default_rng(33)
    x, b = rng.standard_normal((7, 33)).astype(np.float32), rng.standard_normal(33).astype(np.float32)
    assert np.array_equal(nx.add_bias(x, b, 7, 33), x + b[None, :])


def test_scale_buffer():
    rng = np.random.default_rng(34)
    x = rng.standard_normal(1000).astype(np.float32)
    s = np.float32(math.sqrt(2304.0))                               # Gemma: embeddings times sqrt(hidden)
    assert np.array_equal(nx.scale_buffer(x, s), x * s)
    assert np.array_equal(nx.scale_buffer(x, 1.0), x)


# ---- backend/metal/softcap_sdpa_test.go:149-217 (softcap_bounds_scores)
def test_sdpa_softcap_kat():
    q = [1.0, 0, 0, 0]
    k = np.zeros((4, 4), dtype=np.float32)
    k[0, 0] = 10.0
    v = np.eye(4, dtype=np.float32)
    got = nx.sdpa_softcap(q, k, v, 4, 1, 1, 4, 1.0, 5.0, 16)[0]
    s0 = 5.0 * math.tanh(10.0 / 5.0)                                # ≈ 4.82, the other scores are 0
    w0 = math.exp(s0) / (math.exp(s0) + 3.0)
    assert abs(w0 - 0.976) < 1e-3                                   # the test's comment, :210
    assert np.max(np.abs(got - np.array([w0, (1 - w0) / 3, (1 - w0) / 3, (1 - w0) / 3]))) <= 1e-6
    assert got[0] < 0.999
    plain = nx.sdpa(q, k, v, 4, 1, 1, 4, 1.0, 16)[0]
    assert plain[0] > 0.9998                                        # "softmax ≈ 0.9999" without the cap, :209


# ---- softcap_sdpa_test.go:85-141: softcap 0 is plain SDPA; and the prefill form likewise
def test_softcap_zero_is_plain_attention_bit_for_bit():
    rng = np.random.default_rng(35)
    hq, hk, d, n = 8, 4, 64, 37
    q = rng.standard_normal((hq, d)).astype(np.float32)
    k = rng.standard_normal((hk, n, d)).astype(np.float32)
    v = rng.standard_normal((hk, n, d)).astype(np.float32)
    sc = np.float32(1 / math.sqrt(d))
    a = nx.sdpa_softcap(q, k, v, n, hq, hk, d, sc, 0.0, n * d)
    assert np.array_equal(a.view(np.uint32), nx.sdpa(q, k, v, n, hq, hk, d, sc, n * d).view(np.uint32))
    qs = rng.standard_normal((9, hq, d)).astype(np.float32)
    ks = rng.standard_normal((9, hk, d)).astype(np.float32)
    vs = rng.standard_normal((9, hk, d)).astype(np.float32)
    b = nx.sdpa_prefill_softcap(qs, ks, vs, 9, hq, hk, d, sc, 0.0)
    assert np.array_equal(b.view(np.uint32), nx.sdpa_prefill(qs, ks, vs, 9, hq, hk, d, sc).view(np.uint32))


def _attention64(q, keys, vals, scale, cap):
    """softmax(cap * tanh(q.k * scale / cap)) . v in float64, from the definition (backend.go:229-231)."""
    s = keys.astype(np.float64) @ q.astype(np.float64) * float(scale)
    if cap > 0:
        s = cap * np.tanh(s / cap)
    w = np.exp(s - s.max())
    w /= w.sum()
    return w @ vals.astype(np.float64)


# ---- softcap_sdpa_test.go:219-283 (Gemma 2 geometry: 8/4 heads of 256, softcap 30) and :286-478 (prefill, 50)
def test_softcap_against_float64_definition():
    rng = np.random.default_rng(36)
    hq, hk, d, n = 8, 4, 256, 64
    q = (rng.standard_normal((hq, d)) * 3).astype(np.float32)      # scores well into the cap's curved part
    k = (rng.standard_normal((hk, n, d)) * 3).astype(np.float32)
    v = rng.standard_normal((hk, n, d)).astype(np.float32)
    sc = np.float32(1 / math.sqrt(d))
    got = nx.sdpa_softcap(q, k, v, n, hq, hk, d, sc, 30.0, n * d)
    capped = False
    for h in range(hq):
        want = _attention64(q[h], k[h // 2], v[h // 2], sc, 30.0)
        assert np.max(np.abs(got[h] - want)) <= 2e-5
        capped |= bool(np.max(np.abs(got[h] - _attention64(q[h], k[h // 2], v[h // 2], sc, 0.0))) > 1e-3)
    assert capped                                                   # the cap mattered for these inputs
    s, hq, hk, d = 12, 4, 2, 32
    qs = (rng.standard_normal((s, hq, d)) * 4).astype(np.float32)
    ks = (rng.standard_normal((s, hk, d)) * 4).astype(np.float32)
    vs = rng.standard_normal((s, hk, d)).astype(np.float32)
    sc = np.float32(1 / math.sqrt(d))
    got = nx.sdpa_prefill_softcap(qs, ks, vs, s, hq, hk, d, sc, 50.0)
    for t in range(s):
        for h in range(hq):
            want = _attention64(qs[t, h], ks[:t + 1, h // 2], vs[:t + 1, h // 2], sc, 50.0)
            assert np.max(np.abs(got[t, h] - want)) <= 2e-5
    # the first token attends to itself alone: its output is its own V row whatever the cap
    assert np.array_equal(got[0], np.repeat(vs[0], hq // hk, axis=0))


# ---- backend/metal/scaled_rope_test.go:47-  (theta_equivalence, custom_freqs)
@pytest.mark.parametrize("neox", [False, True])
def test_rope_with_freqs_equals_rope_for_theta_frequencies(neox):
    rng = np.random.default_rng(37)
    d, hq, hk, s, start, theta = 128, 8, 4, 3, 5, 10000.0
    q = rng.standard_normal((s, hq, d)).astype(np.float32)
    k = rng.standard_normal((s, hk, d)).astype(np.float32)
    freqs = np.array([np.float32(1.0 / math.pow(theta, (2 * j) / d)) for j in range(d // 2)], dtype=np.float32)
    q1, k1 = nx.rope(q, k, d, hq, hk, s, start, 0, theta, neox)
    q2, k2 = nx.rope_with_freqs(q, k, freqs, d, hq, hk, s, start, neox)
    assert np.array_equal(q1.view(np.uint32), q2.view(np.uint32))
    assert np.array_equal(k1.view(np.uint32), k2.view(np.uint32))
    q3, none = nx.rope_with_freqs(q, None, freqs, d, hq, hk, s, start, neox)
    assert none is None and np.array_equal(q3, q2)


@pytest.mark.parametrize("neox", [False, True])
def test_rope_with_custom_freqs_closed_form(neox):
    d, heads, s, start = 64, 2, 3, 10
    freqs = (0.01 * np.arange(1, d // 2 + 1)).astype(np.float32)   # scaled_rope_test.go:134-138
    rng = np.random.default_rng(38)
    q = rng.standard_normal((s, heads, d)).astype(np.float32)
    got, _ = nx.rope_with_freqs(q, None, freqs, d, heads, heads, s, start, neox)
    for t in range(s):
        for j in range(d // 2):
            i0, i1 = (j, j + d // 2) if neox else (2 * j, 2 * j + 1)
            ang = float(np.float32(start + t) * freqs[j])
            z = (q[t, :, i0].astype(np.float64) + 1j * q[t, :, i1].astype(np.float64)) * complex(math.cos(ang), math.sin(ang))
            assert np.max(np.abs(got[t, :, i0] - z.real)) <= 1e-6 and np.max(np.abs(got[t, :, i1] - z.imag)) <= 1e-6
    # position 0: no rotation
    same, _ = nx.rope_with_freqs(q[:1], None, freqs, d, heads, heads, 1, 0, neox)
    assert np.array_equal(same, q[:1])


# ---- inference/medusa/medusa_test.go:250-318 (SiLU values, the forward pass spelled out) and heads.go:146-171
def test_medusa_forward_and_topk():
    from oracle import host_logic as hl
    rng = np.random.default_rng(39)
    h, v = 64, 100                                                  # medusa_test.go:12-14
    hidden = (rng.random(h) * 2 - 1).astype(np.float32)
    fc1 = ((rng.random((h, h)) * 2 - 1) * math.sqrt(2.0 / h)).astype(np.float32)   # heads.go:60-75
    fc2 = ((rng.random((h, v)) * 2 - 1) * math.sqrt(2.0 / h)).astype(np.float32)
    inter, logits = nx.medusa_forward(hidden, fc1, fc2)
    pre = hidden.astype(np.float64) @ fc1.astype(np.float64)
    want_inter = pre / (1.0 + np.exp(-pre))
    assert np.max(np.abs(inter - want_inter)) <= 2e-6
    assert np.max(np.abs(logits - want_inter @ fc2.astype(np.float64))) <= 5e-6
    # medusa_test.go:297-317: silu(-1) ≈ -0.2689, silu(0) = 0, silu(1) ≈ 0.7311, through a one-column identity FC1
    eye = np.eye(4, dtype=np.float32)
    got, _ = nx.medusa_forward([-1.0, 0.0, 1.0, -2.0], eye, eye)
    assert abs(got[0] + 0.2689) < 1e-4 and got[1] == 0.0 and abs(got[2] - 0.7311) < 1e-4 and abs(got[3] + 0.2384) < 1e-4
    # a transposed FC1 would be a different product
    t_inter, _ = nx.medusa_forward(hidden, fc1.T.copy(), fc2)
    assert np.max(np.abs(t_inter - inter)) > 1e-2
    # top-k: largest first, the first of equal values, -1 when nothing is above -MaxFloat32
    assert hl.medusa_top_k([0.5, 2.0, 2.0, -1.0, 3.0], 4) == [4, 1, 2, 0]
    assert hl.medusa_top_k([float("-inf"), 1.0], 2) == [1, -1]
    assert hl.medusa_top_k([1.0, float("nan"), 2.0], 3) == [2, 0, -1]
    top = hl.medusa_top_k(logits.tolist(), 5)
    assert top == np.argsort(-logits.astype(np.float64), kind="stable")[:5].tolist()


# ---- runtime/model.go:336-350 (ApplyFinalLogitSoftCap)
def test_logit_softcap_closed_form():
    x = np.concatenate([np.linspace(-200, 200, 4001), [0.0, 1e-8, 1e30, -1e30]]).astype(np.float32)
    got = nx.logit_softcap(x, 30.0)
    want = 30.0 * np.tanh(x.astype(np.float64) / 30.0)
    assert np.max(np.abs(got - want)) <= 2e-6
    assert np.all(np.abs(got) <= 30.0) and got[-2] == 30.0 and got[-1] == -30.0
    assert np.all(np.diff(got[:4001]) >= 0)                        # monotone: the greedy choice is unchanged
    assert np.max(np.abs(got[1900:2101] - x[1900:2101])) < 0.4     # near 0 it is almost the identity
    assert np.array_equal(nx.logit_softcap(x, 0.0), x)             # disabled
