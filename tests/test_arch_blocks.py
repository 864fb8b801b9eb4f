"""The oracle's layer for the architectures beside LLaMA (runtime/block.go:763-1081 with NormType, MLPType, HasBias,
ParallelResidual, RoPEDim / RoPENeox, post-norms, the soft-capped first chunk, the embedding scale) against a float64
model written here from the architectures' definitions: Phi-2 (LayerNorm, biases, partial NeoX RoPE, GELU MLP,
parallel residual), Gemma 2 (scaled embeddings, GeGLU, post-norms, soft-capped attention) and Qwen 2 (LLaMA with
Q/K/V biases and NeoX RoPE). The reference's own block tests for these (runtime/phi2_block_test.go,
multimodel_test.go) check shapes and finiteness only, so the wiring is pinned by this independent evaluation."""
import math

import numpy as np
import pytest

from oracle import model as om
from oracle import numerics as nx

BASE = dict(num_layers=2, hidden=256, num_heads=4, num_kv_heads=2, head_dim=64, ffn=512, vocab=300)
PHI = om.ModelConfig(**BASE, norm_type="layer", mlp_type="gelu", parallel_residual=True, rope_dim=32, rope_neox=True)
GEMMA = om.ModelConfig(**BASE, mlp_type="geglu", post_norms=True, attn_softcap=5.0, rope_neox=True,
                       embedding_scale=float(np.float32(math.sqrt(256.0))), eps=1e-6)
QWEN = om.ModelConfig(**BASE, rope_neox=True, rope_theta=1000000.0)
LLAMA = om.ModelConfig(**BASE)          # the plain layer: RMSNorm, SwiGLU, no biases, interleaved RoPE pairs (2j, 2j+1)
ARCHS = {"phi": PHI, "gemma": GEMMA, "qwen": QWEN, "llama": LLAMA}


def make(name, seed=11):
    cfg = ARCHS[name]
    m = om.random_model(cfg, seed, nx.FMT_Q4_0, nx.FMT_Q8_0, max_blocks=16)
    if name == "qwen":                                  # biases on Q/K/V only (the tensors a Qwen 2 file holds)
        rng = np.random.default_rng(seed + 1)
        for lw in m.layers:
            lw.wq_bias = (0.05 * rng.standard_normal(256)).astype(np.float32)
            lw.wk_bias = (0.05 * rng.standard_normal(128)).astype(np.float32)
            lw.wv_bias = (0.05 * rng.standard_normal(128)).astype(np.float32)
    return m


# ---------------------------------------------------------------- the float64 model
def _w(q):
    return nx.dequantize(q.fmt, q.data, q.n * q.k).reshape(q.n, q.k).astype(np.float64)


def _rms(x, w, eps):
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps) * w


def _ln(x, w, b, eps):
    mu = x.mean(axis=-1, keepdims=True)
    return (x - mu) / np.sqrt(((x - mu) ** 2).mean(axis=-1, keepdims=True) + eps) * w + b


def _gelu(x):
    return 0.5 * x * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x ** 3)))


def _rope(x, positions, rope_dim, theta, neox):
    """x [T, heads, D]; the first rope_dim dimensions turn, in pairs (j, j + rope_dim/2) or (2j, 2j+1)."""
    out = x.copy()
    half = rope_dim // 2
    for j in range(half):
        i0, i1 = (j, j + half) if neox else (2 * j, 2 * j + 1)
        ang = np.asarray(positions, dtype=np.float64) * theta ** (-2.0 * j / rope_dim)
        c, s = np.cos(ang)[:, None], np.sin(ang)[:, None]
        out[:, :, i0] = x[:, :, i0] * c - x[:, :, i1] * s
        out[:, :, i1] = x[:, :, i0] * s + x[:, :, i1] * c
    return out


class Float64Model:
    def __init__(self, m, drop=None):
        self.m, self.c, self.drop = m, m.cfg, drop
        self.k = [np.zeros((0, m.cfg.num_kv_heads, m.cfg.head_dim)) for _ in m.layers]
        self.v = [np.zeros((0, m.cfg.num_kv_heads, m.cfg.head_dim)) for _ in m.layers]

    def _b(self, lw, name):
        b = getattr(lw, name)
        return 0.0 if b is None or self.drop == name else b.astype(np.float64)

    def _norm(self, x, w, b):
        if self.c.norm_type == "layer":
            return _ln(x, w.astype(np.float64), 0.0 if b is None else b.astype(np.float64), self.c.eps)
        return _rms(x, w.astype(np.float64), self.c.eps)

    def forward(self, tokens, start):
        c = self.c
        t = len(tokens)
        x = self.m.embedding[np.asarray(tokens)].astype(np.float64)
        if c.embedding_scale > 0:
            x = x * c.embedding_scale
        pos = np.arange(start, start + t)
        g = c.num_heads // c.num_kv_heads
        for li, lw in enumerate(self.m.layers):
            h = self._norm(x, lw.attn_norm, lw.attn_norm_bias)
            q = (h @ _w(lw.wq).T + self._b(lw, "wq_bias")).reshape(t, c.num_heads, c.head_dim)
            k = (h @ _w(lw.wk).T + self._b(lw, "wk_bias")).reshape(t, c.num_kv_heads, c.head_dim)
            v = (h @ _w(lw.wv).T + self._b(lw, "wv_bias")).reshape(t, c.num_kv_heads, c.head_dim)
            rd = c.rope_dim or c.head_dim
            q, k = _rope(q, pos, rd, c.rope_theta, c.rope_neox), _rope(k, pos, rd, c.rope_theta, c.rope_neox)
            # the pool keeps half precision; the first chunk attends to its own unrounded K/V (block.go:875-895)
            k16, v16 = k.astype(np.float16).astype(np.float64), v.astype(np.float16).astype(np.float64)
            self.k[li], self.v[li] = np.concatenate([self.k[li], k16]), np.concatenate([self.v[li], v16])
            keys, vals = (k, v) if start == 0 else (self.k[li], self.v[li])
            cap = c.attn_softcap if (start == 0 and t > 1) else 0.0          # only that arm is soft-capped
            attn = np.zeros((t, c.num_heads, c.head_dim))
            for i in range(t):
                n = start + i + 1
                for hd in range(c.num_heads):
                    s = keys[:n, hd // g] @ q[i, hd] / math.sqrt(c.head_dim)
                    if cap > 0:
                        s = cap * np.tanh(s / cap)
                    w = np.exp(s - s.max())
                    attn[i, hd] = (w / w.sum()) @ vals[:n, hd // g]
            o = attn.reshape(t, -1) @ _w(lw.wo).T + self._b(lw, "wo_bias")
            if c.post_norms:
                o = _rms(o, lw.post_attn_norm.astype(np.float64), c.eps)
            if not c.parallel_residual:
                x = x + o
                h = self._norm(x, lw.ffn_norm, lw.ffn_norm_bias)
            if c.mlp_type == "gelu":
                d = _gelu(h @ _w(lw.w1).T + self._b(lw, "w1_bias")) @ _w(lw.w2).T + self._b(lw, "w2_bias")
            else:
                act = _gelu if c.mlp_type == "geglu" else (lambda z: z / (1.0 + np.exp(-z)))
                d = (act(h @ _w(lw.w1).T) * (h @ _w(lw.w3).T)) @ _w(lw.w2).T
            if c.post_norms:
                d = _rms(d, lw.post_ffn_norm.astype(np.float64), c.eps)
            x = x + o + d if c.parallel_residual else x + d
        last = self._norm(x[-1:], self.m.final_norm, self.m.final_norm_bias)
        return (last @ _w(self.m.lm_head).T)[0]


# ---------------------------------------------------------------- checks
@pytest.mark.parametrize("name", ["phi", "gemma", "qwen", "llama"])
def test_oracle_block_matches_float64_model(name):
    m = make(name)
    ref = Float64Model(m)
    rng = np.random.default_rng(12)
    prompt = rng.integers(0, 300, 19).tolist()
    got = m.prefill_with_paged_kv(prompt, 3, 0)
    want = ref.forward(prompt, 0)
    spread = float(np.abs(want).max())
    assert np.abs(got - want).max() <= 2e-4 * spread, "prefill"
    for step in range(3):                                   # decode: the f16 pool, no soft cap
        tok = int(np.argmax(got))
        assert tok == int(np.argmax(want))
        got = m.decode_with_paged_kv(tok, 3, 19 + step)
        want = ref.forward([tok], 19 + step)
        assert np.abs(got - want).max() <= 5e-4 * spread, "decode step %d" % step
    # a second chunk (multi-query arm over the pool)
    more = rng.integers(0, 300, 5).tolist()
    got = m.prefill_with_paged_kv(more, 3, 22)
    want = ref.forward(more, 22)
    assert np.abs(got - want).max() <= 5e-4 * spread, "second chunk"


@pytest.mark.parametrize("name,drop", [("phi", "wo_bias"), ("phi", "w2_bias"), ("phi", "wv_bias"), ("qwen", "wq_bias")])
def test_the_comparison_sees_a_dropped_bias(name, drop):
    m = make(name)
    prompt = np.random.default_rng(12).integers(0, 300, 19).tolist()
    got = m.prefill_with_paged_kv(prompt, 3, 0)
    want = Float64Model(m, drop=drop).forward(prompt, 0)
    assert np.abs(got - want).max() > 5e-3 * float(np.abs(want).max())


def test_the_comparison_sees_the_rope_pairing_of_the_llama_layer():
    """The float64 model with split pairs (j, j + D/2) in place of LLaMA's interleaved (2j, 2j+1) is a different
    function: the llama case above would not pass with the wrong pairing on either side."""
    import dataclasses
    m = make("llama")
    prompt = np.random.default_rng(12).integers(0, 300, 19).tolist()
    got = m.prefill_with_paged_kv(prompt, 3, 0)
    wrong = Float64Model(m)
    wrong.c = dataclasses.replace(m.cfg, rope_neox=True) if dataclasses.is_dataclass(m.cfg) else m.cfg
    if not dataclasses.is_dataclass(m.cfg):
        import copy
        wrong.c = copy.copy(m.cfg)
        wrong.c.rope_neox = True
    want = wrong.forward(prompt, 0)
    assert np.abs(got - want).max() > 5e-3 * float(np.abs(want).max())


def test_switches_at_their_defaults_are_the_llama_layer():
    """rope_dim = head_dim, absent biases and absent post-norm tensors change nothing, bit for bit."""
    cfg = om.ModelConfig(**BASE)
    a = om.random_model(cfg, 5, nx.FMT_Q4_0, nx.FMT_Q8_0, max_blocks=16)
    b = om.random_model(om.ModelConfig(**BASE, rope_dim=64, post_norms=True), 5, nx.FMT_Q4_0, nx.FMT_Q8_0, max_blocks=16)
    for la, lb in zip(a.layers, b.layers):                  # same matrices; unit norm weights as in `a`
        lb.attn_norm, lb.ffn_norm, lb.post_attn_norm, lb.post_ffn_norm = la.attn_norm, la.ffn_norm, None, None
    b.final_norm = a.final_norm
    prompt = list(range(40, 61))
    la, lb = a.prefill_with_paged_kv(prompt, 1, 0), b.prefill_with_paged_kv(prompt, 1, 0)
    assert np.array_equal(la.view(np.uint32), lb.view(np.uint32))
    da, db = a.decode_with_paged_kv(7, 1, 21), b.decode_with_paged_kv(7, 1, 21)
    assert np.array_equal(da.view(np.uint32), db.view(np.uint32))
