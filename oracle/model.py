"""The reference's layer and decode drivers, chained from the oracle kernels
(TEST INFRASTRUCTURE ONLY).

  OracleModel.execute_with_paged_kv  inference/runtime/block.go:763-1081 (every arm: RMSNorm / LayerNorm, SwiGLU /
                                     GELU / GeGLU, serial / parallel residual, biases, partial and NeoX RoPE,
                                     post-norms, the soft-capped first prefill chunk)
  OracleModel.decode_with_paged_kv   inference/runtime/decode.go:339-461
  OracleModel.decode_batched         inference/runtime/decode.go:612-654 (sequential loop)
  OracleModel.prefill_with_paged_kv  inference/runtime/decode.go:961-1096
  OracleModel.verify_tree/tree_step  whole-tree form of scheduler/medusa_scheduler.go:733-861 (the reference
                                     verifies one path; pinned by equality with verify_with_paged_kv on every
                                     root-to-node path)
The KV pool holds real data here (numpy uint16 = f16 bits, or float32), addressed as
inference/runtime/gpu_block_pool.go:15-19,107-108.
"""
import math
from dataclasses import dataclass
from typing import List, Optional

import numpy as np

from . import numerics as nx
from .host_logic import GPUBlockPool


@dataclass
class ModelConfig:
    num_layers: int
    hidden: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    ffn: int
    vocab: int
    eps: float = 1e-5
    rope_theta: float = 10000.0
    block_size: int = 16  # inference/runtime/model.go:321
    # the architecture switches of runtime/config.go:14-62,120-131 and block.go:245-254,339-340; the defaults are LLaMA
    norm_type: str = "rms"            # "rms" | "layer" (NormType)
    mlp_type: str = "swiglu"          # "swiglu" | "gelu" | "geglu" (MLPType)
    parallel_residual: bool = False   # x + attn(norm(x)) + mlp(norm(x))
    rope_dim: int = 0                 # rotated dimensions, 0 = the whole head
    rope_neox: bool = False           # pairs (j, j + half) instead of (2j, 2j+1)
    attn_softcap: float = 0.0         # AttentionLogitSoftCap
    post_norms: bool = False          # HasPostNorms
    embedding_scale: float = 0.0      # EmbeddingScale, <= 0 = none (decode.go:197-205)
    final_softcap: float = 0.0        # FinalLogitSoftCap: on the logits a request is sampled from (scheduler.go:772-773)


@dataclass
class QWeight:
    fmt: int          # numerics.FMT_*
    data: np.ndarray  # uint8 [N, row_bytes]
    n: int
    k: int


@dataclass
class LayerWeights:
    attn_norm: np.ndarray
    wq: QWeight
    wk: QWeight
    wv: QWeight
    wo: QWeight
    ffn_norm: np.ndarray
    w1: QWeight
    w3: Optional[QWeight]                     # unused by the GELU MLP (block.go:265)
    w2: QWeight
    # block.go:266-283: LayerNorm biases, projection biases, Gemma 2's post-norms; None = the tensor is absent
    attn_norm_bias: Optional[np.ndarray] = None
    ffn_norm_bias: Optional[np.ndarray] = None
    wq_bias: Optional[np.ndarray] = None
    wk_bias: Optional[np.ndarray] = None
    wv_bias: Optional[np.ndarray] = None
    wo_bias: Optional[np.ndarray] = None
    w1_bias: Optional[np.ndarray] = None
    w2_bias: Optional[np.ndarray] = None
    post_attn_norm: Optional[np.ndarray] = None
    post_ffn_norm: Optional[np.ndarray] = None


def _mm(a, w: QWeight, m):
    # block.go:506-552 matMulTransposed dispatch on the quant profile; fmt 0 = a float32 [n,k] matrix
    # (a dequantized or tied output head, model.go:394-404 -> Backend.MatMulTransposed)
    if w.fmt == 0:
        return nx.matmul_t_f32(a, w.data, m, w.n, w.k)
    return nx.matmul_quant(w.fmt, a, w.data, m, w.n, w.k)


def _mm_bias(a, w: QWeight, bias, m):
    """block.go:555-560 (matMulTransposedWithBias): the product, then AddBias when the bias tensor exists."""
    out = _mm(a, w, m)
    return out if bias is None else nx.add_bias(out, bias, m, w.n)


class OracleModel:
    def __init__(self, cfg: ModelConfig, embedding_f32, layers: List[LayerWeights], final_norm,
                 lm_head: QWeight, max_blocks, kv_fp16=True, final_norm_bias=None):
        self.cfg = cfg
        # block.go:972-976 keeps the attention output in the buffer the gated MLPs write W3's product to: the
        # parallel residual exists for the GELU MLP only
        assert not cfg.parallel_residual or cfg.mlp_type == "gelu"
        self.final_norm_bias = final_norm_bias
        self.embedding = np.ascontiguousarray(embedding_f32, dtype=np.float32)
        self.layers = layers
        self.final_norm = final_norm
        self.lm_head = lm_head
        self.pool = GPUBlockPool(cfg.num_layers, cfg.num_kv_heads, cfg.head_dim, cfg.block_size,
                                 max_blocks, use_fp16=kv_fp16)
        elems = max_blocks * 2 * cfg.block_size * cfg.num_kv_heads * cfg.head_dim
        dt = np.uint16 if kv_fp16 else np.float32
        self.kv = [np.zeros(elems, dtype=dt) for _ in range(cfg.num_layers)]

    # ---------------------------------------------------------------- one layer
    def _norm(self, x, weight, bias, rows):
        """block.go:562-576 (applyNorm): LayerNorm with its bias, or RMSNorm, which ignores the bias."""
        c = self.cfg
        if c.norm_type == "layer":
            b = bias if bias is not None else np.zeros(c.hidden, dtype=np.float32)
            return nx.layernorm(x, weight, b, rows, c.hidden, c.eps)
        return nx.rmsnorm(x, weight, rows, c.hidden, c.eps)

    def _mlp(self, norm, lw, seq_len):
        """block.go:1001-1063: the GELU MLP with biases, or the gated one (SiLU or GELU gate) without."""
        c = self.cfg
        if c.mlp_type == "gelu":
            gate = nx.gelu(_mm_bias(norm, lw.w1, lw.w1_bias, seq_len))         # :1010-1021
            return _mm_bias(gate, lw.w2, lw.w2_bias, seq_len)                  # :1036
        gate = _mm(norm, lw.w1, seq_len)                                       # :1043-1050
        up = _mm(norm, lw.w3, seq_len)
        act = nx.gelu_mul(gate, up) if c.mlp_type == "geglu" else nx.silu_mul(gate, up)  # :1051-1056
        return _mm(act, lw.w2, seq_len)                                        # :1058-1061

    def execute_with_paged_kv(self, x, seq_id, layer_idx, start_pos):
        """x [seqLen, hidden] float32, updated copy returned. block.go:763-1081."""
        c = self.cfg
        lw = self.layers[layer_idx]
        seq_len = x.shape[0]
        norm = self._norm(x, lw.attn_norm, lw.attn_norm_bias, seq_len)         # :834-837
        q = _mm_bias(norm, lw.wq, lw.wq_bias, seq_len)                         # :841-854
        k = _mm_bias(norm, lw.wk, lw.wk_bias, seq_len)
        v = _mm_bias(norm, lw.wv, lw.wv_bias, seq_len)
        q, k = nx.rope(q, k, c.head_dim, c.num_heads, c.num_kv_heads, seq_len, start_pos, c.rope_dim,
                       c.rope_theta, c.rope_neox)                              # :858 (applyRoPE, :497-503)
        scale = np.float32(1.0 / math.sqrt(float(c.head_dim)))                 # :862
        slots = self.pool.store_kv_slots(layer_idx, seq_id, start_pos, seq_len)  # :868 / :878
        bi = [s[0] for s in slots]
        bo = [s[1] for s in slots]
        nx.reshape_paged_kv(k, self.kv[layer_idx], bi, bo, c.num_kv_heads, c.head_dim, c.block_size, False)
        nx.reshape_paged_kv(v, self.kv[layer_idx], bi, bo, c.num_kv_heads, c.head_dim, c.block_size, True)
        if seq_len == 1:                                                       # :866-874 (no soft cap on this arm)
            bt, nb, til = self.pool.attention_args(layer_idx, seq_id)
            attn = nx.sdpa_paged_decode(q, self.kv[layer_idx], bt, nb, c.block_size, c.num_heads,
                                        c.num_kv_heads, c.head_dim, scale, til).reshape(1, -1)
        elif start_pos > 0:                                                    # :881-890 (nor on this one)
            kv_lens = [start_pos + i + 1 for i in range(seq_len)]
            bt = self.pool.seqs[seq_id].block_tables[layer_idx]
            attn = nx.sdpa_paged_multiquery(q, self.kv[layer_idx], bt, kv_lens, c.block_size, c.num_heads,
                                            c.num_kv_heads, c.head_dim, scale).reshape(seq_len, -1)
        elif c.attn_softcap > 0:                                               # :891-892
            attn = nx.sdpa_prefill_softcap(q, k, v, seq_len, c.num_heads, c.num_kv_heads, c.head_dim, scale,
                                           c.attn_softcap).reshape(seq_len, -1)
        else:                                                                  # :893-895 dense causal on F32 K/V
            attn = nx.sdpa_prefill(q, k, v, seq_len, c.num_heads, c.num_kv_heads, c.head_dim,
                                   scale).reshape(seq_len, -1)
        return self._tail(x, norm, attn, lw, seq_len)

    def _tail(self, x, norm, attn, lw, seq_len):
        """block.go:981-1077: output projection, post-norm, residual(s), FFN norm, MLP. `norm` is the attention
        norm's output (what the parallel residual's MLP reads)."""
        c = self.cfg
        o = _mm_bias(attn, lw.wo, lw.wo_bias, seq_len)                         # :981-983
        if c.post_norms and lw.post_attn_norm is not None:                     # :985-987
            o = nx.rmsnorm(o, lw.post_attn_norm, seq_len, c.hidden, c.eps)
        if not c.parallel_residual:
            x = nx.add(x, o)                                                   # :989-991
            if lw.ffn_norm is not None:                                        # :996-998
                norm = self._norm(x, lw.ffn_norm, lw.ffn_norm_bias, seq_len)
        down = self._mlp(norm, lw, seq_len)                                    # :1001-1063
        if c.post_norms and lw.post_ffn_norm is not None:                      # :1066-1069
            down = nx.rmsnorm(down, lw.post_ffn_norm, seq_len, c.hidden, c.eps)
        if c.parallel_residual:                                                # :1072-1075
            x = nx.add(x, o)
        return nx.add(x, down)                                                 # :1075-1077

    def _embed(self, tokens):
        c = self.cfg
        x = nx.embedding(tokens, self.embedding, c.vocab, c.hidden)           # decode.go:405-407
        if c.embedding_scale > 0:                                              # decode.go:197-205, 408
            x = nx.scale_buffer(x, c.embedding_scale)
        return x

    # ---------------------------------------------------------------- drivers
    def _ensure_seq(self, seq_id):
        if not self.pool.has_sequence(seq_id):                                 # decode.go:361-363
            self.pool.create_sequence(seq_id)

    def _head(self, state, rows):
        c = self.cfg
        state = self._norm(state, self.final_norm, self.final_norm_bias, rows)  # model.go:207-226
        # model.go:352-422: quantized lm_head runs one M=1 call per row (same numbers)
        return _mm(state, self.lm_head, rows)

    def decode_with_paged_kv(self, token, seq_id, pos):
        """decode.go:339-461 with one token -> logits [vocab]."""
        c = self.cfg
        self._ensure_seq(seq_id)
        x = self._embed([token])
        for i in range(c.num_layers):                                          # decode.go:432-437
            x = self.execute_with_paged_kv(x, seq_id, i, pos)
        return self._head(x, 1)[0]

    def decode_batched(self, tokens, seq_ids, positions):
        """decode.go:612-654: the batch is a loop over sequences -> logits [B, vocab]."""
        assert len(tokens) == len(seq_ids) == len(positions)
        return np.stack([self.decode_with_paged_kv(t, s, p) for t, s, p in zip(tokens, seq_ids, positions)])

    def prefill_with_paged_kv(self, tokens, seq_id, start_pos):
        """decode.go:961-1096 -> logits of the last token [vocab]."""
        c = self.cfg
        self._ensure_seq(seq_id)
        n = len(tokens)
        x = self._embed(tokens)
        for i in range(c.num_layers):
            x = self.execute_with_paged_kv(x, seq_id, i, start_pos)
        last = x[n - 1:n]                                                      # decode.go:1057-1066
        return self._head(last, 1)[0]

    def verify_with_paged_kv(self, tokens, seq_id, start_pos):
        """decode.go:1446-1569: logits for every position [n, vocab]."""
        c = self.cfg
        self._ensure_seq(seq_id)
        n = len(tokens)
        x = self._embed(tokens)
        for i in range(c.num_layers):
            x = self.execute_with_paged_kv(x, seq_id, i, start_pos)
        return self._head(x, n)


    # ---------------------------------------------------------------- tree verification
    def _execute_tree_layer(self, x, seq_id, layer_idx, start_pos, positions, mask):
        """block.go:763-1081 for the rows [input token, candidate nodes]: row r is stored at pool position
        start_pos + r, rotated at positions[r] (start_pos + its depth in the tree) and attends to every earlier
        pool position and to the rows the mask names (tree.go:186-202). The architecture's switches act as in
        execute_with_paged_kv's multi-query arm (a chunk behind a context: no soft cap on the scores)."""
        c = self.cfg
        lw = self.layers[layer_idx]
        rows = x.shape[0]
        norm = self._norm(x, lw.attn_norm, lw.attn_norm_bias, rows)
        q = _mm_bias(norm, lw.wq, lw.wq_bias, rows)
        k = _mm_bias(norm, lw.wk, lw.wk_bias, rows)
        v = _mm_bias(norm, lw.wv, lw.wv_bias, rows)
        q, k = nx.rope_positions(q, k, c.head_dim, c.num_heads, c.num_kv_heads, positions, c.rope_dim, c.rope_theta,
                                 c.rope_neox)
        scale = np.float32(1.0 / math.sqrt(float(c.head_dim)))
        slots = self.pool.store_kv_slots(layer_idx, seq_id, start_pos, rows)
        bi = [s[0] for s in slots]
        bo = [s[1] for s in slots]
        nx.reshape_paged_kv(k, self.kv[layer_idx], bi, bo, c.num_kv_heads, c.head_dim, c.block_size, False)
        nx.reshape_paged_kv(v, self.kv[layer_idx], bi, bo, c.num_kv_heads, c.head_dim, c.block_size, True)
        bt = self.pool.seqs[seq_id].block_tables[layer_idx]
        attn = nx.sdpa_paged_multiquery(q, self.kv[layer_idx], bt, None, c.block_size, c.num_heads, c.num_kv_heads,
                                        c.head_dim, scale, tree_mask=mask, tree_base=start_pos).reshape(rows, -1)
        return self._tail(x, norm, attn, lw, rows)

    def verify_tree(self, input_token, node_tokens, parent_idx, seq_id, start_pos):
        """Logits [1 + nodes, vocab] of one pass over the input token and a candidate tree given as
        CandidateTree.Linearize returns it (tree.go:144-178: parent_idx -1 = child of the input token). Every
        root-to-node path sees what VerifySpeculativeWithPagedKV (decode.go:1446-1569) would show it on
        [input token, path tokens]: same positions, same visible keys. The rows' K/V stay in the pool at
        start_pos .. start_pos + nodes."""
        from .host_logic import build_tree_attention_mask, tree_depths
        c = self.cfg
        self._ensure_seq(seq_id)
        n = len(node_tokens)
        rows = n + 1
        # row 0 is the input token: every node descends from it
        parents = [-1] + [p + 1 for p in parent_idx]
        mask = np.array(build_tree_attention_mask(rows, parents), dtype=np.uint8).reshape(rows, rows)
        positions = [start_pos + d for d in tree_depths(parents)]
        x = self._embed([input_token] + list(node_tokens))
        for i in range(c.num_layers):
            x = self._execute_tree_layer(x, seq_id, i, start_pos, positions, mask)
        return self._head(x, rows)

    def insert_fragment(self, seq_id, name, insert_pos):
        """PagedKVCache.InsertFragment (kv/paged_cache.go:285-322) with the read-time RoPE shift of
        GetKVSliceForAttention (:225-283) done once, at insertion: the fragment's token rows go to positions
        insert_pos.. of the sequence, K rotated by RoPEShift(insert_pos) (backend/cpu/backend.go:244-276) and, in
        an F16 pool, rounded to half precision again; V as it is. -> tokens inserted (0 for an unknown name)."""
        c, pool = self.cfg, self.pool
        frag = pool.fragment(name)
        if frag is None:
            return 0
        if not pool.has_sequence(seq_id):
            pool.create_sequence(seq_id)
        st = pool.seqs[seq_id]
        assert insert_pos == st.seq_len, "a fragment goes to the end of the sequence"
        n, blocks = frag
        row = c.num_kv_heads * c.head_dim
        blk = 2 * c.block_size * row                                       # gpu_block_pool.go:107-108
        for layer in range(c.num_layers if n > 0 else 0):
            slots = pool.store_kv_slots(layer, seq_id, insert_pos, n)      # the blocks StoreKV would take, :234-252
            for t in range(n):
                src = blocks[layer][t // c.block_size] * blk + (t % c.block_size) * row
                dst = slots[t][0] * blk + slots[t][1] * row
                k = self.kv[layer][src:src + row]
                kf = nx.f16_to_f32_array(k) if pool.use_fp16 else k.astype(np.float32)
                kf = nx.rope_shift(kf, c.head_dim, c.num_kv_heads, 1, insert_pos, c.rope_theta).reshape(-1)
                self.kv[layer][dst:dst + row] = nx.f32_to_f16_array(kf) if pool.use_fp16 else kf
                v0, v1 = src + c.block_size * row, dst + c.block_size * row
                self.kv[layer][v1:v1 + row] = self.kv[layer][v0:v0 + row].copy()
        st.seq_len = insert_pos + n
        return n

    def _move_kv_row(self, layer, seq_id, src_pos, dst_pos):
        c = self.cfg
        bt = self.pool.seqs[seq_id].block_tables[layer]
        row = c.num_kv_heads * c.head_dim
        blk = 2 * c.block_size * row                                       # gpu_block_pool.go:107-108
        for half in (0, 1):                                                # K rows, then V rows of the block
            s = bt[src_pos // c.block_size] * blk + half * c.block_size * row + (src_pos % c.block_size) * row
            d = bt[dst_pos // c.block_size] * blk + half * c.block_size * row + (dst_pos % c.block_size) * row
            self.kv[layer][d:d + row] = self.kv[layer][s:s + row].copy()

    def tree_step(self, input_token, node_tokens, parent_idx, seq_id, start_pos):
        """verify_tree, greedy acceptance over the whole tree, then the rollback of
        medusa_scheduler.go:852-861: the accepted nodes' K/V move up to the positions right after the input
        token (a path is not contiguous in the pool) and the sequence is truncated to
        start_pos + 1 + accepted. -> (accepted node indices, final token, logits)."""
        logits = self.verify_tree(input_token, node_tokens, parent_idx, seq_id, start_pos)
        return self._accept_and_roll_back(logits, node_tokens, parent_idx, seq_id, start_pos)

    def tree_step_batched(self, input_tokens, trees, seq_ids, start_positions):
        """tree_step for several sequences whose trees are verified in the same pass: every sequence's rows
        take their blocks first (in the order given), then every sequence is rolled back (same order).
        -> [(accepted node indices, final token, logits)] per sequence."""
        logits = [self.verify_tree(t, tr[0], tr[1], sid, sp)
                  for t, tr, sid, sp in zip(input_tokens, trees, seq_ids, start_positions)]
        return [self._accept_and_roll_back(lg, tr[0], tr[1], sid, sp)
                for lg, tr, sid, sp in zip(logits, trees, seq_ids, start_positions)]

    def _accept_and_roll_back(self, logits, node_tokens, parent_idx, seq_id, start_pos):
        from .host_logic import greedy_tree_accept, argmax_list, cache_len_after_verify
        am = [argmax_list(row) for row in logits]
        accepted, final = greedy_tree_accept(list(node_tokens), list(parent_idx), am[0], am[1:])
        for layer in range(self.cfg.num_layers):
            for k, node in enumerate(accepted):                            # ascending: a source is never overwritten
                if node != k:
                    self._move_kv_row(layer, seq_id, start_pos + 1 + node, start_pos + 1 + k)
        self.pool.truncate_sequence(seq_id, cache_len_after_verify(start_pos, len(accepted)))
        return accepted, final, logits


def random_model(cfg: ModelConfig, seed, fmt, head_fmt, emb_fmt=None, max_blocks=64, kv_fp16=True,
                 fmt_overrides=None):
    """Random-init model: N(0,0.02) weights quantized to `fmt`; norm weights = 1;
    embedding table = dequantised `emb_fmt` matrix (loader rule,
    inference/runtime/loader.go:79-200,275-288). fmt_overrides maps a weight name
    (wq, wk, wv, wo, w1, w2, w3) to another format."""
    from . import quantize as qz
    rng = np.random.default_rng(seed)
    fo = fmt_overrides or {}

    def qw(name, n, k):
        f = fo.get(name, fmt)
        return QWeight(f, qz.random_quant(f, rng, n, k), n, k)

    qd = cfg.num_heads * cfg.head_dim
    kvd = cfg.num_kv_heads * cfg.head_dim
    layers = []
    for _ in range(cfg.num_layers):
        layers.append(LayerWeights(
            attn_norm=np.ones(cfg.hidden, dtype=np.float32),
            wq=qw("wq", qd, cfg.hidden), wk=qw("wk", kvd, cfg.hidden), wv=qw("wv", kvd, cfg.hidden),
            wo=qw("wo", cfg.hidden, qd),
            ffn_norm=np.ones(cfg.hidden, dtype=np.float32),
            w1=qw("w1", cfg.ffn, cfg.hidden), w3=qw("w3", cfg.ffn, cfg.hidden), w2=qw("w2", cfg.hidden, cfg.ffn)))
    ef = emb_fmt if emb_fmt is not None else head_fmt
    emb_q = qz.random_quant(ef, rng, cfg.vocab, cfg.hidden)
    emb = nx.dequantize(ef, emb_q, cfg.vocab * cfg.hidden).reshape(cfg.vocab, cfg.hidden)
    head = QWeight(head_fmt, qz.random_quant(head_fmt, rng, cfg.vocab, cfg.hidden), cfg.vocab, cfg.hidden)
    final_norm, final_bias = np.ones(cfg.hidden, dtype=np.float32), None
    if not is_llama(cfg):
        # the tensors the other architectures add, from a stream of their own (the LLaMA draws above are unchanged):
        # norm weights around 1, small biases, so that a dropped or misplaced one moves the logits visibly
        r2 = np.random.default_rng(seed + 7919)
        vec = lambda n, mean, sd: (mean + sd * r2.standard_normal(n)).astype(np.float32)
        bias = cfg.norm_type == "layer" or cfg.mlp_type == "gelu"           # HasBias models (Phi)
        for lw in layers:
            lw.attn_norm, lw.ffn_norm = vec(cfg.hidden, 1.0, 0.1), vec(cfg.hidden, 1.0, 0.1)
            if cfg.norm_type == "layer":
                lw.attn_norm_bias, lw.ffn_norm_bias = vec(cfg.hidden, 0.0, 0.05), vec(cfg.hidden, 0.0, 0.05)
            if bias:
                lw.wq_bias, lw.wk_bias, lw.wv_bias = vec(qd, 0.0, 0.05), vec(kvd, 0.0, 0.05), vec(kvd, 0.0, 0.05)
                lw.wo_bias = vec(cfg.hidden, 0.0, 0.05)
            if cfg.mlp_type == "gelu":
                lw.w1_bias, lw.w2_bias, lw.w3 = vec(cfg.ffn, 0.0, 0.05), vec(cfg.hidden, 0.0, 0.05), None
            if cfg.post_norms:
                lw.post_attn_norm, lw.post_ffn_norm = vec(cfg.hidden, 1.0, 0.1), vec(cfg.hidden, 1.0, 0.1)
        final_norm = vec(cfg.hidden, 1.0, 0.1)
        if cfg.norm_type == "layer":
            final_bias = vec(cfg.hidden, 0.0, 0.05)
    return OracleModel(cfg, emb, layers, final_norm, head, max_blocks, kv_fp16, final_norm_bias=final_bias)


def is_llama(cfg: ModelConfig):
    """Every architecture switch at its default."""
    return (cfg.norm_type == "rms" and cfg.mlp_type == "swiglu" and not cfg.parallel_residual and cfg.rope_dim == 0
            and not cfg.rope_neox and cfg.attn_softcap == 0 and not cfg.post_norms and cfg.embedding_scale <= 0
            and cfg.final_softcap <= 0)
