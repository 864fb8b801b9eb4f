"""Shared test plumbing: builds the same random model in the CPU oracle and on the GPU, and
installs the same synthetic pre-filled paged contexts in both."""
import numpy as np

from oracle import model as om
from oracle import numerics as nx


def gpu_model_from_oracle(be, omodel, pool_blocks, max_seqs=64, max_blocks_per_seq=None, max_batch=64):
    from vexel_amd.runtime import ModelRuntime
    c = omodel.cfg
    mr = ModelRuntime(be, c.num_layers, c.hidden, c.num_heads, c.num_kv_heads, c.head_dim, c.ffn, c.vocab,
                      eps=c.eps, rope_theta=c.rope_theta, block_size=c.block_size, pool_blocks=pool_blocks,
                      max_seqs=max_seqs, max_blocks_per_seq=max_blocks_per_seq, max_batch=max_batch,
                      kv_fp16=omodel.pool.use_fp16)
    from oracle.model import is_llama
    from vexel_amd.runtime import EXTRA_NAMES
    if not is_llama(c):
        mr.set_architecture(c.norm_type, c.mlp_type, c.parallel_residual, c.rope_dim, c.rope_neox, c.post_norms,
                            c.attn_softcap, c.embedding_scale, c.final_softcap)
    for i, lw in enumerate(omodel.layers):
        ws = {n: (getattr(lw, n).fmt, getattr(lw, n).data, getattr(lw, n).n, getattr(lw, n).k)
              for n in ("wq", "wk", "wv", "wo", "w1", "w2", "w3") if getattr(lw, n) is not None}
        mr.set_layer(i, lw.attn_norm, lw.ffn_norm, ws)
        extras = {n: getattr(lw, n) for n in EXTRA_NAMES if getattr(lw, n) is not None}
        if extras:
            mr.set_layer_extras(i, **extras)
    h = omodel.lm_head
    mr.set_head(omodel.embedding, omodel.final_norm, (h.fmt, h.data, h.n, h.k))
    if omodel.final_norm_bias is not None:
        mr.set_final_norm_bias(omodel.final_norm_bias)
    return mr


def install_context(omodel, mr, be, seq_id, blocks, seq_len, rng):
    """Gives sequence seq_id a pre-filled context of seq_len tokens living in the given physical
    blocks: N(0,1) K/V values (f16-rounded when the pool is F16), identical in oracle and GPU."""
    c = omodel.cfg
    pool = omodel.pool
    blocks = [int(b) for b in blocks]
    pool.create_sequence(seq_id)
    st = pool.seqs[seq_id]
    for layer in range(c.num_layers):
        st.block_tables[layer] = list(blocks)
        for b in blocks:
            pool.free_lists[layer].remove(b)
            pool.ref_counts[layer][b] = 1
    st.seq_len = seq_len
    mr.create_sequence(seq_id)
    mr.adopt_blocks(seq_id, blocks, seq_len)
    per_block = 2 * c.block_size * c.num_kv_heads * c.head_dim
    esz = 2 if pool.use_fp16 else 4
    for layer in range(c.num_layers):
        for b in blocks:
            vals = rng.standard_normal(per_block).astype(np.float32)
            data = nx.f32_to_f16_array(vals) if pool.use_fp16 else vals
            omodel.kv[layer][b * per_block:(b + 1) * per_block] = data
            be.to_device(mr.kv_pool(layer) + b * per_block * esz, data)


def assert_logits_close(got, want, what=""):
    """north-star tolerance: 1e-2 absolute / 1e-3 relative in float32."""
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    lim = 1e-2 + 1e-3 * np.abs(want.astype(np.float64))
    assert np.all(err <= lim), "%s: max err %.3e" % (what, err.max())
    return float(err.max())
