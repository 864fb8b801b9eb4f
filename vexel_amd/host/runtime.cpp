// Host runtime above the C ABI of include/vexel_hip.h: the part of vexel's Go runtime
// that drives the batched-decode path, restated in C++ because no Go toolchain exists in
// the build image. It calls the device only through the vx_* entry points, exactly as
// the Go packages would through the cgo shim.
//
//   BlockPool      inference/runtime/gpu_block_pool.go (free list, ref counts, block tables,
//                  truncate, share, stats). Every layer's bookkeeping is identical there, so
//                  one table per sequence serves all layers here, with a device-resident
//                  mirror (block-table matrix, free stack) that vx_pack_batch advances in
//                  lock step with the host rule.
//   execute_layer  inference/runtime/block.go:763-1081 (LLaMA arm) for a whole batch of
//                  single-token sequences (block.go:1087-1119 loops over them instead).
//   vh_decode_batched  inference/runtime/decode.go:612-654 (+339-461).
//   vh_prefill     inference/runtime/decode.go:961-1096 / 1446-1569 for one sequence.
//   vh_decode_graph  the decode step captured once in a hipGraph and replayed with all
//                  per-step metadata built on the device; greedy sampling as
//                  inference/pkg/sampler/sampler.go:80-91.
#include <math.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <map>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "vexel_host.h"

namespace {

thread_local char g_err[512] = "";

int fail(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return VH_ERR;
}

#define VXC(expr)                                                         \
    do {                                                                  \
        int _rc = (expr);                                                 \
        if (_rc != VX_OK) return fail("%s: %s", #expr, vx_last_error());  \
    } while (0)
#define VHC(expr)                      \
    do {                               \
        if ((expr) != VH_OK) return VH_ERR; \
    } while (0)

struct SeqState {
    std::vector<int32_t> table;  // logical block -> physical block (same for every layer)
    int seq_len = 0;
    int slot = -1;               // row in the device block-table matrix
    bool dirty = true;           // device row differs from `table`
};

struct Fragment {                 // kv/fragment.go:9-16
    int num_tokens = 0;
    std::vector<int32_t> blocks;  // the cached sequence's table (the same for every layer), one reference each
};

struct BlockPool {
    int block_size = 16, max_blocks = 0;
    std::map<std::string, Fragment> fragments;    // kv/fragment.go:19-23
    std::vector<int32_t> free_list;               // gpu_block_pool.go:110-116
    std::unordered_map<int32_t, int> ref_counts;  // gpu_block_pool.go:42-43
    std::map<int64_t, SeqState> seqs;
    std::mutex mu;                                // gpu_block_pool.go:46
    std::vector<int> free_slots;
    bool free_dirty = true;

    int alloc_block(int32_t *out) {               // gpu_block_pool.go:200-209
        if (free_list.empty()) return fail("no free blocks (max=%d)", max_blocks);
        *out = free_list.back();
        free_list.pop_back();
        ref_counts[*out] = 1;
        free_dirty = true;
        return VH_OK;
    }
    void release_block(int32_t b) {               // gpu_block_pool.go:211-219
        auto it = ref_counts.find(b);
        int rc = it == ref_counts.end() ? 0 : it->second;
        if (rc <= 1) {
            if (it != ref_counts.end()) ref_counts.erase(it);
            free_list.push_back(b);
            free_dirty = true;
        } else {
            it->second = rc - 1;
        }
    }
    int ensure_blocks(SeqState &s, int end_pos) {  // gpu_block_pool.go:234-245
        if (end_pos <= 0) return VH_OK;
        int last = (end_pos - 1) / block_size;
        while ((int)s.table.size() <= last) {
            int32_t b;
            VHC(alloc_block(&b));
            s.table.push_back(b);
            s.dirty = true;
        }
        return VH_OK;
    }
};

}  // namespace

struct vh_model {
    vx_backend *be = nullptr;
    vh_config cfg{};
    std::vector<vh_layer_weights> layers;
    const float *embedding = nullptr;
    const float *final_norm = nullptr;
    vh_qweight lm_head{};
    std::vector<void *> adopted;  // device buffers a loader handed over (vh_model_adopt_buffer)
    BlockPool pool;
    std::vector<void *> kv;

    int32_t *d_tables = nullptr, *d_num_blocks = nullptr, *d_free = nullptr, *d_free_count = nullptr;
    int32_t *d_slots = nullptr, *d_positions = nullptr, *d_tokens = nullptr, *d_next = nullptr;
    int32_t *d_cu = nullptr, *d_token_pos = nullptr, *d_slot_map = nullptr, *d_kv_lens = nullptr;
    int32_t *d_pos_in = nullptr;  // positions of a host-driven step, input of the packing kernel
    int32_t *d_status = nullptr, *d_step = nullptr, *d_log = nullptr;
    int log_cap = 0;  // steps the log can hold

    float *x = nullptr, *norm = nullptr, *q = nullptr, *k = nullptr, *v = nullptr, *attn = nullptr;
    float *gate = nullptr, *up = nullptr, *logits = nullptr;

    bool fused = true;  // take the fused decode entry points where the weights allow it

    vh_arch arch{};                       // all zero: the LLaMA arm
    std::vector<vh_layer_extras> extras;  // per layer, all NULL by default
    const float *final_norm_bias = nullptr;
    float *zeros = nullptr;               // [hidden] zeros: the bias of a LayerNorm whose bias tensor is absent
    bool general = false;                 // some switch or extra tensor is set: the one-call-per-operation sequence
    bool fused_ok = true;                 // the layer differs from LLaMA's at most by Q/K/V biases and the RoPE form
    bool attn_fused_ok = true;            // the attention half does (RMSNorm without a bias in front of Q|K|V): its fused block serves it
                                          // (Qwen 2): decode may still take the fused entry points

    vx_graph *graph = nullptr;
    int graph_batch = 0;
    uint64_t graph_scratch_gen = 0;  // vx_scratch_generation() when the graph was captured
    std::vector<int64_t> dev_seq_ids;  // batch currently loaded in d_slots (device-driven mode)
    std::vector<int32_t> dev_positions;
};

namespace {

template <class T>
int dev_alloc(vh_model *m, T **p, size_t count) {
    *p = (T *)vx_alloc_permanent(m->be, (count ? count : 1) * sizeof(T));
    if (!*p) return fail("vx_alloc_permanent(%zu): %s", count * sizeof(T), vx_last_error());
    return VH_OK;
}

SeqState *find_seq(vh_model *m, int64_t id) {
    auto it = m->pool.seqs.find(id);
    return it == m->pool.seqs.end() ? nullptr : &it->second;
}

int create_seq_locked(vh_model *m, int64_t id) {  // gpu_block_pool.go:126-135 (replaces an existing entry)
    BlockPool &p = m->pool;
    auto it = p.seqs.find(id);
    int slot;
    if (it != p.seqs.end()) {
        slot = it->second.slot;
    } else {
        if (p.free_slots.empty()) return fail("more than %d live sequences", m->cfg.max_seqs);
        slot = p.free_slots.back();
        p.free_slots.pop_back();
    }
    SeqState s;
    s.slot = slot;
    p.seqs[id] = s;
    return VH_OK;
}

int sync_pool_to_device(vh_model *m) {
    BlockPool &p = m->pool;
    const int mb = m->cfg.max_blocks_per_seq;
    for (auto &kv : p.seqs) {
        SeqState &s = kv.second;
        if (!s.dirty) continue;
        if ((int)s.table.size() > mb)
            return fail("sequence %lld needs %zu blocks, the table holds %d", (long long)kv.first, s.table.size(), mb);
        if (!s.table.empty())
            VXC(vx_to_device(m->be, m->d_tables + (size_t)s.slot * mb, s.table.data(), s.table.size() * 4));
        int32_t nb = (int32_t)s.table.size();
        VXC(vx_to_device(m->be, m->d_num_blocks + s.slot, &nb, 4));
        s.dirty = false;
    }
    if (p.free_dirty) {
        if (!p.free_list.empty()) VXC(vx_to_device(m->be, m->d_free, p.free_list.data(), p.free_list.size() * 4));
        int32_t fc = (int32_t)p.free_list.size();
        VXC(vx_to_device(m->be, m->d_free_count, &fc, 4));
        p.free_dirty = false;
    }
    return VH_OK;
}

bool fast(const vh_qweight &w) { return vx_matmul_quant_has_fast_path(w.fmt, w.data, w.n, w.k) != 0; }

// out = act * w^T (+ residual) where `act` is both in the backend's prepared slot (when `prepared`) and,
// unless every consumer takes the prepared path, in float32 at a_f32.
int mm(vh_model *m, bool prepared, const float *a_f32, const vh_qweight &w, float *out, const float *residual, int rows) {
    if (!w.data) return fail("weight not set");
    if (w.fmt == VH_F32) {  // a float32 output head: Backend.MatMulTransposed (model.go:394-404)
        if (!a_f32) return fail("internal: a float32 matrix needs the float32 activation");
        VXC(vx_matmul_transposed(m->be, a_f32, (const float *)w.data, out, rows, w.n, w.k));
        if (residual) VXC(vx_add(m->be, out, residual, out, rows * w.n));
        return VH_OK;
    }
    if (prepared && fast(w)) {
        VXC(vx_matmul_quant_prepared(m->be, w.fmt, w.data, out, residual, rows, w.n, w.k));
        return VH_OK;
    }
    VXC(vx_matmul_quant(m->be, w.fmt, a_f32, w.data, out, residual, rows, w.n, w.k));
    return VH_OK;
}

// RMSNorm feeding the given weights: fused norm + prepare when any of them has the MFMA path.
int norm_for(vh_model *m, const float *x, const float *nw, float *norm, int rows, const vh_qweight *const *ws, int nws,
             bool *prepared) {
    const vh_config &c = m->cfg;
    int nfast = 0;
    for (int i = 0; i < nws; i++) nfast += fast(*ws[i]) ? 1 : 0;
    // a single row goes through the matrix-vector kernel, which reads the float32 activation
    *prepared = rows > 1 && nfast > 0 && c.hidden % 256 == 0;
    if (*prepared)
        VXC(vx_rmsnorm_prepare(m->be, x, nw, nfast == nws ? nullptr : norm, rows, c.hidden, c.eps));
    else
        VXC(vx_rmsnorm(m->be, x, nw, norm, rows, c.hidden, c.eps));
    return VH_OK;
}

// attention output -> Wo (+x), FFN norm, gate/up, SiLU*up, down (+x): block.go:981-1077, shared by decode and prefill
int layer_tail(vh_model *m, const vh_layer_weights &w, float *x, float *norm, const float *attn, float *gate, float *up,
               int rows) {
    const vh_config &c = m->cfg;
    VHC(mm(m, false, attn, w.wo, x, x, rows));                                            // block.go:981-990
    bool prep;
    const vh_qweight *w13[2] = {&w.w1, &w.w3};
    VHC(norm_for(m, x, w.ffn_norm, norm, rows, w13, 2, &prep));                           // block.go:996-998
    VHC(mm(m, prep, norm, w.w1, gate, nullptr, rows));                                    // block.go:1043-1050
    VHC(mm(m, prep, norm, w.w3, up, nullptr, rows));
    if (rows > 1 && fast(w.w2) && c.ffn % 256 == 0) {                                     // block.go:1056-1077
        VXC(vx_silu_mul_prepare(m->be, gate, up, nullptr, rows, c.ffn));
        VHC(mm(m, true, nullptr, w.w2, x, x, rows));
    } else {
        VXC(vx_silu_mul(m->be, gate, up, gate, rows * c.ffn));
        VHC(mm(m, false, gate, w.w2, x, x, rows));
    }
    return VH_OK;
}

// ---- the general sequence of block.go:834-1077 for the architectures beside LLaMA ----

// applyNorm (block.go:562-576): LayerNorm with its bias, or RMSNorm, which ignores the bias
int g_norm(vh_model *m, const float *x, const float *w, const float *b, float *out, int rows) {
    const vh_config &c = m->cfg;
    if (m->arch.norm_type == VH_NORM_LAYER)
        VXC(vx_layernorm(m->be, x, w, b ? b : m->zeros, out, rows, c.hidden, c.eps));
    else
        VXC(vx_rmsnorm(m->be, x, w, out, rows, c.hidden, c.eps));
    return VH_OK;
}

// matMulTransposedWithBias (block.go:555-560); prepared: the activation is in the backend's prepared slot already
int g_mm(vh_model *m, const float *a, const vh_qweight &w, const float *bias, float *out, int rows, bool prepared = false) {
    VHC(mm(m, prepared, a, w, out, nullptr, rows));
    if (bias) VXC(vx_add_bias(m->be, out, bias, out, rows, w.n));
    return VH_OK;
}

// block.go:834-854: the attention norm and the three projections
int g_qkv(vh_model *m, int layer, const float *x, float *norm, float *q, float *k, float *v, int rows) {
    const vh_layer_weights &w = m->layers[layer];
    const vh_layer_extras &e = m->extras[layer];
    VHC(g_norm(m, x, w.attn_norm, e.attn_norm_bias, norm, rows));
    // (the three projections read one prepared copy of the normalised rows)
    const bool prep = rows > 1 && m->cfg.hidden % 256 == 0 && fast(w.wq) && fast(w.wk) && fast(w.wv);
    if (prep) VXC(vx_prepare_act(m->be, norm, rows, m->cfg.hidden));
    VHC(g_mm(m, norm, w.wq, e.wq_bias, q, rows, prep));
    VHC(g_mm(m, norm, w.wk, e.wk_bias, k, rows, prep));
    VHC(g_mm(m, norm, w.wv, e.wv_bias, v, rows, prep));
    return VH_OK;
}

// block.go:834-868 for rows whose K/V go to the pool at given slots (decode batches, later prompt chunks, tree rows) in an
// architecture whose norm the fused attention block does not have (LayerNorm, a norm bias): the norm by its own
// kernel, one prepared copy of its output, then that block's grouped projection, biases, RoPE form and KV store.
// false: the weights or the row count have no such path (the caller takes g_qkv and the separate RoPE + store).
bool g_qkv_fusable(const vh_model *m, int layer, int rows) {
    if (!m->fused || rows < 2 || layer >= m->cfg.num_layers || m->cfg.hidden % 256 != 0) return false;
    const vh_layer_weights &w = m->layers[layer];
    return w.wq.data && w.wk.data && w.wv.data && fast(w.wq) && fast(w.wk) && fast(w.wv) &&
           vx_decode_attn_qkv_supported(&w.wq, &w.wk, &w.wv, m->cfg.head_dim) != 0;
}
// k_dense / v_dense (a prompt's first chunk): the rotated K and the V rows also as dense floats.
int g_qkv_store(vh_model *m, int layer, const float *x, float *norm, float *q, int rows, const int32_t *d_pos,
                const int32_t *d_slot, float *k_dense = nullptr, float *v_dense = nullptr) {
    const vh_config &c = m->cfg;
    const vh_layer_weights &w = m->layers[layer];
    const vh_layer_extras &e = m->extras[layer];
    VHC(g_norm(m, x, w.attn_norm, e.attn_norm_bias, norm, rows));
    VXC(vx_prepare_act(m->be, norm, rows, c.hidden));
    VXC(vx_prefill_attn_qkv(m->be, nullptr, nullptr, c.eps, 1, &w.wq, &w.wk, &w.wv, e.wq_bias, e.wk_bias, e.wv_bias, rows, d_pos,
                            d_slot, m->kv[layer], c.kv_fp16, c.num_heads, c.num_kv_heads, c.head_dim, c.block_size,
                            c.rope_theta, m->arch.rope_dim, m->arch.rope_neox, q, k_dense, v_dense));
    return VH_OK;
}

// block.go:972-1077: Wo, post-norm, residual(s), FFN norm, MLP. `norm` holds the attention norm's output on entry.
int g_tail(vh_model *m, int layer, float *x, float *norm, const float *attn, float *gate, float *up, int rows) {
    const vh_config &c = m->cfg;
    const vh_arch &a = m->arch;
    const vh_layer_weights &w = m->layers[layer];
    const vh_layer_extras &e = m->extras[layer];
    vx_backend *be = m->be;
    float *o = a.parallel_residual ? up : norm;                                        // :972-978
    VHC(g_mm(m, attn, w.wo, e.wo_bias, o, rows));                                      // :981-983
    if (a.post_norms && e.post_attn_norm) VXC(vx_rmsnorm(be, o, e.post_attn_norm, o, rows, c.hidden, c.eps));  // :985-987
    // The activation can leave its kernel as W2's prepared operand (one launch less). That kernel takes a workgroup per
    // row, and GELU's double-precision tanh makes it slow where the rows are few: a prompt chunk's rows only.
    const bool act_prepared = rows >= 128 && fast(w.w2) && c.ffn % 256 == 0;
    bool gated_prepared = false;  // RMSNorm in front of a gated MLP: one launch normalises and prepares W1's and W3's operand
    if (!a.parallel_residual) {
        VXC(vx_add(be, x, o, x, rows * c.hidden));                                     // :989-991
        if (w.ffn_norm && a.norm_type != VH_NORM_LAYER && a.mlp_type != VH_MLP_GELU) {
            const vh_qweight *w13[2] = {&w.w1, &w.w3};
            VHC(norm_for(m, x, w.ffn_norm, norm, rows, w13, 2, &gated_prepared));      // :996-998
        } else if (w.ffn_norm) {
            VHC(g_norm(m, x, w.ffn_norm, e.ffn_norm_bias, norm, rows));                // :996-998
        }
    }
    if (a.mlp_type == VH_MLP_GELU) {                                                   // :1004-1037
        VHC(g_mm(m, norm, w.w1, e.w1_bias, gate, rows));
        if (act_prepared) {
            VXC(vx_gelu_prepare(be, gate, nullptr, rows, c.ffn));
            VHC(g_mm(m, nullptr, w.w2, e.w2_bias, norm, rows, true));
        } else {
            VXC(vx_gelu(be, gate, gate, rows * c.ffn));
            VHC(g_mm(m, gate, w.w2, e.w2_bias, norm, rows));
        }
    } else {                                                                           // :1040-1062
        VHC(mm(m, gated_prepared, norm, w.w1, gate, nullptr, rows));
        VHC(mm(m, gated_prepared, norm, w.w3, up, nullptr, rows));
        if (act_prepared) {
            if (a.mlp_type == VH_MLP_GEGLU)
                VXC(vx_gelu_mul_prepare(be, gate, up, nullptr, rows, c.ffn));
            else
                VXC(vx_silu_mul_prepare(be, gate, up, nullptr, rows, c.ffn));
            VHC(mm(m, true, nullptr, w.w2, norm, nullptr, rows));
        } else {
            if (a.mlp_type == VH_MLP_GEGLU)
                VXC(vx_gelu_mul(be, gate, up, gate, rows * c.ffn));
            else
                VXC(vx_silu_mul(be, gate, up, gate, rows * c.ffn));
            VHC(mm(m, false, gate, w.w2, norm, nullptr, rows));
        }
    }
    if (a.post_norms && e.post_ffn_norm) VXC(vx_rmsnorm(be, norm, e.post_ffn_norm, norm, rows, c.hidden, c.eps));  // :1066-1069
    if (a.parallel_residual) VXC(vx_add(be, x, o, x, rows * c.hidden));                // :1072-1075
    VXC(vx_add(be, x, norm, x, rows * c.hidden));
    return VH_OK;
}

// embedding scale (decode.go:197-205) and the final norm (model.go:207-226) of the general sequence
int g_scale_embedding(vh_model *m, float *x, int rows) {
    if (m->arch.embedding_scale > 0.f) VXC(vx_scale_buffer(m->be, x, m->arch.embedding_scale, rows * m->cfg.hidden));
    return VH_OK;
}

bool attn_fusable(const vh_model *m, int layer) {
    if (!m->fused || (m->general && !m->attn_fused_ok) || layer >= m->cfg.num_layers) return false;
    const vh_layer_weights &w = m->layers[layer];
    return w.wq.data && w.wk.data && w.wv.data && vx_decode_attn_qkv_supported(&w.wq, &w.wk, &w.wv, m->cfg.head_dim) != 0;
}

// One layer for `rows` single-token sequences; positions, slots, tables and lengths are on the device.
// *chained says, on entry, that the backend's prepared slot already holds RMSNorm(x)*attn_norm of this
// layer (left there by the previous layer's fused tail) and, on exit, the same for `next_norm`.
int execute_layer_decode(vh_model *m, int layer, int rows, int max_kv_len, const float *next_norm, bool *chained) {
    const vh_config &c = m->cfg;
    const vh_layer_weights &w = m->layers[layer];
    const float scale = (float)(1.0 / sqrt((double)c.head_dim));                          // block.go:862
    if (m->general && !attn_fusable(m, layer)) {
        if (*chained) return fail("internal: prepared activation handed to a general layer");
        if (g_qkv_fusable(m, layer, rows)) {
            VHC(g_qkv_store(m, layer, m->x, m->norm, m->q, rows, m->d_token_pos, m->d_slot_map));
        } else {
            VHC(g_qkv(m, layer, m->x, m->norm, m->q, m->k, m->v, rows));
            VXC(vx_rope_store_paged_ex(m->be, m->q, m->k, m->v, m->d_token_pos, m->d_slot_map, m->kv[layer], c.kv_fp16, rows,
                                       c.num_heads, c.num_kv_heads, c.head_dim, c.block_size, c.rope_theta, m->arch.rope_dim,
                                       m->arch.rope_neox));                           // :858, :868
        }
        VXC(vx_sdpa_paged_decode_ragged(m->be, m->q, m->kv[layer], c.kv_fp16, m->d_tables, m->d_slots, m->d_kv_lens,
                                        m->attn, rows, c.max_blocks_per_seq, c.block_size, c.num_heads, c.num_kv_heads,
                                        c.head_dim, scale, max_kv_len));               // :872 (no soft cap on this arm)
        return g_tail(m, layer, m->x, m->norm, m->attn, m->gate, m->up, rows);
    }
    if (attn_fusable(m, layer)) {   // block.go:834-868; one row: matrix-vector launches inside the same entry points
        const vh_layer_extras &e = m->extras[layer];
        VXC(vx_decode_attn_qkv_ex(m->be, m->x, w.attn_norm, c.eps, *chained ? 1 : 0, &w.wq, &w.wk, &w.wv, e.wq_bias, e.wk_bias,
                                  e.wv_bias, rows, m->d_token_pos, m->d_slot_map, m->kv[layer], c.kv_fp16, c.num_heads,
                                  c.num_kv_heads, c.head_dim, c.block_size, c.rope_theta, m->arch.rope_dim, m->arch.rope_neox,
                                  m->q));
    } else {
        if (*chained) return fail("internal: prepared activation handed to an unfused layer");
        bool prep;
        const vh_qweight *qkv[3] = {&w.wq, &w.wk, &w.wv};
        VHC(norm_for(m, m->x, w.attn_norm, m->norm, rows, qkv, 3, &prep));                // block.go:834-837
        VHC(mm(m, prep, m->norm, w.wq, m->q, nullptr, rows));                             // block.go:841-854
        VHC(mm(m, prep, m->norm, w.wk, m->k, nullptr, rows));
        VHC(mm(m, prep, m->norm, w.wv, m->v, nullptr, rows));
        VXC(vx_rope_store_paged(m->be, m->q, m->k, m->v, m->d_token_pos, m->d_slot_map, m->kv[layer], c.kv_fp16, rows,
                                c.num_heads, c.num_kv_heads, c.head_dim, c.block_size, c.rope_theta));  // :858, :868
    }
    // (a layer whose second half is not LLaMA's - post-norms, GeGLU: Gemma - keeps the general sequence there)
    const bool tail_general = m->general && !m->fused_ok;
    const bool ffn_fused = !tail_general && m->fused && w.wo.data && w.w1.data && w.w2.data && w.w3.data &&
                           vx_decode_ffn_supported(&w.wo, &w.w1, &w.w3, &w.w2);
    // the fused tail can merge the attention's split-KV partials itself
    const bool split = ffn_fused && (size_t)w.wo.k * 4 <= 64 * 1024 && c.head_dim % 4 == 0 &&
                       vx_sdpa_paged_decode_split_supported(c.kv_fp16, c.block_size, c.num_heads, c.num_kv_heads, c.head_dim);
    VXC(vx_sdpa_paged_decode_ragged(m->be, m->q, m->kv[layer], c.kv_fp16, m->d_tables, m->d_slots, m->d_kv_lens,
                                    split ? nullptr : m->attn, rows, c.max_blocks_per_seq, c.block_size, c.num_heads,
                                    c.num_kv_heads, c.head_dim, scale, max_kv_len));       // block.go:872
    *chained = false;
    if (ffn_fused) {                                                                      // block.go:981-1077
        VXC(vx_decode_ffn(m->be, split ? nullptr : m->attn, m->x, &w.wo, w.ffn_norm, c.eps, &w.w1, &w.w3, &w.w2, rows,
                          next_norm));
        *chained = next_norm != nullptr;
        return VH_OK;
    }
    if (tail_general) return g_tail(m, layer, m->x, m->norm, m->attn, m->gate, m->up, rows);
    return layer_tail(m, w, m->x, m->norm, m->attn, m->gate, m->up, rows);
}

// embedding -> layers -> final norm -> lm_head -> argmax for a decode batch (decode.go:404-452)
int forward_decode(vh_model *m, int rows, int max_kv_len) {
    const vh_config &c = m->cfg;
    VXC(vx_embedding(m->be, m->d_tokens, rows, m->embedding, m->x, c.vocab, c.hidden));
    VHC(g_scale_embedding(m, m->x, rows));
    const bool head_prepared = rows > 1 && m->fused && (!m->general || m->fused_ok) && fast(m->lm_head) && c.hidden % 256 == 0;
    bool chained = false;
    // the step's RoPE angles once for all layers: the fused Q|K|V launches then rotate and store their own rows
    if (m->fused && !m->general) VXC(vx_rope_table_prepare(m->be, m->d_token_pos, rows, c.head_dim, c.rope_theta));
    for (int l = 0; l < c.num_layers; l++) {
        const float *next_norm = l + 1 < c.num_layers ? (rows > 1 && attn_fusable(m, l + 1) ? m->layers[l + 1].attn_norm : nullptr)
                                                      : (head_prepared ? m->final_norm : nullptr);
        VHC(execute_layer_decode(m, l, rows, max_kv_len, next_norm, &chained));
    }
    if (chained) {                                                                        // model.go:207-226, 352-422
        VHC(mm(m, true, nullptr, m->lm_head, m->logits, nullptr, rows));
    } else if (m->general && !m->fused_ok) {
        VHC(g_norm(m, m->x, m->final_norm, m->final_norm_bias, m->norm, rows));
        VHC(mm(m, false, m->norm, m->lm_head, m->logits, nullptr, rows));
    } else {
        bool prep;
        const vh_qweight *hw[1] = {&m->lm_head};
        VHC(norm_for(m, m->x, m->final_norm, m->norm, rows, hw, 1, &prep));
        VHC(mm(m, prep, m->norm, m->lm_head, m->logits, nullptr, rows));
    }
    VXC(vx_argmax_rows(m->be, m->logits, rows, c.vocab, m->d_next));
    return VH_OK;
}

int check_ready(vh_model *m) {
    if (!m->embedding || !m->final_norm || !m->lm_head.data) return fail("model head / embedding not set");
    for (auto &l : m->layers)
        if (!l.attn_norm || !l.wq.data) return fail("a layer's weights are not set");
    if (m->arch.mlp_type != VH_MLP_GELU)
        for (auto &l : m->layers)
            if (!l.w3.data) return fail("a layer has no w3 and the MLP is gated");
    return VH_OK;
}

}  // namespace

extern "C" {

const char *vh_last_error(void) { return g_err; }
void vh_set_error(const char *text) { snprintf(g_err, sizeof(g_err), "%s", text ? text : ""); }  // for gguf.cpp

void vh_model_get_config(const vh_model *m, vh_config *out) {
    if (m && out) *out = m->cfg;
}

void vh_model_adopt_buffer(vh_model *m, void *device_ptr) {
    if (m && device_ptr) m->adopted.push_back(device_ptr);
}

int vh_model_create(vx_backend *be, const vh_config *cfg, vh_model **out) {
    if (!be || !cfg || !out) return fail("null argument");
    const vh_config &c = *cfg;
    if (c.num_layers <= 0 || c.hidden <= 0 || c.num_heads <= 0 || c.num_kv_heads <= 0 || c.head_dim <= 0 ||
        c.ffn <= 0 || c.vocab <= 0 || c.block_size <= 0 || c.pool_blocks <= 0 || c.max_seqs <= 0 ||
        c.max_blocks_per_seq <= 0 || c.max_batch <= 0 || c.max_batch > 1024)
        return fail("bad configuration");
    if (c.num_heads % c.num_kv_heads) return fail("%d heads not a multiple of %d kv heads", c.num_heads, c.num_kv_heads);
    vh_model *m = new vh_model();
    m->be = be;
    m->cfg = c;
    m->layers.resize(c.num_layers);
    m->extras.resize(c.num_layers);
    m->pool.block_size = c.block_size;
    m->pool.max_blocks = c.pool_blocks;
    m->pool.free_list.resize(c.pool_blocks);
    for (int i = 0; i < c.pool_blocks; i++) m->pool.free_list[i] = i;
    for (int i = c.max_seqs - 1; i >= 0; i--) m->pool.free_slots.push_back(i);
    const size_t kv_bytes = (size_t)c.pool_blocks * 2 * c.block_size * c.num_kv_heads * c.head_dim * (c.kv_fp16 ? 2 : 4);
    m->kv.resize(c.num_layers, nullptr);
    for (int l = 0; l < c.num_layers; l++) {
        m->kv[l] = vx_alloc_permanent(be, kv_bytes);
        if (!m->kv[l]) {
            fail("KV pool layer %d (%zu bytes): %s", l, kv_bytes, vx_last_error());
            vh_model_destroy(m);
            return VH_ERR;
        }
    }
    const size_t mb = c.max_batch;
    int rc = VH_OK;
    rc |= dev_alloc(m, &m->d_tables, (size_t)c.max_seqs * c.max_blocks_per_seq);
    rc |= dev_alloc(m, &m->d_num_blocks, c.max_seqs);
    rc |= dev_alloc(m, &m->d_free, c.pool_blocks);
    rc |= dev_alloc(m, &m->d_free_count, 1);
    rc |= dev_alloc(m, &m->d_slots, mb);
    rc |= dev_alloc(m, &m->d_positions, mb);
    rc |= dev_alloc(m, &m->d_tokens, mb);
    rc |= dev_alloc(m, &m->d_next, mb);
    rc |= dev_alloc(m, &m->d_cu, mb + 1);
    rc |= dev_alloc(m, &m->d_token_pos, mb);
    rc |= dev_alloc(m, &m->d_slot_map, mb);
    rc |= dev_alloc(m, &m->d_kv_lens, mb);
    rc |= dev_alloc(m, &m->d_pos_in, mb);
    rc |= dev_alloc(m, &m->d_status, 1);
    rc |= dev_alloc(m, &m->d_step, 1);
    rc |= dev_alloc(m, &m->x, mb * c.hidden);
    rc |= dev_alloc(m, &m->norm, mb * c.hidden);
    rc |= dev_alloc(m, &m->q, mb * c.num_heads * c.head_dim);
    rc |= dev_alloc(m, &m->k, mb * c.num_kv_heads * c.head_dim);
    rc |= dev_alloc(m, &m->v, mb * c.num_kv_heads * c.head_dim);
    rc |= dev_alloc(m, &m->attn, mb * c.num_heads * c.head_dim);
    rc |= dev_alloc(m, &m->gate, mb * c.ffn);
    rc |= dev_alloc(m, &m->up, mb * c.ffn);
    rc |= dev_alloc(m, &m->logits, mb * c.vocab);
    if (rc) {
        vh_model_destroy(m);
        return VH_ERR;
    }
    std::vector<int32_t> zeros((size_t)c.max_seqs * c.max_blocks_per_seq, 0);
    if (vx_to_device(be, m->d_tables, zeros.data(), zeros.size() * 4) ||
        vx_to_device(be, m->d_num_blocks, zeros.data(), (size_t)c.max_seqs * 4)) {
        fail("init: %s", vx_last_error());
        vh_model_destroy(m);
        return VH_ERR;
    }
    *out = m;
    return VH_OK;
}

static void drop_graph(vh_model *m);

void vh_model_destroy(vh_model *m) {
    if (!m) return;
    drop_graph(m);
    for (void *p : m->kv) vx_free(m->be, p);
    void *bufs[] = {m->d_tables, m->d_num_blocks, m->d_free, m->d_free_count, m->d_slots, m->d_positions, m->d_tokens,
                    m->d_next, m->d_cu, m->d_token_pos, m->d_slot_map, m->d_kv_lens, m->d_pos_in, m->d_status, m->d_step, m->d_log,
                    m->x, m->norm, m->q, m->k, m->v, m->attn, m->gate, m->up, m->logits, m->zeros};
    for (void *p : bufs) vx_free(m->be, p);
    for (void *p : m->adopted) vx_free(m->be, p);
    delete m;
}

int vh_model_set_layer(vh_model *m, int layer, const vh_layer_weights *w) {
    if (!m || !w || layer < 0 || layer >= m->cfg.num_layers) return fail("bad layer index");
    const vh_config &c = m->cfg;
    const int qd = c.num_heads * c.head_dim, kvd = c.num_kv_heads * c.head_dim;
    if (w->wq.n != qd || w->wq.k != c.hidden || w->wk.n != kvd || w->wv.n != kvd || w->wo.n != c.hidden ||
        w->wo.k != qd || w->w1.n != c.ffn || (w->w3.data && w->w3.n != c.ffn) || w->w2.n != c.hidden || w->w2.k != c.ffn)
        return fail("layer %d: weight shapes do not match the configuration", layer);
    drop_graph(m);  // a recorded step holds the previous matrices' addresses
    m->layers[layer] = *w;
    // Decode batches stream load-time packed copies of the projections (formats and shapes without one stay as
    // they are); a model that never runs more than one row at a time has no use for them.
    static const bool no_pack = getenv("VEXEL_HIP_NO_PACK") != nullptr;
    if (c.max_batch >= 2 && !no_pack) {
        const vh_qweight *all[7] = {&w->wq, &w->wk, &w->wv, &w->wo, &w->w1, &w->w3, &w->w2};
        for (const vh_qweight *q : all) {
            if (!q->data) continue;
            const int rc = vx_qweight_pack(m->be, q);
            if (rc != VX_OK && rc != VX_ERR_UNSUPPORTED) return fail("layer %d: %s", layer, vx_last_error());
        }
    }
    return VH_OK;
}

int vh_model_set_head(vh_model *m, const float *embedding, const float *final_norm, const vh_qweight *lm_head) {
    if (!m || !embedding || !final_norm || !lm_head) return fail("null argument");
    if (lm_head->n != m->cfg.vocab || lm_head->k != m->cfg.hidden) return fail("lm_head shape mismatch");
    drop_graph(m);
    m->embedding = embedding;
    m->final_norm = final_norm;
    m->lm_head = *lm_head;
    // (the output head of a batched model streams a packed copy like the projections)
    if (m->cfg.max_batch >= 2 && getenv("VEXEL_HIP_NO_PACK") == nullptr) {
        const int rc = vx_qweight_pack(m->be, lm_head);
        if (rc != VX_OK && rc != VX_ERR_UNSUPPORTED) return fail("lm_head: %s", vx_last_error());
    }
    return VH_OK;
}

// A recorded step goes away: because it was recorded with another kernel sequence or other addresses, or with its
// model. The stream is drained first, so that no replay is in flight when the executable graph is destroyed.
static void drop_graph(vh_model *m) {
    if (m->graph) {
        (void)vx_sync(m->be);
        vx_graph_destroy(m->graph);
        m->graph = nullptr;
        m->graph_batch = 0;
    }
}

static void refresh_general(vh_model *m) {
    const vh_arch &a = m->arch;
    bool g = a.norm_type || a.mlp_type || a.parallel_residual || a.rope_dim || a.rope_neox || a.post_norms ||
             a.attn_softcap > 0.f || a.embedding_scale > 0.f || m->final_norm_bias;
    for (const vh_layer_extras &e : m->extras)
        g = g || e.attn_norm_bias || e.ffn_norm_bias || e.wq_bias || e.wk_bias || e.wv_bias || e.wo_bias || e.w1_bias ||
            e.w2_bias || e.post_attn_norm || e.post_ffn_norm;
    bool f = !a.norm_type && !a.mlp_type && !a.parallel_residual && !a.post_norms && !m->final_norm_bias;
    for (const vh_layer_extras &e : m->extras)
        f = f && !e.attn_norm_bias && !e.ffn_norm_bias && !e.wo_bias && !e.w1_bias && !e.w2_bias && !e.post_attn_norm &&
            !e.post_ffn_norm;
    bool af = !a.norm_type;
    for (const vh_layer_extras &e : m->extras) af = af && !e.attn_norm_bias;
    if (g != m->general || f != m->fused_ok || af != m->attn_fused_ok) drop_graph(m);
    m->general = g;
    m->fused_ok = f;
    m->attn_fused_ok = af;
}

int vh_model_set_architecture(vh_model *m, const vh_arch *arch) {
    if (!m || !arch) return fail("null argument");
    const vh_arch &a = *arch;
    if (a.norm_type < 0 || a.norm_type > VH_NORM_LAYER || a.mlp_type < 0 || a.mlp_type > VH_MLP_GEGLU)
        return fail("unknown norm type %d / MLP type %d", a.norm_type, a.mlp_type);
    if (a.parallel_residual && a.mlp_type != VH_MLP_GELU)
        return fail("the parallel residual goes with the GELU MLP only");  // block.go:972-976 shares a buffer with W3's product
    if (a.rope_dim < 0 || a.rope_dim > m->cfg.head_dim || a.rope_dim % 2 != 0)
        return fail("rope_dim %d invalid for head_dim %d", a.rope_dim, m->cfg.head_dim);
    if (a.attn_softcap < 0.f || a.final_softcap < 0.f) return fail("negative soft cap");
    if (a.mlp_type == VH_MLP_GELU && m->cfg.ffn < m->cfg.hidden && a.parallel_residual)
        return fail("the parallel residual keeps the attention output in an [rows, ffn] buffer: ffn %d < hidden %d", m->cfg.ffn,
                    m->cfg.hidden);
    if (a.norm_type == VH_NORM_LAYER && !m->zeros) {
        std::vector<float> z((size_t)m->cfg.hidden, 0.f);
        m->zeros = (float *)vx_alloc_permanent(m->be, z.size() * 4);
        if (!m->zeros) return fail("zero bias: %s", vx_last_error());
        VXC(vx_to_device(m->be, m->zeros, z.data(), z.size() * 4));
    }
    m->arch = a;
    drop_graph(m);
    refresh_general(m);
    return VH_OK;
}

void vh_model_get_architecture(const vh_model *m, vh_arch *out) {
    if (m && out) *out = m->arch;
}

int vh_model_set_layer_extras(vh_model *m, int layer, const vh_layer_extras *extras) {
    if (!m || !extras || layer < 0 || layer >= m->cfg.num_layers) return fail("bad layer index");
    m->extras[layer] = *extras;
    drop_graph(m);
    refresh_general(m);
    return VH_OK;
}

int vh_model_set_final_norm_bias(vh_model *m, const float *bias) {
    if (!m) return fail("null argument");
    m->final_norm_bias = bias;
    refresh_general(m);
    return VH_OK;
}

void vh_model_set_fused(vh_model *m, int on) {
    if (!m) return;
    m->fused = on != 0;
    drop_graph(m);  // the captured step was recorded with the other kernel sequence
}

void *vh_kv_pool(vh_model *m, int layer) {
    return (m && layer >= 0 && layer < m->cfg.num_layers) ? m->kv[layer] : nullptr;
}

void vh_step_buffers(vh_model *m, const int32_t **block_tables, const int32_t **table_rows, const int32_t **kv_lens) {
    if (block_tables) *block_tables = m ? m->d_tables : nullptr;
    if (table_rows) *table_rows = m ? m->d_slots : nullptr;
    if (kv_lens) *kv_lens = m ? m->d_kv_lens : nullptr;
}

// ------------------------------------------------------------------ GPUBlockPool
int vh_pool_create_sequence(vh_model *m, int64_t seq_id) {
    std::lock_guard<std::mutex> g(m->pool.mu);
    return create_seq_locked(m, seq_id);
}

int vh_pool_delete_sequence(vh_model *m, int64_t seq_id) {  // gpu_block_pool.go:138-157
    std::lock_guard<std::mutex> g(m->pool.mu);
    SeqState *s = find_seq(m, seq_id);
    if (!s) return VH_OK;
    for (int32_t b : s->table) m->pool.release_block(b);
    m->pool.free_slots.push_back(s->slot);
    m->pool.seqs.erase(seq_id);
    return VH_OK;
}

int vh_pool_truncate_sequence(vh_model *m, int64_t seq_id, int new_len) {  // gpu_block_pool.go:162-190
    std::lock_guard<std::mutex> g(m->pool.mu);
    SeqState *s = find_seq(m, seq_id);
    if (!s || new_len >= s->seq_len) return VH_OK;
    int keep = 0;
    if (new_len > 0) keep = (new_len - 1) / m->pool.block_size + 1;
    for (int i = keep; i < (int)s->table.size(); i++) m->pool.release_block(s->table[i]);
    if (keep < (int)s->table.size()) {
        s->table.resize(keep);
        s->dirty = true;
    }
    s->seq_len = new_len;
    return VH_OK;
}

int vh_pool_has_sequence(vh_model *m, int64_t seq_id) {
    std::lock_guard<std::mutex> g(m->pool.mu);
    return find_seq(m, seq_id) ? 1 : 0;
}

int vh_pool_share_blocks(vh_model *m, int64_t src_id, int64_t dst_id, int num_tokens) {  // gpu_block_pool.go:572-607
    std::lock_guard<std::mutex> g(m->pool.mu);
    SeqState *src = find_seq(m, src_id);
    if (!src) return fail("source sequence %lld not found", (long long)src_id);
    SeqState *dst = find_seq(m, dst_id);
    if (!dst) return fail("destination sequence %lld not found", (long long)dst_id);
    int nb = (num_tokens + m->pool.block_size - 1) / m->pool.block_size;
    if (nb > (int)src->table.size())
        return fail("source seq %lld has %zu blocks, need %d", (long long)src_id, src->table.size(), nb);
    for (int i = 0; i < nb; i++) {
        dst->table.push_back(src->table[i]);
        m->pool.ref_counts[src->table[i]]++;
    }
    dst->dirty = true;
    if (num_tokens > dst->seq_len) dst->seq_len = num_tokens;
    return VH_OK;
}

// ------------------------------------------------------------------ named fragments (kv/fragment.go, kv/paged_cache.go:285-343)
static void release_fragment(vh_model *m, const Fragment &f) {  // fragment.go:83-89
    for (int32_t b : f.blocks) m->pool.release_block(b);
}

int vh_fragment_cache(vh_model *m, const char *name, int64_t seq_id) {  // paged_cache.go:324-343, fragment.go:36-60
    if (!m || !name) return fail("bad arguments");
    std::lock_guard<std::mutex> g(m->pool.mu);
    SeqState *s = find_seq(m, seq_id);
    if (!s) return VH_OK;  // paged_cache.go:331-333: an unknown sequence caches nothing
    auto old = m->pool.fragments.find(name);
    if (old != m->pool.fragments.end()) {  // fragment.go:41-43: a fragment of that name gives its blocks back first
        release_fragment(m, old->second);
        m->pool.fragments.erase(old);
    }
    Fragment f;
    f.num_tokens = s->seq_len;
    f.blocks = s->table;
    for (int32_t b : f.blocks) m->pool.ref_counts[b]++;  // fragment.go:46-50 (AddRef)
    m->pool.fragments[name] = f;
    return VH_OK;
}

int vh_fragment_tokens(vh_model *m, const char *name) {  // fragment.go:63-68; -1: no such fragment
    if (!m || !name) return -1;
    std::lock_guard<std::mutex> g(m->pool.mu);
    auto it = m->pool.fragments.find(name);
    return it == m->pool.fragments.end() ? -1 : it->second.num_tokens;
}

int vh_fragment_count(vh_model *m) {  // fragment.go:92-101
    if (!m) return 0;
    std::lock_guard<std::mutex> g(m->pool.mu);
    return (int)m->pool.fragments.size();
}

int vh_fragment_delete(vh_model *m, const char *name) {  // fragment.go:71-79
    if (!m || !name) return fail("bad arguments");
    std::lock_guard<std::mutex> g(m->pool.mu);
    auto it = m->pool.fragments.find(name);
    if (it == m->pool.fragments.end()) return VH_OK;
    release_fragment(m, it->second);
    m->pool.fragments.erase(it);
    return VH_OK;
}

// The reference shares the fragment's blocks with the sequence and rotates K by insert_pos every time it reads
// them (paged_cache.go:225-283). Here the rotation happens once, at insertion: the fragment's rows are copied
// into the sequence's own blocks with K turned by insert_pos, so the attention kernels read the pool as it is and
// the fragment's blocks stay untouched for the next insertion at another position.
int vh_fragment_insert(vh_model *m, int64_t seq_id, const char *name, int insert_pos, int *num_tokens) {
    if (num_tokens) *num_tokens = 0;
    if (!m || !name || insert_pos < 0) return fail("bad arguments");
    const vh_config &c = m->cfg;
    if (m->arch.rope_neox || (m->arch.rope_dim != 0 && m->arch.rope_dim != c.head_dim))
        return fail("fragments are rotated as RoPEShift rotates (whole head, pairs 2j and 2j+1): not this model's RoPE");
    std::lock_guard<std::mutex> g(m->pool.mu);
    auto it = m->pool.fragments.find(name);
    if (it == m->pool.fragments.end()) return VH_OK;  // paged_cache.go:290-293: nothing to insert
    SeqState *s = find_seq(m, seq_id);
    if (!s) {  // paged_cache.go:296-300: the sequence comes into being
        VHC(create_seq_locked(m, seq_id));
        s = find_seq(m, seq_id);
    }
    if (insert_pos != s->seq_len)
        return fail("fragment \"%s\" can only go to the end of sequence %lld (length %d), not to position %d", name,
                    (long long)seq_id, s->seq_len, insert_pos);
    const Fragment &f = it->second;
    const int n = f.num_tokens, bs = m->pool.block_size;
    if ((insert_pos + n - 1) / bs + 1 > c.max_blocks_per_seq && n > 0)
        return fail("sequence %lld: %d tokens at position %d exceed max_blocks_per_seq %d", (long long)seq_id, n, insert_pos,
                    c.max_blocks_per_seq);
    const size_t blocks_before = s->table.size();
    // what the sequence gained goes back when a later step fails (the reference's InsertFragment has no failing step
    // after its allocation, paged_cache.go:302-314)
    auto roll_back = [&]() {
        while (s->table.size() > blocks_before) {
            m->pool.release_block(s->table.back());
            s->table.pop_back();
        }
        s->dirty = true;
    };
    if (m->pool.ensure_blocks(*s, insert_pos + n) != VH_OK) {
        roll_back();
        return VH_ERR;
    }
    if (n > 0) {
        std::vector<int32_t> slots(2 * (size_t)n);
        for (int t = 0; t < n; t++) {
            slots[t] = f.blocks[t / bs] * bs + t % bs;
            const int p = insert_pos + t;
            slots[n + t] = s->table[p / bs] * bs + p % bs;
        }
        // a buffer of its own, freed below: the per-step pool is only recycled by the next decode call
        int32_t *d_slots = (int32_t *)vx_alloc_permanent(m->be, slots.size() * 4);
        if (!d_slots) {
            roll_back();
            return fail("vx_alloc_permanent: %s", vx_last_error());
        }
        int rc = vx_to_device(m->be, d_slots, slots.data(), slots.size() * 4);
        // (the K rotation's table of angles is the same for every layer: the library keeps it from the first call)
        for (int l = 0; l < c.num_layers && rc == VX_OK; l++)
            rc = vx_paged_kv_copy_shifted(m->be, m->kv[l], c.kv_fp16, d_slots, d_slots + n, n, c.num_kv_heads, c.head_dim, bs,
                                          insert_pos, c.rope_theta);
        if (rc == VX_OK) rc = vx_sync(m->be);
        vx_free(m->be, d_slots);  // (drains the stream first)
        if (rc != VX_OK) {
            roll_back();
            return fail("fragment copy: %s", vx_last_error());
        }
    }
    s->seq_len = insert_pos + n;  // paged_cache.go:316-319
    s->dirty = true;
    if (num_tokens) *num_tokens = n;
    return VH_OK;
}

void vh_pool_block_stats(vh_model *m, int *total, int *free_blocks, int *shared) {  // gpu_block_pool.go:610-624
    std::lock_guard<std::mutex> g(m->pool.mu);
    int sh = 0;
    for (auto &kv : m->pool.ref_counts)
        if (kv.second > 1) sh++;
    if (total) *total = m->pool.max_blocks * m->cfg.num_layers;
    if (free_blocks) *free_blocks = (int)m->pool.free_list.size() * m->cfg.num_layers;
    if (shared) *shared = sh * m->cfg.num_layers;
}

int vh_pool_seq_len(vh_model *m, int64_t seq_id) {
    std::lock_guard<std::mutex> g(m->pool.mu);
    SeqState *s = find_seq(m, seq_id);
    return s ? s->seq_len : -1;
}

int vh_pool_block_table(vh_model *m, int64_t seq_id, int32_t *out, int cap) {
    std::lock_guard<std::mutex> g(m->pool.mu);
    SeqState *s = find_seq(m, seq_id);
    if (!s) return -1;
    int n = (int)s->table.size();
    for (int i = 0; i < n && i < cap; i++) out[i] = s->table[i];
    return n;
}

int vh_pool_adopt_blocks(vh_model *m, int64_t seq_id, const int32_t *blocks, int num_blocks, int seq_len) {
    std::lock_guard<std::mutex> g(m->pool.mu);
    SeqState *s = find_seq(m, seq_id);
    if (!s) return fail("sequence %lld not found", (long long)seq_id);
    if (!s->table.empty()) return fail("sequence %lld already owns blocks", (long long)seq_id);
    if (seq_len > num_blocks * m->pool.block_size || seq_len <= (num_blocks - 1) * m->pool.block_size)
        return fail("%d tokens do not fill exactly %d blocks", seq_len, num_blocks);
    BlockPool &p = m->pool;
    for (int i = 0; i < num_blocks; i++) {
        auto it = std::find(p.free_list.begin(), p.free_list.end(), blocks[i]);
        if (it == p.free_list.end()) return fail("block %d is not free", blocks[i]);
        p.free_list.erase(it);
        p.ref_counts[blocks[i]] = 1;
        s->table.push_back(blocks[i]);
    }
    p.free_dirty = true;
    s->dirty = true;
    s->seq_len = seq_len;
    return VH_OK;
}

int vh_pool_device_matches_host(vh_model *m) {
    std::lock_guard<std::mutex> g(m->pool.mu);
    const int mb = m->cfg.max_blocks_per_seq;
    if (vx_sync(m->be)) return -1;
    std::vector<int32_t> row(mb);
    for (auto &kv : m->pool.seqs) {
        SeqState &s = kv.second;
        if (s.dirty) continue;  // not pushed yet: nothing to compare
        int32_t nb = -1;
        if (vx_to_host(m->be, &nb, m->d_num_blocks + s.slot, 4)) return -1;
        if (nb != (int32_t)s.table.size()) return 0;
        if (nb > 0 && vx_to_host(m->be, row.data(), m->d_tables + (size_t)s.slot * mb, (size_t)nb * 4)) return -1;
        for (int i = 0; i < nb; i++)
            if (row[i] != s.table[i]) return 0;
    }
    if (!m->pool.free_dirty) {
        int32_t fc = -1;
        if (vx_to_host(m->be, &fc, m->d_free_count, 4)) return -1;
        if (fc != (int32_t)m->pool.free_list.size()) return 0;
        std::vector<int32_t> fl(fc > 0 ? fc : 1);
        if (fc > 0 && vx_to_host(m->be, fl.data(), m->d_free, (size_t)fc * 4)) return -1;
        for (int i = 0; i < fc; i++)
            if (fl[i] != m->pool.free_list[i]) return 0;
    }
    return 1;
}

// ------------------------------------------------------------------ decode (host-built metadata)
int vh_decode_batched(vh_model *m, const int32_t *tokens, const int64_t *seq_ids, const int32_t *positions, int batch,
                      float *logits_out, int32_t *argmax_out) {
    if (!m || !tokens || !seq_ids || !positions) return fail("null argument");
    if (batch == 0) return VH_OK;                                                    // decode.go:619-621
    if (batch < 0 || batch > m->cfg.max_batch) return fail("batch %d exceeds max_batch %d", batch, m->cfg.max_batch);
    VHC(check_ready(m));
    const vh_config &c = m->cfg;
    std::vector<int32_t> slots(batch), slot_map(batch), kv_lens(batch);
    int max_kv = 1;
    {
        std::lock_guard<std::mutex> g(m->pool.mu);
        for (int i = 0; i < batch; i++) {
            if (tokens[i] < 0 || tokens[i] >= c.vocab) return fail("token %d out of range", tokens[i]);
            if (!find_seq(m, seq_ids[i])) VHC(create_seq_locked(m, seq_ids[i]));       // decode.go:361-363
            SeqState *s = find_seq(m, seq_ids[i]);
            const int pos = positions[i];
            VHC(m->pool.ensure_blocks(*s, pos + 1));                                  // gpu_block_pool.go:234-245
            slot_map[i] = s->table[pos / c.block_size] * c.block_size + pos % c.block_size;  // :250-252
            if (pos + 1 > s->seq_len) s->seq_len = pos + 1;                           // :318-320
            kv_lens[i] = s->seq_len;                                                  // :354 (kvLen = seq.seqLen)
            slots[i] = s->slot;
            max_kv = std::max(max_kv, kv_lens[i]);
        }
        VHC(sync_pool_to_device(m));
    }
    vx_reset_pool(m->be);                                                            // decode.go:366-368
    VXC(vx_to_device(m->be, m->d_tokens, tokens, (size_t)batch * 4));                 // decode.go:389-395
    VXC(vx_to_device(m->be, m->d_slots, slots.data(), (size_t)batch * 4));
    bool at_end = true;  // every sequence decodes at its end: kv length = position + 1
    for (int i = 0; i < batch; i++) at_end = at_end && kv_lens[i] == positions[i] + 1;
    if (at_end) {
        // The blocks are there already (host pool, mirrored above), so the packing kernel allocates nothing and
        // only derives slots and lengths on the device, and leaves the attention's work list with them.
        VXC(vx_to_device(m->be, m->d_pos_in, positions, (size_t)batch * 4));
        VXC(vx_pack_batch(m->be, m->d_slots, m->d_pos_in, nullptr, batch, batch, m->d_tables, c.max_blocks_per_seq,
                          m->d_num_blocks, m->d_free, m->d_free_count, c.block_size, m->d_cu, m->d_token_pos,
                          m->d_slot_map, m->d_kv_lens, m->d_status));
    } else {
        VXC(vx_to_device(m->be, m->d_token_pos, positions, (size_t)batch * 4));
        VXC(vx_to_device(m->be, m->d_slot_map, slot_map.data(), (size_t)batch * 4));
        VXC(vx_to_device(m->be, m->d_kv_lens, kv_lens.data(), (size_t)batch * 4));
    }
    VHC(forward_decode(m, batch, max_kv));
    if (logits_out) VXC(vx_to_host(m->be, logits_out, m->logits, (size_t)batch * c.vocab * 4));
    if (argmax_out) VXC(vx_to_host(m->be, argmax_out, m->d_next, (size_t)batch * 4));
    VXC(vx_sync(m->be));                                                             // decode.go:651
    return VH_OK;
}

// Sampler.Sample (pkg/sampler/sampler.go:48-77) for the rows of the last decode step, on the device.
int vh_sample_last_logits(vh_model *m, int rows, const float *temperature, const int32_t *top_k, const float *top_p,
                          const float *uniform, int32_t *tokens_out) {
    if (!m || rows < 0 || !temperature || !top_k || !top_p || !uniform || !tokens_out) return fail("bad arguments");
    if (rows == 0) return VH_OK;
    if (rows > m->cfg.max_batch) return fail("%d rows exceed max_batch %d", rows, m->cfg.max_batch);
    vx_backend *be = m->be;
    float *d_t = (float *)vx_alloc(be, (size_t)rows * 4), *d_p = (float *)vx_alloc(be, (size_t)rows * 4);
    float *d_u = (float *)vx_alloc(be, (size_t)rows * 4);
    int32_t *d_k = (int32_t *)vx_alloc(be, (size_t)rows * 4), *d_out = (int32_t *)vx_alloc(be, (size_t)rows * 4);
    if (!d_t || !d_p || !d_u || !d_k || !d_out) return fail("sampling buffers: %s", vx_last_error());
    VXC(vx_to_device(be, d_t, temperature, (size_t)rows * 4));
    VXC(vx_to_device(be, d_k, top_k, (size_t)rows * 4));
    VXC(vx_to_device(be, d_p, top_p, (size_t)rows * 4));
    VXC(vx_to_device(be, d_u, uniform, (size_t)rows * 4));
    if (m->arch.final_softcap > 0.f)  // scheduler.go:772-773: the logits a request is sampled from are capped first
        for (int r = 0; r < rows; r++)
            if (temperature[r] > 0.f)
                VXC(vx_logit_softcap(be, m->logits + (size_t)r * m->cfg.vocab, m->cfg.vocab, m->arch.final_softcap));
    VXC(vx_sample_rows(be, m->logits, rows, m->cfg.vocab, d_t, d_k, d_p, d_u, d_out));
    VXC(vx_to_host(be, tokens_out, d_out, (size_t)rows * 4));
    VXC(vx_sync(be));
    return VH_OK;
}

// ------------------------------------------------------------------ prefill / verify of one sequence
int vh_prefill(vh_model *m, const int32_t *tokens, int n, int64_t seq_id, int start_pos, int all_logits,
               float *logits_out) {
    if (!m || !tokens || n <= 0 || start_pos < 0) return fail("bad arguments");
    VHC(check_ready(m));
    const vh_config &c = m->cfg;
    std::vector<int32_t> page(n), offs(n), kvl(n), table;
    int seq_len;
    {
        std::lock_guard<std::mutex> g(m->pool.mu);
        if (!find_seq(m, seq_id)) VHC(create_seq_locked(m, seq_id));
        SeqState *s = find_seq(m, seq_id);
        VHC(m->pool.ensure_blocks(*s, start_pos + n));
        for (int i = 0; i < n; i++) {
            const int pos = start_pos + i;
            page[i] = s->table[pos / c.block_size];
            offs[i] = pos % c.block_size;
            kvl[i] = start_pos + i + 1;                                               // block.go:884-887
        }
        if (start_pos + n > s->seq_len) s->seq_len = start_pos + n;
        seq_len = s->seq_len;
        table = s->table;
        VHC(sync_pool_to_device(m));
    }
    vx_backend *be = m->be;
    vx_reset_pool(be);
    const size_t qd = (size_t)c.num_heads * c.head_dim, kvd = (size_t)c.num_kv_heads * c.head_dim;
    auto fa = [&](size_t count) { return (float *)vx_alloc(be, count * 4); };
    auto ia = [&](size_t count) { return (int32_t *)vx_alloc(be, count * 4); };
    int32_t *d_tok = ia(n), *d_page = ia(n), *d_offs = ia(n), *d_kvl = ia(n), *d_bt = ia(table.size());
    float *x = fa((size_t)n * c.hidden), *norm = fa((size_t)n * c.hidden), *q = fa(n * qd), *k = fa(n * kvd);
    float *v = fa(n * kvd), *attn = fa(n * qd), *gate = fa((size_t)n * c.ffn), *up = fa((size_t)n * c.ffn);
    const int out_rows = all_logits ? n : 1;
    float *logits = fa((size_t)out_rows * c.vocab);
    if (!d_tok || !d_page || !d_offs || !d_kvl || !d_bt || !x || !norm || !q || !k || !v || !attn || !gate || !up || !logits)
        return fail("prefill buffers: %s", vx_last_error());
    VXC(vx_to_device(be, d_tok, tokens, (size_t)n * 4));
    VXC(vx_to_device(be, d_page, page.data(), (size_t)n * 4));
    VXC(vx_to_device(be, d_offs, offs.data(), (size_t)n * 4));
    VXC(vx_to_device(be, d_kvl, kvl.data(), (size_t)n * 4));
    VXC(vx_to_device(be, d_bt, table.data(), table.size() * 4));
    VXC(vx_embedding(be, d_tok, n, m->embedding, x, c.vocab, c.hidden));               // decode.go:1005-1010
    VHC(g_scale_embedding(m, x, n));                                                   // decode.go:1030
    const float scale = (float)(1.0 / sqrt((double)c.head_dim));
    // A later chunk reads every key from the pool (block.go:881-890), so its projections can take the decode step's
    // fused form: Q|K|V in one launch that rotates and stores K/V itself; the fused tail serves every chunk.
    const bool later = n > 1 && start_pos > 0;
    // The first chunk attends over its own rows as dense floats (block.go:891-895): the same fused projection block
    // leaves the rotated K and V rows in that form too, beside the pool store.
    const bool first = n > 1 && start_pos == 0;
    const bool tails_fusable = n > 1 && m->fused && (!m->general || m->fused_ok);
    int32_t *d_pos = nullptr, *d_slot = nullptr;
    if (later || first) {
        std::vector<int32_t> pos(n), slot(n);
        for (int i = 0; i < n; i++) {
            pos[i] = start_pos + i;
            slot[i] = page[i] * c.block_size + offs[i];
        }
        d_pos = ia(n), d_slot = ia(n);
        if (!d_pos || !d_slot) return fail("prefill buffers: %s", vx_last_error());
        VXC(vx_to_device(be, d_pos, pos.data(), (size_t)n * 4));
        VXC(vx_to_device(be, d_slot, slot.data(), (size_t)n * 4));
    }
    bool chained = false;  // the backend's prepared slot holds RMSNorm(x) * attn_norm of the layer about to run
    for (int l = 0; l < c.num_layers; l++) {
        const vh_layer_weights &w = m->layers[l];
        const bool attn_fused = later && attn_fusable(m, l);
        if (attn_fused) {
            const vh_layer_extras &e = m->extras[l];
            VXC(vx_decode_attn_qkv_ex(be, x, w.attn_norm, c.eps, chained ? 1 : 0, &w.wq, &w.wk, &w.wv, e.wq_bias, e.wk_bias,
                                      e.wv_bias, n, d_pos, d_slot, m->kv[l], c.kv_fp16, c.num_heads, c.num_kv_heads, c.head_dim,
                                      c.block_size, c.rope_theta, m->arch.rope_dim, m->arch.rope_neox, q));
            chained = false;
            VXC(vx_sdpa_paged_decode_multiquery(be, q, m->kv[l], c.kv_fp16, d_bt, attn, d_kvl, (int)table.size(),
                                                c.block_size, c.num_heads, c.num_kv_heads, c.head_dim, scale, n));
        } else if (first && attn_fusable(m, l)) {
            const vh_layer_extras &e = m->extras[l];
            VXC(vx_prefill_attn_qkv(be, x, w.attn_norm, c.eps, chained ? 1 : 0, &w.wq, &w.wk, &w.wv, e.wq_bias, e.wk_bias,
                                    e.wv_bias, n, d_pos, d_slot, m->kv[l], c.kv_fp16, c.num_heads, c.num_kv_heads, c.head_dim,
                                    c.block_size, c.rope_theta, m->arch.rope_dim, m->arch.rope_neox, q, k, v));
            chained = false;
            if (m->arch.attn_softcap > 0.f)                                               // block.go:891-892
                VXC(vx_sdpa_prefill_softcap(be, q, k, v, attn, n, c.num_heads, c.num_kv_heads, c.head_dim, scale,
                                            m->arch.attn_softcap));
            else                                                                           // block.go:893-895
                VXC(vx_sdpa_prefill(be, q, k, v, attn, n, c.num_heads, c.num_kv_heads, c.head_dim, scale));
        } else if (first && m->general && g_qkv_fusable(m, l, n)) {   // (a LayerNorm in front of the same fused projections)
            if (chained) return fail("internal: prepared activation handed to a general layer");
            VHC(g_qkv_store(m, l, x, norm, q, n, d_pos, d_slot, k, v));
            if (m->arch.attn_softcap > 0.f)
                VXC(vx_sdpa_prefill_softcap(be, q, k, v, attn, n, c.num_heads, c.num_kv_heads, c.head_dim, scale,
                                            m->arch.attn_softcap));
            else
                VXC(vx_sdpa_prefill(be, q, k, v, attn, n, c.num_heads, c.num_kv_heads, c.head_dim, scale));
        } else if (later && m->general && g_qkv_fusable(m, l, n)) {   // (a LayerNorm in front of the same fused projections)
            if (chained) return fail("internal: prepared activation handed to a general layer");
            VHC(g_qkv_store(m, l, x, norm, q, n, d_pos, d_slot));
            VXC(vx_sdpa_paged_decode_multiquery(be, q, m->kv[l], c.kv_fp16, d_bt, attn, d_kvl, (int)table.size(),
                                                c.block_size, c.num_heads, c.num_kv_heads, c.head_dim, scale, n));
        } else {
            if (chained) return fail("internal: prepared activation handed to an unfused layer");
            if (m->general) {
                VHC(g_qkv(m, l, x, norm, q, k, v, n));
            } else {
                bool prep;
                const vh_qweight *qkv[3] = {&w.wq, &w.wk, &w.wv};
                VHC(norm_for(m, x, w.attn_norm, norm, n, qkv, 3, &prep));
                VHC(mm(m, prep, norm, w.wq, q, nullptr, n));
                VHC(mm(m, prep, norm, w.wk, k, nullptr, n));
                VHC(mm(m, prep, norm, w.wv, v, nullptr, n));
            }
            VXC(vx_rope(be, q, k, c.head_dim, c.num_heads, c.num_kv_heads, n, start_pos, m->arch.rope_dim, c.rope_theta,
                        m->arch.rope_neox));                                               // block.go:858 (applyRoPE, :497-503)
            if (c.kv_fp16) {                                                               // gpu_block_pool.go:262-272
                VXC(vx_reshape_paged_kv_f16(be, k, m->kv[l], d_page, d_offs, n, c.num_kv_heads, c.head_dim, c.block_size, 0));
                VXC(vx_reshape_paged_kv_f16(be, v, m->kv[l], d_page, d_offs, n, c.num_kv_heads, c.head_dim, c.block_size, 1));
            } else {
                VXC(vx_reshape_paged_kv(be, k, m->kv[l], d_page, d_offs, n, c.num_kv_heads, c.head_dim, c.block_size, 0));
                VXC(vx_reshape_paged_kv(be, v, m->kv[l], d_page, d_offs, n, c.num_kv_heads, c.head_dim, c.block_size, 1));
            }
            if (n == 1) {                                                                  // block.go:866-874
                const int nb = (seq_len + c.block_size - 1) / c.block_size;
                const int til = seq_len - (nb - 1) * c.block_size;                        // gpu_block_pool.go:359-363
                if (c.kv_fp16)
                    VXC(vx_sdpa_paged_decode_f16(be, q, m->kv[l], d_bt, attn, nb, c.block_size, c.num_heads,
                                                 c.num_kv_heads, c.head_dim, scale, til));
                else
                    VXC(vx_sdpa_paged_decode(be, q, m->kv[l], d_bt, attn, nb, c.block_size, c.num_heads, c.num_kv_heads,
                                             c.head_dim, scale, til));
            } else if (start_pos > 0) {                                                    // block.go:881-890
                VXC(vx_sdpa_paged_decode_multiquery(be, q, m->kv[l], c.kv_fp16, d_bt, attn, d_kvl, (int)table.size(),
                                                    c.block_size, c.num_heads, c.num_kv_heads, c.head_dim, scale, n));
            } else if (m->arch.attn_softcap > 0.f) {                                       // block.go:891-892
                VXC(vx_sdpa_prefill_softcap(be, q, k, v, attn, n, c.num_heads, c.num_kv_heads, c.head_dim, scale,
                                            m->arch.attn_softcap));
            } else {                                                                       // block.go:893-895
                VXC(vx_sdpa_prefill(be, q, k, v, attn, n, c.num_heads, c.num_kv_heads, c.head_dim, scale));
            }
        }
        if (tails_fusable && w.wo.data && w.w1.data && w.w2.data && w.w3.data &&
            vx_decode_ffn_supported(&w.wo, &w.w1, &w.w3, &w.w2)) {                      // block.go:981-1077
            const float *next_norm = l + 1 < c.num_layers && (later || first) && attn_fusable(m, l + 1) ? m->layers[l + 1].attn_norm : nullptr;
            VXC(vx_decode_ffn(be, attn, x, &w.wo, w.ffn_norm, c.eps, &w.w1, &w.w3, &w.w2, n, next_norm));
            chained = next_norm != nullptr;
        } else if (m->general) {
            VHC(g_tail(m, l, x, norm, attn, gate, up, n));
        } else {
            VHC(layer_tail(m, w, x, norm, attn, gate, up, n));
        }
    }
    const float *last = all_logits ? x : x + (size_t)(n - 1) * c.hidden;                // decode.go:1057-1066
    if (m->general) {
        VHC(g_norm(m, last, m->final_norm, m->final_norm_bias, norm, out_rows));
        VHC(mm(m, false, norm, m->lm_head, logits, nullptr, out_rows));
    } else {
        bool prep;
        const vh_qweight *hw[1] = {&m->lm_head};
        VHC(norm_for(m, last, m->final_norm, norm, out_rows, hw, 1, &prep));
        VHC(mm(m, prep, norm, m->lm_head, logits, nullptr, out_rows));
    }
    if (logits_out) VXC(vx_to_host(be, logits_out, logits, (size_t)out_rows * c.vocab * 4));
    VXC(vx_sync(be));
    return VH_OK;
}

// ------------------------------------------------------------------ tree verification of a batch of sequences
int vh_verify_tree(vh_model *m, int n_seqs, const int64_t *seq_ids, const int32_t *input_tokens, const int32_t *start_pos,
                   const int32_t *n_nodes, const int32_t *node_tokens, const int32_t *parent_idx, int32_t *num_accepted,
                   int32_t *accepted_nodes, int32_t *final_tokens, float *logits_out) {
    if (!m || n_seqs < 0 || !seq_ids || !input_tokens || !start_pos || !n_nodes || !num_accepted || !final_tokens)
        return fail("bad arguments");
    if (n_seqs == 0) return VH_OK;
    VHC(check_ready(m));
    const vh_config &c = m->cfg;
    struct SeqRows { int row0, rows, node0, start, slot, pad; };
    std::vector<SeqRows> sr(n_seqs);
    int total = 0, nodes_total = 0, max_rows = 1;
    for (int i = 0; i < n_seqs; i++) {
        if (n_nodes[i] < 0 || start_pos[i] < 0) return fail("sequence %d: bad counts", i);
        max_rows = std::max(max_rows, 1 + n_nodes[i]);
    }
    // With the batched tree attention a sequence's rows fill whole entries of `rg` rows: the rows that pad the
    // last entry repeat the sequence's last row (same token, position and pool slot), their results are dropped.
    static const bool per_sequence = getenv("VEXEL_HIP_TREE_PER_SEQUENCE") != nullptr;
    const int rg0 = vx_sdpa_paged_tree_rows_per_entry(c.kv_fp16, c.block_size, c.num_heads, c.num_kv_heads, c.head_dim);
    int rg = (rg0 > 0 && max_rows <= 64 && max_rows <= c.head_dim && !per_sequence) ? rg0 : 0;
    if (rg && rg % 2 == 0) {  // entries of half as many rows where the full ones would add rows of padding (small trees)
        int full = 0, half = 0;
        for (int i = 0; i < n_seqs; i++) {
            const int rows = 1 + n_nodes[i];
            full += (rows + rg - 1) / rg * rg;
            half += (rows + rg / 2 - 1) / (rg / 2) * (rg / 2);
        }
        if (half < full) rg /= 2;
    }
    for (int i = 0; i < n_seqs; i++) {
        const int rows = 1 + n_nodes[i], pad = rg ? (rows + rg - 1) / rg * rg : rows;
        sr[i] = {total, rows, nodes_total, start_pos[i], -1, pad};
        total += pad;
        nodes_total += n_nodes[i];
    }
    if (nodes_total > 0 && (!node_tokens || !parent_idx || !accepted_nodes)) return fail("null node arrays");
    for (int i = 0; i < n_seqs; i++)
        for (int j = i + 1; j < n_seqs; j++)
            if (seq_ids[i] == seq_ids[j]) return fail("sequence %lld appears twice", (long long)seq_ids[i]);
    // rows: [input token, nodes] per sequence; row r of a sequence lives at pool position start + r and is rotated
    // at start + its depth; it sees the rows of its ancestors (tree.go:186-202) and everything before start
    std::vector<int32_t> tok(total), pos(total), slot_map(total);
    std::vector<uint8_t> mask;
    std::vector<size_t> mask_off(n_seqs);
    {
        std::lock_guard<std::mutex> g(m->pool.mu);
        for (int i = 0; i < n_seqs; i++) {
            const SeqRows &q = sr[i];
            if (input_tokens[i] < 0 || input_tokens[i] >= c.vocab) return fail("token %d out of range", input_tokens[i]);
            if (!find_seq(m, seq_ids[i])) VHC(create_seq_locked(m, seq_ids[i]));
            SeqState *s = find_seq(m, seq_ids[i]);
            if (s->seq_len != q.start)
                return fail("sequence %lld holds %d tokens, verification starts at %d", (long long)seq_ids[i], s->seq_len, q.start);
            VHC(m->pool.ensure_blocks(*s, q.start + q.rows));                               // gpu_block_pool.go:234-245
            if ((int)s->table.size() > c.max_blocks_per_seq)
                return fail("sequence %lld needs %zu blocks, the table holds %d", (long long)seq_ids[i], s->table.size(),
                            c.max_blocks_per_seq);
            mask_off[i] = mask.size();
            mask.resize(mask.size() + (size_t)q.rows * q.rows, 0);
            uint8_t *mk = mask.data() + mask_off[i];
            std::vector<int> depth(q.rows, 0);
            for (int r = 0; r < q.rows; r++) {
                int parent = -1;  // row index of the parent; the input token has none
                if (r > 0) {
                    const int node = r - 1, p = parent_idx[q.node0 + node];
                    if (p < -1 || p >= node) return fail("sequence %d: parent of node %d is %d", i, node, p);
                    const int t = node_tokens[q.node0 + node];
                    if (t < 0 || t >= c.vocab) return fail("token %d out of range", t);
                    tok[q.row0 + r] = t;
                    parent = p + 1;
                    depth[r] = depth[parent] + 1;
                    memcpy(mk + (size_t)r * q.rows, mk + (size_t)parent * q.rows, q.rows);  // the parent's ancestors
                } else {
                    tok[q.row0] = input_tokens[i];
                }
                mk[(size_t)r * q.rows + r] = 1;
                const int p = q.start + r;
                pos[q.row0 + r] = q.start + depth[r];
                slot_map[q.row0 + r] = s->table[p / c.block_size] * c.block_size + p % c.block_size;  // :250-252
            }
            for (int r = q.rows; r < q.pad; r++) {
                tok[q.row0 + r] = tok[q.row0 + q.rows - 1];
                pos[q.row0 + r] = pos[q.row0 + q.rows - 1];
                slot_map[q.row0 + r] = slot_map[q.row0 + q.rows - 1];
            }
            s->seq_len = q.start + q.rows;
            sr[i].slot = s->slot;
        }
        VHC(sync_pool_to_device(m));
    }
    vx_backend *be = m->be;
    vx_reset_pool(be);
    const int n = total;
    const size_t qd = (size_t)c.num_heads * c.head_dim, kvd = (size_t)c.num_kv_heads * c.head_dim;
    auto fa = [&](size_t count) { return (float *)vx_alloc(be, count * 4); };
    auto ia = [&](size_t count) { return (int32_t *)vx_alloc(be, count * 4); };
    int32_t *d_tok = ia(n), *d_pos = ia(n), *d_slot = ia(n), *d_am = ia(n);
    uint8_t *d_mask = (uint8_t *)vx_alloc(be, mask.size());
    float *x = fa((size_t)n * c.hidden), *norm = fa((size_t)n * c.hidden), *q = fa(n * qd), *k = fa(n * kvd);
    float *v = fa(n * kvd), *attn = fa(n * qd), *gate = fa((size_t)n * c.ffn), *up = fa((size_t)n * c.ffn);
    float *logits = fa((size_t)n * c.vocab);
    if (!d_tok || !d_pos || !d_slot || !d_am || !d_mask || !x || !norm || !q || !k || !v || !attn || !gate || !up || !logits)
        return fail("verification buffers: %s", vx_last_error());
    VXC(vx_to_device(be, d_tok, tok.data(), (size_t)n * 4));
    VXC(vx_to_device(be, d_pos, pos.data(), (size_t)n * 4));
    VXC(vx_to_device(be, d_slot, slot_map.data(), (size_t)n * 4));
    VXC(vx_to_device(be, d_mask, mask.data(), mask.size()));
    int32_t *d_ent_rows = nullptr, *d_ent_lens = nullptr, *d_info = nullptr, *d_moff = nullptr;
    int entries = 0, max_start = 0;
    if (rg) {
        std::vector<int32_t> ent_rows, ent_lens, info((size_t)n * 4), moff(n);
        for (int i = 0; i < n_seqs; i++) {
            const SeqRows &s = sr[i];
            max_start = std::max(max_start, s.start);
            for (int e = 0; e < s.pad / rg; e++) {
                ent_rows.push_back(s.slot);
                ent_lens.push_back(s.start);
            }
            for (int r = 0; r < s.pad; r++) {
                int32_t *f = &info[(size_t)(s.row0 + r) * 4];
                f[0] = s.slot, f[1] = s.start, f[2] = std::min(r, s.rows - 1), f[3] = s.rows;
                moff[s.row0 + r] = (int32_t)mask_off[i];
            }
        }
        entries = (int)ent_rows.size();
        d_ent_rows = ia(entries), d_ent_lens = ia(entries), d_info = ia((size_t)n * 4), d_moff = ia(n);
        if (!d_ent_rows || !d_ent_lens || !d_info || !d_moff) return fail("verification buffers: %s", vx_last_error());
        VXC(vx_to_device(be, d_ent_rows, ent_rows.data(), (size_t)entries * 4));
        VXC(vx_to_device(be, d_ent_lens, ent_lens.data(), (size_t)entries * 4));
        VXC(vx_to_device(be, d_info, info.data(), (size_t)n * 16));
        VXC(vx_to_device(be, d_moff, moff.data(), (size_t)n * 4));
    }
    VXC(vx_embedding(be, d_tok, n, m->embedding, x, c.vocab, c.hidden));
    VHC(g_scale_embedding(m, x, n));
    const float scale = (float)(1.0 / sqrt((double)c.head_dim));
    // the layers as in forward_decode: fused projection groups where the weights allow them, each fused tail
    // leaving the next norm's activation prepared; the other architectures' switches as in execute_layer_decode
    const bool tail_general = m->general && !m->fused_ok;
    const bool head_prepared = n > 1 && m->fused && !tail_general && fast(m->lm_head) && c.hidden % 256 == 0;
    bool chained = false;
    for (int l = 0; l < c.num_layers; l++) {
        const vh_layer_weights &w = m->layers[l];
        if (attn_fusable(m, l)) {
            const vh_layer_extras &e = m->extras[l];
            VXC(vx_decode_attn_qkv_ex(be, x, w.attn_norm, c.eps, chained ? 1 : 0, &w.wq, &w.wk, &w.wv, e.wq_bias, e.wk_bias,
                                      e.wv_bias, n, d_pos, d_slot, m->kv[l], c.kv_fp16, c.num_heads, c.num_kv_heads, c.head_dim,
                                      c.block_size, c.rope_theta, m->arch.rope_dim, m->arch.rope_neox, q));
        } else if (m->general) {
            if (chained) return fail("internal: prepared activation handed to a general layer");
            if (g_qkv_fusable(m, l, n)) {
                VHC(g_qkv_store(m, l, x, norm, q, n, d_pos, d_slot));
            } else {
                VHC(g_qkv(m, l, x, norm, q, k, v, n));
                VXC(vx_rope_store_paged_ex(be, q, k, v, d_pos, d_slot, m->kv[l], c.kv_fp16, n, c.num_heads, c.num_kv_heads,
                                           c.head_dim, c.block_size, c.rope_theta, m->arch.rope_dim, m->arch.rope_neox));
            }
        } else {
            if (chained) return fail("internal: prepared activation handed to an unfused layer");
            bool prep;
            const vh_qweight *qkv[3] = {&w.wq, &w.wk, &w.wv};
            VHC(norm_for(m, x, w.attn_norm, norm, n, qkv, 3, &prep));
            VHC(mm(m, prep, norm, w.wq, q, nullptr, n));
            VHC(mm(m, prep, norm, w.wk, k, nullptr, n));
            VHC(mm(m, prep, norm, w.wv, v, nullptr, n));
            VXC(vx_rope_store_paged(be, q, k, v, d_pos, d_slot, m->kv[l], c.kv_fp16, n, c.num_heads, c.num_kv_heads,
                                    c.head_dim, c.block_size, c.rope_theta));
        }
        if (rg) {  // every tree in two launches, each sequence's context read once per entry of rg rows
            VXC(vx_sdpa_paged_tree_batched(be, q, m->kv[l], m->d_tables, c.max_blocks_per_seq, d_ent_rows, d_ent_lens, entries,
                                           d_info, d_mask, d_moff, attn, n, max_rows, c.num_heads, c.num_kv_heads, c.head_dim,
                                           scale, max_start));
        } else {
            for (int i = 0; i < n_seqs; i++) {
                const SeqRows &s = sr[i];
                VXC(vx_sdpa_paged_tree(be, q + s.row0 * qd, m->kv[l], c.kv_fp16,
                                       m->d_tables + (size_t)s.slot * c.max_blocks_per_seq, attn + s.row0 * qd,
                                       d_mask + mask_off[i], s.start, c.block_size, c.num_heads, c.num_kv_heads, c.head_dim,
                                       scale, s.rows));
            }
        }
        chained = false;
        if (tail_general) {
            VHC(g_tail(m, l, x, norm, attn, gate, up, n));
            continue;
        }
        const bool ffn_fused = m->fused && n > 1 && w.wo.data && w.w1.data && w.w2.data && w.w3.data &&
                               vx_decode_ffn_supported(&w.wo, &w.w1, &w.w3, &w.w2);
        if (ffn_fused) {
            const float *next_norm = l + 1 < c.num_layers ? (attn_fusable(m, l + 1) ? m->layers[l + 1].attn_norm : nullptr)
                                                          : (head_prepared ? m->final_norm : nullptr);
            VXC(vx_decode_ffn(be, attn, x, &w.wo, w.ffn_norm, c.eps, &w.w1, &w.w3, &w.w2, n, next_norm));
            chained = next_norm != nullptr;
        } else {
            VHC(layer_tail(m, w, x, norm, attn, gate, up, n));
        }
    }
    if (chained) {
        VHC(mm(m, true, nullptr, m->lm_head, logits, nullptr, n));
    } else if (tail_general) {                                                            // model.go:207-226
        VHC(g_norm(m, x, m->final_norm, m->final_norm_bias, norm, n));
        VHC(mm(m, false, norm, m->lm_head, logits, nullptr, n));
    } else {
        bool prep;
        const vh_qweight *hw[1] = {&m->lm_head};
        VHC(norm_for(m, x, m->final_norm, norm, n, hw, 1, &prep));
        VHC(mm(m, prep, norm, m->lm_head, logits, nullptr, n));
    }
    VXC(vx_argmax_rows(be, logits, n, c.vocab, d_am));
    std::vector<int32_t> am(n);
    VXC(vx_to_host(be, am.data(), d_am, (size_t)n * 4));
    if (logits_out) {
        size_t out_row = 0;
        for (int i = 0; i < n_seqs; i++) {  // the real rows of each sequence
            VXC(vx_to_host(be, logits_out + out_row * c.vocab, logits + (size_t)sr[i].row0 * c.vocab,
                           (size_t)sr[i].rows * c.vocab * 4));
            out_row += sr[i].rows;
        }
    }
    VXC(vx_sync(be));

    // greedy acceptance per sequence, then the moves that make each accepted path contiguous
    std::vector<int32_t> chain_off(1, 0), src, dst;
    for (int i = 0; i < n_seqs; i++) {
        const SeqRows &s = sr[i];
        int cur = -1, want = am[s.row0], acc = 0;
        for (;;) {
            int next = -1;
            for (int node = cur + 1; node < s.rows - 1; node++)
                if (parent_idx[s.node0 + node] == cur && node_tokens[s.node0 + node] == want) {
                    next = node;
                    break;
                }
            if (next < 0) break;
            accepted_nodes[s.node0 + acc] = next;
            if (next != acc) {  // pool position start+1+next -> start+1+acc
                src.push_back(slot_map[s.row0 + 1 + next]);
                dst.push_back(slot_map[s.row0 + 1 + acc]);
            }
            acc++;
            cur = next;
            want = am[s.row0 + 1 + next];
        }
        num_accepted[i] = acc;
        final_tokens[i] = want;
        if ((int)src.size() > chain_off.back()) chain_off.push_back((int32_t)src.size());
    }
    if (!src.empty()) {
        const int chains = (int)chain_off.size() - 1;
        int32_t *d_co = ia(chain_off.size()), *d_src = ia(src.size()), *d_dst = ia(dst.size());
        if (!d_co || !d_src || !d_dst) return fail("verification buffers: %s", vx_last_error());
        VXC(vx_to_device(be, d_co, chain_off.data(), chain_off.size() * 4));
        VXC(vx_to_device(be, d_src, src.data(), src.size() * 4));
        VXC(vx_to_device(be, d_dst, dst.data(), dst.size() * 4));
        for (int l = 0; l < c.num_layers; l++)
            VXC(vx_paged_kv_move(be, m->kv[l], c.kv_fp16, d_co, d_src, d_dst, chains, c.num_kv_heads, c.head_dim,
                                 c.block_size));
        VXC(vx_sync(be));
    }
    for (int i = 0; i < n_seqs; i++)                                                       // medusa_scheduler.go:852-861
        VHC(vh_pool_truncate_sequence(m, seq_ids[i], sr[i].start + 1 + num_accepted[i]));
    return VH_OK;
}

// ------------------------------------------------------------------ device-driven greedy decode
// The device-driven steps allocate blocks on the device and cannot stop half way: the host, which knows every
// table and the free count, checks before the first launch that `steps` more tokens per sequence fit
// (gpu_block_pool.go:234-245 applied steps times), and fails without touching the device when they do not.
static int check_room(vh_model *m, const int64_t *seq_ids, const int32_t *positions, int batch, int steps) {
    const int bs = m->pool.block_size;
    long long need = 0;
    for (int i = 0; i < batch; i++) {
        const SeqState *s = find_seq(m, seq_ids[i]);
        const int blocks = (positions[i] + steps - 1) / bs + 1;  // blocks holding positions 0 .. positions[i] + steps - 1
        if (blocks > m->cfg.max_blocks_per_seq)
            return fail("sequence %lld: %d more tokens need %d blocks, max_blocks_per_seq is %d", (long long)seq_ids[i], steps,
                        blocks, m->cfg.max_blocks_per_seq);
        need += std::max(0, blocks - (int)s->table.size());
    }
    if (need > (long long)m->pool.free_list.size())
        return fail("%d more tokens for %d sequences need %lld free blocks, the pool has %zu", steps, batch, need,
                    m->pool.free_list.size());
    return VH_OK;
}

static int device_step(vh_model *m, int batch) {
    const vh_config &c = m->cfg;
    VXC(vx_pack_batch(m->be, m->d_slots, m->d_positions, nullptr, batch, batch, m->d_tables, c.max_blocks_per_seq,
                      m->d_num_blocks, m->d_free, m->d_free_count, c.block_size, m->d_cu, m->d_token_pos,
                      m->d_slot_map, m->d_kv_lens, m->d_status));
    VHC(forward_decode(m, batch, c.max_blocks_per_seq * c.block_size));
    VXC(vx_decode_advance(m->be, m->d_tokens, m->d_positions, m->d_next, m->d_log, m->d_step, batch));
    return VH_OK;
}

int vh_decode_graph(vh_model *m, const int32_t *first_tokens, const int64_t *seq_ids, const int32_t *positions,
                    int batch, int steps, int use_graph, int32_t *out_tokens, float *ms_per_step) {
    if (!m || batch <= 0 || steps <= 0) return fail("bad arguments");
    if (batch > m->cfg.max_batch) return fail("batch %d exceeds max_batch %d", batch, m->cfg.max_batch);
    VHC(check_ready(m));
    const vh_config &c = m->cfg;
    std::lock_guard<std::mutex> g(m->pool.mu);
    if (first_tokens) {
        if (!seq_ids || !positions) return fail("seq_ids / positions missing");
        std::vector<int32_t> slots(batch);
        for (int i = 0; i < batch; i++) {
            SeqState *s = find_seq(m, seq_ids[i]);
            if (!s) return fail("sequence %lld not found", (long long)seq_ids[i]);
            if (positions[i] != s->seq_len)
                return fail("sequence %lld: position %d is not its length %d", (long long)seq_ids[i], positions[i], s->seq_len);
            slots[i] = s->slot;
        }
        VHC(check_room(m, seq_ids, positions, batch, steps));
        VHC(sync_pool_to_device(m));
        VXC(vx_to_device(m->be, m->d_tokens, first_tokens, (size_t)batch * 4));
        VXC(vx_to_device(m->be, m->d_positions, positions, (size_t)batch * 4));
        VXC(vx_to_device(m->be, m->d_slots, slots.data(), (size_t)batch * 4));
        m->dev_seq_ids.assign(seq_ids, seq_ids + batch);
        m->dev_positions.assign(positions, positions + batch);
    } else {
        if ((int)m->dev_seq_ids.size() != batch) return fail("no batch of %d sequences is loaded on the device", batch);
        for (int i = 0; i < batch; i++)
            if (!find_seq(m, m->dev_seq_ids[i]))
                return fail("sequence %lld of the batch on the device was deleted; pass the batch again", (long long)m->dev_seq_ids[i]);
        VHC(check_room(m, m->dev_seq_ids.data(), m->dev_positions.data(), batch, steps));
        VHC(sync_pool_to_device(m));  // lifecycle events since the last call (no-op when nothing changed)
    }
    if (m->log_cap < steps) {
        if (m->d_log) vx_free(m->be, m->d_log);
        m->d_log = nullptr;
        VHC(dev_alloc(m, &m->d_log, (size_t)steps * c.max_batch));
        m->log_cap = steps;
        drop_graph(m);  // the graph holds the old log pointer
    }
    int32_t zero = 0;
    VXC(vx_to_device(m->be, m->d_step, &zero, 4));
    vx_reset_pool(m->be);
    int done = 0;
    // a recording holds the library's scratch addresses: once an eager call in between (a longer prefill, a tree
    // verification, a larger batch) has made one of them grow, it is stale
    if (use_graph && (!m->graph || m->graph_batch != batch || m->graph_scratch_gen != vx_scratch_generation(m->be))) {
        drop_graph(m);
        VHC(device_step(m, batch));  // eager: sizes the library scratch; it is step 0 of this call
        done = 1;
        VXC(vx_graph_begin_capture(m->be));
        int rc = device_step(m, batch);
        vx_graph *gr = nullptr;
        int rc2 = vx_graph_end_capture(m->be, &gr);
        if (rc != VH_OK) {
            if (gr) vx_graph_destroy(gr);
            return VH_ERR;
        }
        if (rc2 != VX_OK) return fail("graph capture: %s", vx_last_error());
        m->graph = gr;
        m->graph_batch = batch;
        m->graph_scratch_gen = vx_scratch_generation(m->be);
    }
    VXC(vx_timer_start(m->be));
    const int timed = steps - done;
    for (int s = done; s < steps; s++) {
        if (use_graph)
            VXC(vx_graph_launch(m->be, m->graph));
        else
            VHC(device_step(m, batch));
    }
    float ms = 0.f;
    VXC(vx_timer_stop_ms(m->be, &ms));
    if (ms_per_step) *ms_per_step = timed > 0 ? ms / timed : 0.f;
    int32_t status = 0;
    VXC(vx_to_host(m->be, &status, m->d_status, 4));
    if (status != 0) {
        // check_room() rules this out; should it happen all the same, the device tables are no longer the host's:
        // have the next call rebuild them
        for (auto &kv : m->pool.seqs) kv.second.dirty = true;
        m->pool.free_dirty = true;
        m->dev_seq_ids.clear();
        return fail("the block pool ran out of blocks during the device-driven steps");
    }
    std::vector<int32_t> log((size_t)steps * batch);
    VXC(vx_to_host(m->be, log.data(), m->d_log, log.size() * 4));
    if (out_tokens) memcpy(out_tokens, log.data(), log.size() * 4);
    // advance the host pool by the same rule, in the same order (step-major, batch order)
    for (int s = 0; s < steps; s++)
        for (int i = 0; i < batch; i++) {
            SeqState *st = find_seq(m, m->dev_seq_ids[i]);
            const int pos = m->dev_positions[i] + s;
            VHC(m->pool.ensure_blocks(*st, pos + 1));
            if (pos + 1 > st->seq_len) st->seq_len = pos + 1;
        }
    for (int i = 0; i < batch; i++) {
        m->dev_positions[i] += steps;
        find_seq(m, m->dev_seq_ids[i])->dirty = false;  // the device made the same allocations itself
    }
    m->pool.free_dirty = false;
    return VH_OK;
}

}  // extern "C"
