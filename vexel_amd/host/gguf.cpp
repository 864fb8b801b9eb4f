// GGUF reader and the loader rule that turns a checkpoint into a vh_model.
//
// The reader restates inference/pkg/gguf/gguf.go (header, metadata, tensor table, data offset, tensor sizes,
// the llama.* configuration keys) over a read-only mapping of the file; the loader follows
// inference/runtime/loader.go:28-212,275-288,596-600: projection matrices and the output head stay raw quantized
// blocks on the device, token_embd and the norm vectors become float32, a missing output.weight falls back to
// the embedding. Nothing here touches the GPU except vh_model_load_gguf.
#include <fcntl.h>
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <map>
#include <string>
#include <vector>

#include "vexel_host.h"

extern "C" void vh_set_error(const char *text);  // runtime.cpp: what vh_last_error() returns

namespace {

int gfail(const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    vh_set_error(buf);
    return VH_ERR;
}

// gguf.go:19-36
enum { MT_U8 = 0, MT_I8, MT_U16, MT_I16, MT_U32, MT_I32, MT_F32, MT_BOOL, MT_STRING, MT_ARRAY, MT_U64, MT_I64, MT_F64 };

struct Meta {
    uint32_t type = 0;
    uint64_t u = 0;  // unsigned types, bool
    int64_t i = 0;   // signed types
    double f = 0;    // float32 / float64 (a float32 is exact in a double)
    std::string s;
    uint32_t arr_type = 0;
    uint64_t arr_len = 0;
    std::vector<std::string> arr_s;  // string arrays keep their elements; numeric arrays only their length
};

struct Tensor {
    std::string name;
    int n_dims = 0;
    uint64_t dims[VH_GGUF_MAX_DIMS] = {0, 0, 0, 0};
    uint32_t type = 0;
    uint64_t offset = 0;
};

}  // namespace

struct vh_gguf {
    int fd = -1;
    const uint8_t *map = nullptr;
    size_t size = 0;
    uint32_t version = 0;
    std::map<std::string, Meta> meta;  // a repeated key keeps its last value, as the Go map does
    std::vector<std::string> keys;     // in file order, first occurrence
    std::vector<Tensor> tensors;
    int64_t data_offset = 0;
};

namespace {

struct Reader {
    const uint8_t *p;
    size_t size, pos = 0;
    bool ok = true;
    template <class T>
    T get() {
        T v{};
        if (!ok || size - pos < sizeof(T)) {
            ok = false;
            return v;
        }
        memcpy(&v, p + pos, sizeof(T));  // little endian, as the host
        pos += sizeof(T);
        return v;
    }
    bool str(std::string *out) {  // gguf.go:337-350
        const uint64_t n = get<uint64_t>();
        if (!ok || n > 65535 || size - pos < n) return ok = false;
        out->assign((const char *)p + pos, (size_t)n);
        pos += (size_t)n;
        return true;
    }
};

bool read_scalar(Reader &r, uint32_t type, Meta *v) {
    switch (type) {
    case MT_U8: v->u = r.get<uint8_t>(); break;
    case MT_I8: v->i = r.get<int8_t>(); break;
    case MT_U16: v->u = r.get<uint16_t>(); break;
    case MT_I16: v->i = r.get<int16_t>(); break;
    case MT_U32: v->u = r.get<uint32_t>(); break;
    case MT_I32: v->i = r.get<int32_t>(); break;
    case MT_U64: v->u = r.get<uint64_t>(); break;
    case MT_I64: v->i = r.get<int64_t>(); break;
    case MT_F32: v->f = r.get<float>(); break;
    case MT_F64: v->f = r.get<double>(); break;
    case MT_BOOL: v->u = r.get<uint8_t>() != 0; break;
    case MT_STRING: return r.str(&v->s);
    default: return false;
    }
    return r.ok;
}

// gguf.go:366-424. An array of arrays (which the reference reads as zero bytes per element and then loses its
// place in the file) is refused.
bool read_value(Reader &r, Meta *v) {
    v->type = r.get<uint32_t>();
    if (!r.ok) return false;
    if (v->type != MT_ARRAY) return read_scalar(r, v->type, v);
    v->arr_type = r.get<uint32_t>();
    v->arr_len = r.get<uint64_t>();
    if (!r.ok || v->arr_type == MT_ARRAY || v->arr_type > MT_F64) return false;
    for (uint64_t i = 0; i < v->arr_len; i++) {
        Meta e;
        if (!read_scalar(r, v->arr_type, &e)) return false;
        if (v->arr_type == MT_STRING) v->arr_s.push_back(e.s);
    }
    return true;
}

// gguf.go:94-106
uint64_t block_elems(uint32_t t) {
    switch (t) {
    case 0: case 1: case 30: return 1;
    case 2: case 3: case 6: case 7: case 8: case 9: return 32;
    case 12: case 13: case 14: return 256;
    }
    return 32;
}
// gguf.go:108-131
uint64_t block_bytes(uint32_t t) {
    switch (t) {
    case 0: return 4;
    case 1: case 30: return 2;
    case 2: return 18;
    case 6: return 22;
    case 7: return 24;
    case 8: return 34;
    case 12: return 144;
    case 13: return 176;
    case 14: return 210;
    }
    return 32;
}

uint64_t num_elements(const Tensor &t) {  // gguf.go:209-218
    if (t.n_dims == 0) return 0;
    uint64_t n = 1;
    for (int i = 0; i < t.n_dims; i++) n *= t.dims[i];
    return n;
}

const Meta *find_meta(const vh_gguf *g, const std::string &key) {
    auto it = g->meta.find(key);
    return it == g->meta.end() ? nullptr : &it->second;
}
// MetadataValue.AsUint32 / AsUint64 / AsFloat32 (gguf.go:158-199)
uint32_t as_u32(const Meta &m) {
    switch (m.type) {
    case MT_U32: case MT_U64: return (uint32_t)m.u;
    case MT_I32: return (uint32_t)m.i;
    }
    return 0;
}
uint64_t as_u64(const Meta &m) { return (m.type == MT_U64 || m.type == MT_U32) ? m.u : 0; }
float as_f32(const Meta &m) { return (m.type == MT_F32 || m.type == MT_F64) ? (float)m.f : 0.f; }

void fill_tensor(const vh_gguf *g, const Tensor &t, vh_gguf_tensor *out) {
    out->name = t.name.c_str();
    out->n_dims = t.n_dims;
    for (int i = 0; i < VH_GGUF_MAX_DIMS; i++) out->dims[i] = t.dims[i];
    out->type = t.type;
    out->offset = t.offset;
    const uint64_t be = block_elems(t.type);
    out->n_bytes = (num_elements(t) + be - 1) / be * block_bytes(t.type);  // gguf.go:600-604
    const uint64_t at = (uint64_t)g->data_offset + t.offset;
    out->data = (at <= g->size && out->n_bytes <= g->size - at) ? g->map + at : nullptr;
}

}  // namespace

extern "C" {

int vh_gguf_open(const char *path, vh_gguf **out) {
    if (!path || !out) return gfail("vh_gguf_open: null argument");
    *out = nullptr;
    const int fd = open(path, O_RDONLY);
    if (fd < 0) return gfail("failed to open file: %s", path);
    struct stat st;
    if (fstat(fd, &st) != 0 || st.st_size <= 0) {
        close(fd);
        return gfail("failed to stat %s (or the file is empty)", path);
    }
    void *map = mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
    if (map == MAP_FAILED) {
        close(fd);
        return gfail("failed to map %s", path);
    }
    vh_gguf *g = new vh_gguf;
    g->fd = fd;
    g->map = (const uint8_t *)map;
    g->size = (size_t)st.st_size;
    Reader r{g->map, g->size};
    auto bad = [&](const char *what) {
        vh_gguf_close(g);
        return gfail("%s: %s", path, what);
    };
    // gguf.go:278-335
    if (r.get<uint32_t>() != 0x46554747u || !r.ok) return bad("invalid magic");
    g->version = r.get<uint32_t>();
    if (!r.ok || g->version < 2 || g->version > 3) return bad("unsupported version");
    const uint64_t n_tensors = r.get<uint64_t>(), n_meta = r.get<uint64_t>();
    if (!r.ok) return bad("failed to read the counts");
    for (uint64_t i = 0; i < n_meta; i++) {
        std::string key;
        Meta v;
        if (!r.str(&key) || !read_value(r, &v)) return bad("failed to read metadata");
        if (!g->meta.count(key)) g->keys.push_back(key);
        g->meta[key] = v;
    }
    for (uint64_t i = 0; i < n_tensors; i++) {  // gguf.go:465-502
        Tensor t;
        if (!r.str(&t.name)) return bad("failed to read tensor info");
        const uint32_t nd = r.get<uint32_t>();
        if (!r.ok || nd > VH_GGUF_MAX_DIMS) return bad("failed to read tensor info (more than 4 dimensions?)");
        t.n_dims = (int)nd;
        for (uint32_t d = 0; d < nd; d++) t.dims[d] = r.get<uint64_t>();
        t.type = r.get<uint32_t>();
        t.offset = r.get<uint64_t>();
        if (!r.ok) return bad("failed to read tensor info");
        g->tensors.push_back(t);
    }
    uint64_t alignment = 32;
    if (const Meta *a = find_meta(g, "general.alignment")) alignment = as_u64(*a);
    if (alignment == 0) return bad("general.alignment is zero or not an unsigned integer");
    g->data_offset = (int64_t)(((uint64_t)r.pos + alignment - 1) / alignment * alignment);
    *out = g;
    return VH_OK;
}

void vh_gguf_close(vh_gguf *g) {
    if (!g) return;
    if (g->map) munmap((void *)g->map, g->size);
    if (g->fd >= 0) close(g->fd);
    delete g;
}

uint32_t vh_gguf_version(const vh_gguf *g) { return g ? g->version : 0; }
int64_t vh_gguf_data_offset(const vh_gguf *g) { return g ? g->data_offset : -1; }
int vh_gguf_num_tensors(const vh_gguf *g) { return g ? (int)g->tensors.size() : 0; }
int vh_gguf_num_metadata(const vh_gguf *g) { return g ? (int)g->keys.size() : 0; }
const char *vh_gguf_metadata_key(const vh_gguf *g, int i) {
    return (g && i >= 0 && i < (int)g->keys.size()) ? g->keys[i].c_str() : nullptr;
}

int vh_gguf_tensor_at(const vh_gguf *g, int i, vh_gguf_tensor *out) {
    if (!g || !out || i < 0 || i >= (int)g->tensors.size()) return gfail("vh_gguf_tensor_at: bad index");
    fill_tensor(g, g->tensors[i], out);
    return VH_OK;
}

int vh_gguf_find_tensor(const vh_gguf *g, const char *name, vh_gguf_tensor *out) {  // File.GetTensor: first match
    if (!g || !name || !out) return gfail("vh_gguf_find_tensor: null argument");
    for (const Tensor &t : g->tensors)
        if (t.name == name) {
            fill_tensor(g, t, out);
            return VH_OK;
        }
    return gfail("tensor not found: %s", name);
}

int vh_gguf_meta_type(const vh_gguf *g, const char *key) {
    const Meta *m = (g && key) ? find_meta(g, key) : nullptr;
    return m ? (int)m->type : -1;
}
uint32_t vh_gguf_meta_u32(const vh_gguf *g, const char *key) {
    const Meta *m = (g && key) ? find_meta(g, key) : nullptr;
    return m ? as_u32(*m) : 0;
}
uint64_t vh_gguf_meta_u64(const vh_gguf *g, const char *key) {
    const Meta *m = (g && key) ? find_meta(g, key) : nullptr;
    return m ? as_u64(*m) : 0;
}
float vh_gguf_meta_f32(const vh_gguf *g, const char *key) {
    const Meta *m = (g && key) ? find_meta(g, key) : nullptr;
    return m ? as_f32(*m) : 0.f;
}
const char *vh_gguf_meta_str(const vh_gguf *g, const char *key) {
    const Meta *m = (g && key) ? find_meta(g, key) : nullptr;
    return (m && m->type == MT_STRING) ? m->s.c_str() : nullptr;
}
int64_t vh_gguf_meta_array_len(const vh_gguf *g, const char *key) {
    const Meta *m = (g && key) ? find_meta(g, key) : nullptr;
    return (m && m->type == MT_ARRAY) ? (int64_t)m->arr_len : -1;
}

// File.extractModelConfig (gguf.go:504-582), the keys the LLaMA path uses.
int vh_gguf_get_config(const vh_gguf *g, vh_gguf_config *c) {
    if (!g || !c) return gfail("vh_gguf_get_config: null argument");
    memset(c, 0, sizeof *c);
    std::string arch;
    if (const Meta *m = find_meta(g, "general.architecture")) arch = m->s;
    snprintf(c->architecture, sizeof c->architecture, "%s", arch.c_str());
    const std::string prefix = (arch.empty() ? std::string("llama") : arch) + ".";
    auto u32 = [&](const char *k, int *dst) {
        if (const Meta *m = find_meta(g, prefix + k)) {
            *dst = (int)as_u32(*m);
            return true;
        }
        return false;
    };
    u32("block_count", &c->num_layers);
    u32("embedding_length", &c->hidden);
    u32("attention.head_count", &c->num_heads);
    if (!u32("attention.head_count_kv", &c->num_kv_heads)) c->num_kv_heads = c->num_heads;
    u32("feed_forward_length", &c->ffn);
    u32("context_length", &c->context_length);
    if (const Meta *m = find_meta(g, prefix + "rope.freq_base")) c->rope_theta = as_f32(*m);
    else c->rope_theta = 10000.0f;
    u32("rope.dimension_count", &c->rope_dim_count);
    if (const Meta *m = find_meta(g, prefix + "attention.layer_norm_rms_epsilon")) c->rms_eps = as_f32(*m);
    u32("attention.key_length", &c->head_dim);
    if (const Meta *m = find_meta(g, prefix + "attn_logit_softcapping")) c->attn_softcap = as_f32(*m);
    if (const Meta *m = find_meta(g, prefix + "final_logit_softcapping")) c->final_softcap = as_f32(*m);
    if (const Meta *m = find_meta(g, "tokenizer.ggml.tokens"))
        if (m->type == MT_ARRAY) c->vocab = (int)m->arr_len;
    return VH_OK;
}

// gguf.GetLayerTensorName (pkg/gguf/loader.go:121-228) for the tensors of a LLaMA-family block; any other name
// comes back unchanged, as there.
int vh_gguf_tensor_name(const char *hf_name, char *out, size_t cap) {
    if (!hf_name || !out || cap == 0) return gfail("vh_gguf_tensor_name: null argument");
    static const char *global[][2] = {{"model.embed_tokens.weight", "token_embd.weight"},
                                      {"lm_head.weight", "output.weight"},
                                      {"model.norm.weight", "output_norm.weight"},
                                      {"model.norm.bias", "output_norm.bias"}};
    static const char *suffix[][2] = {{"self_attn.q_proj.weight", "attn_q.weight"},
                                      {"self_attn.k_proj.weight", "attn_k.weight"},
                                      {"self_attn.v_proj.weight", "attn_v.weight"},
                                      {"self_attn.q_proj.bias", "attn_q.bias"},
                                      {"self_attn.k_proj.bias", "attn_k.bias"},
                                      {"self_attn.v_proj.bias", "attn_v.bias"},
                                      {"self_attn.o_proj.weight", "attn_output.weight"},
                                      {"self_attn.o_proj.bias", "attn_output.bias"},
                                      {"mlp.gate_proj.weight", "ffn_gate.weight"},
                                      {"mlp.up_proj.weight", "ffn_up.weight"},
                                      {"mlp.down_proj.weight", "ffn_down.weight"},
                                      {"input_layernorm.weight", "attn_norm.weight"},
                                      {"input_layernorm.bias", "attn_norm.bias"},
                                      {"post_attention_layernorm.weight", "ffn_norm.weight"},
                                      {"post_attention_layernorm.bias", "ffn_norm.bias"}};
    std::string res = hf_name;
    const std::string name = hf_name;
    if (name.rfind("model.layers.", 0) != 0) {
        for (auto &gm : global)
            if (name == gm[0]) res = gm[1];
    } else {
        const size_t idx0 = strlen("model.layers.");
        const size_t dot = name.find('.', idx0);
        if (dot != std::string::npos && dot + 1 < name.size()) {
            const std::string layer = name.substr(idx0, dot - idx0), rest = name.substr(dot + 1);
            for (auto &sm : suffix)
                if (rest == sm[0]) res = "blk." + layer + "." + sm[1];
        }
    }
    if (res.size() + 1 > cap) return gfail("vh_gguf_tensor_name: buffer too small");
    memcpy(out, res.c_str(), res.size() + 1);
    return VH_OK;
}

}  // extern "C"

// ------------------------------------------------------------------ the loader rule
namespace {

enum { T_F32 = 0, T_F16 = 1, T_Q4_0 = 2, T_Q5_0 = 6, T_Q8_0 = 8, T_Q4_K = 12, T_Q5_K = 13, T_Q6_K = 14, T_BF16 = 30 };

int quant_fmt(uint32_t type) {  // GGUF tensor type -> VX_* format of the quantized matmuls, 0 if it has none
    switch (type) {
    case T_Q4_0: return VX_Q4_0;
    case T_Q8_0: return VX_Q8_0;
    case T_Q4_K: return VX_Q4_K;
    case T_Q6_K: return VX_Q6_K;
    case T_Q5_0: return VX_Q5_0;
    case T_Q5_K: return VX_Q5_K;
    case T_BF16: return VX_BF16;
    }
    return 0;
}

int fmt_block(int fmt) { return fmt == VX_BF16 ? 1 : (fmt == VX_Q4_0 || fmt == VX_Q8_0 || fmt == VX_Q5_0) ? 32 : 256; }

float f16_to_f32(uint16_t h) {  // dequant.go:231-261
    const uint32_t sign = (uint32_t)(h >> 15) << 31;
    uint32_t exp = (h >> 10) & 0x1F, mant = h & 0x3FF, bits;
    if (exp == 0) {
        if (mant == 0) {
            bits = sign;
        } else {  // subnormal: normalise
            exp = 127 - 15 + 1;
            while ((mant & 0x400) == 0) {
                mant <<= 1;
                exp--;
            }
            bits = sign | (exp << 23) | ((mant & 0x3FF) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (mant << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (mant << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

struct Loader {
    vx_backend *be;
    vh_gguf *g;
    vh_model *m = nullptr;
    std::vector<void *> owned;

    int find(const std::string &name, vh_gguf_tensor *t) {
        if (vh_gguf_find_tensor(g, name.c_str(), t) != VH_OK) return VH_ERR;
        if (!t->data) return gfail("tensor %s lies outside the file", name.c_str());
        return VH_OK;
    }
    void *dev_copy(const void *src, size_t bytes) {
        // 16 spare bytes: the kernels read weights in aligned 16-byte pieces
        void *p = vx_alloc_permanent(be, (bytes + 15) / 16 * 16 + 16);
        if (!p) return nullptr;
        if (vx_to_device(be, p, src, bytes) != VX_OK) {
            vx_free(be, p);
            return nullptr;
        }
        owned.push_back(p);
        return p;
    }
    // Raw quantized matrix [n, k] (GGUF dims [k, n]) for the quantized matmuls (loader.go:79-186).
    int matrix(const std::string &name, int n, int k, vh_qweight *w) {
        vh_gguf_tensor t;
        if (find(name, &t)) return VH_ERR;
        if (t.n_dims != 2 || (int64_t)t.dims[0] != k || (int64_t)t.dims[1] != n)
            return gfail("%s: shape [%llu, %llu] does not match the configuration's [%d, %d]", name.c_str(),
                         (unsigned long long)t.dims[1], (unsigned long long)t.dims[0], n, k);
        const int fmt = quant_fmt(t.type);
        if (!fmt) return gfail("%s: tensor type %u has no quantized matmul here (Q4_0, Q8_0, Q4_K, Q6_K, Q5_0, Q5_K, BF16 do)", name.c_str(), t.type);
        void *p = dev_copy(t.data, (size_t)t.n_bytes);
        if (!p) return gfail("%s: device copy failed: %s", name.c_str(), vx_last_error());
        w->fmt = fmt;
        w->data = p;
        w->n = n;
        w->k = k;
        return VH_OK;
    }
    bool has(const std::string &name) {
        vh_gguf_tensor t;
        return vh_gguf_find_tensor(g, name.c_str(), &t) == VH_OK;
    }
    // as_f32 for a tensor that may be absent (*out stays NULL then)
    int opt_f32(const std::string &name, int64_t elems, const float **out) {
        *out = nullptr;
        return has(name) ? as_f32(name, elems, out) : (int)VH_OK;
    }
    // Any supported type as float32 on the device (loader.go:187-203: gguf.Dequantize at load).
    int as_f32(const std::string &name, int64_t elems, const float **out) {
        vh_gguf_tensor t;
        if (find(name, &t)) return VH_ERR;
        int64_t n = t.n_dims ? 1 : 0;
        for (int i = 0; i < t.n_dims; i++) n *= (int64_t)t.dims[i];
        if (n != elems) return gfail("%s: %lld elements, the configuration needs %lld", name.c_str(), (long long)n, (long long)elems);
        void *dst = nullptr;
        if (t.type == T_F32) {
            dst = dev_copy(t.data, (size_t)n * 4);
        } else if (t.type == T_F16) {
            std::vector<float> tmp((size_t)n);
            const uint16_t *h = (const uint16_t *)t.data;
            for (int64_t i = 0; i < n; i++) tmp[(size_t)i] = f16_to_f32(h[i]);
            dst = dev_copy(tmp.data(), (size_t)n * 4);
        } else if (const int fmt = quant_fmt(t.type)) {
            if (n % fmt_block(fmt) != 0) return gfail("%s: not a whole number of blocks", name.c_str());
            void *raw = vx_alloc_permanent(be, (size_t)t.n_bytes);
            dst = vx_alloc_permanent(be, (size_t)n * 4);
            bool ok = raw && dst && vx_to_device(be, raw, t.data, (size_t)t.n_bytes) == VX_OK &&
                      vx_dequantize(be, fmt, raw, (float *)dst, n) == VX_OK && vx_sync(be) == VX_OK;
            if (raw) vx_free(be, raw);
            if (!ok) {
                if (dst) vx_free(be, dst);
                dst = nullptr;
            } else {
                owned.push_back(dst);
            }
        } else {
            return gfail("%s: tensor type %u cannot be converted to float32 here", name.c_str(), t.type);
        }
        if (!dst) return gfail("%s: device copy failed: %s", name.c_str(), vx_last_error());
        *out = (const float *)dst;
        return VH_OK;
    }
};

}  // namespace

extern "C" int vh_model_load_gguf(vx_backend *be, const char *path, const vh_load_options *opt, vh_model **out) {
    if (!be || !path || !opt || !out) return gfail("vh_model_load_gguf: null argument");
    *out = nullptr;
    vh_gguf *g = nullptr;
    if (vh_gguf_open(path, &g) != VH_OK) return VH_ERR;
    Loader L{be, g};
    auto done = [&](int rc) {
        if (rc != VH_OK) {
            std::string keep = vh_last_error();
            for (void *p : L.owned) vx_free(be, p);
            if (L.m) vh_model_destroy(L.m);  // frees the adopted buffers
            vh_set_error(keep.c_str());
        }
        vh_gguf_close(g);
        return rc;
    };
    vh_gguf_config gc;
    vh_gguf_get_config(g, &gc);
    vh_gguf_tensor embd;
    if (L.find("token_embd.weight", &embd)) return done(VH_ERR);
    if (gc.num_layers <= 0 || gc.hidden <= 0 || gc.num_heads <= 0 || gc.ffn <= 0)
        return done(gfail("%s: block_count / embedding_length / head_count / feed_forward_length missing", path));
    vh_config c;
    memset(&c, 0, sizeof c);
    c.num_layers = gc.num_layers;
    c.hidden = gc.hidden;
    c.num_heads = gc.num_heads;
    c.num_kv_heads = gc.num_kv_heads;
    c.head_dim = gc.head_dim > 0 ? gc.head_dim : gc.hidden / gc.num_heads;  // config.go: explicit key_length wins
    c.ffn = gc.ffn;
    // the vocabulary is the embedding's row count; the tokenizer list, when present, must agree
    c.vocab = embd.n_dims == 2 ? (int)embd.dims[1] : 0;
    if (c.vocab <= 0 || (int64_t)embd.dims[0] != c.hidden) return done(gfail("token_embd.weight: unexpected shape"));
    if (gc.vocab > 0 && gc.vocab != c.vocab) return done(gfail("tokenizer lists %d tokens, token_embd has %d rows", gc.vocab, c.vocab));
    c.eps = gc.rms_eps > 0.f ? gc.rms_eps : 1e-5f;  // gguf.go:232: 0 = use the default
    c.rope_theta = gc.rope_theta;
    c.block_size = opt->block_size > 0 ? opt->block_size : 16;
    c.pool_blocks = opt->pool_blocks;
    c.max_seqs = opt->max_seqs;
    c.max_blocks_per_seq = opt->max_blocks_per_seq;
    c.max_batch = opt->max_batch;
    c.kv_fp16 = opt->kv_fp16;
    // ModelConfigFromGGUF (runtime/config.go:388-470): the architecture's switches
    const std::string archname = gc.architecture;
    vh_arch a;
    memset(&a, 0, sizeof a);
    bool qkv_bias = false, all_bias = false, fused_qkv = false, fused_gate_up = false;
    if (archname.empty() || archname == "llama" || archname == "mistral") {
    } else if (archname == "qwen2") {
        qkv_bias = true;
        a.rope_neox = 1;
    } else if (archname == "gemma" || archname == "gemma2") {
        a.mlp_type = VH_MLP_GEGLU;
        a.embedding_scale = (float)sqrt((double)c.hidden);
        if (archname == "gemma2") {
            a.post_norms = 1;
            a.attn_softcap = gc.attn_softcap != 0.f ? gc.attn_softcap : 50.0f;  // config.go:443-446
            a.final_softcap = gc.final_softcap;
        }
    } else if (archname == "phi" || archname == "phi2") {
        a.norm_type = VH_NORM_LAYER;
        a.mlp_type = VH_MLP_GELU;
        a.parallel_residual = 1;
        a.rope_neox = 1;
        all_bias = fused_qkv = true;
    } else if (archname == "phi3") {
        // config.go:419-424: RMSNorm, SwiGLU over a pre-fused gate+up tensor, serial residual, split RoPE pairs
        a.rope_neox = 1;
        fused_qkv = fused_gate_up = true;
    } else {
        return done(gfail("%s: architecture '%s' has no loader here (llama, mistral, qwen2, gemma, gemma2, phi, phi2, phi3 do)", path,
                          archname.c_str()));
    }
    if (gc.rope_dim_count < 0 || gc.rope_dim_count > c.head_dim || gc.rope_dim_count % 2 != 0)
        return done(gfail("rope.dimension_count %d invalid for heads of %d", gc.rope_dim_count, c.head_dim));
    a.rope_dim = gc.rope_dim_count == c.head_dim ? 0 : gc.rope_dim_count;  // config.go:487 (0 = the whole head)
    if (vh_model_create(be, &c, &L.m) != VH_OK) return done(VH_ERR);
    if (vh_model_set_architecture(L.m, &a) != VH_OK) return done(VH_ERR);
    auto adopt_all = [&]() {
        for (void *p : L.owned) vh_model_adopt_buffer(L.m, p);
        L.owned.clear();
    };
    const int qd = c.num_heads * c.head_dim, kvd = c.num_kv_heads * c.head_dim;
    for (int l = 0; l < c.num_layers; l++) {
        const std::string b = "blk." + std::to_string(l) + ".";
        vh_layer_weights w;
        vh_layer_extras e;
        memset(&w, 0, sizeof w);
        memset(&e, 0, sizeof e);
        int rc = L.as_f32(b + "attn_norm.weight", c.hidden, &w.attn_norm) || L.matrix(b + "attn_output.weight", c.hidden, qd, &w.wo) ||
                 L.matrix(b + "ffn_down.weight", c.hidden, c.ffn, &w.w2);
        if (!rc && fused_qkv) {
            // Phi's attn_qkv [q + 2 kv rows, hidden]: Wq, Wk, Wv are its row ranges, in place (loader.go:610-640, 1018-1060)
            vh_qweight all;
            memset(&all, 0, sizeof all);
            rc = L.matrix(b + "attn_qkv.weight", qd + 2 * kvd, c.hidden, &all);
            if (!rc) {
                vh_gguf_tensor t;
                L.find(b + "attn_qkv.weight", &t);
                const size_t row_bytes = (size_t)t.n_bytes / (size_t)(qd + 2 * kvd);
                const uint8_t *base = (const uint8_t *)all.data;
                w.wq = vh_qweight{all.fmt, base, qd, c.hidden};
                w.wk = vh_qweight{all.fmt, base + (size_t)qd * row_bytes, kvd, c.hidden};
                w.wv = vh_qweight{all.fmt, base + (size_t)(qd + kvd) * row_bytes, kvd, c.hidden};
                const float *bias = nullptr;
                rc = L.opt_f32(b + "attn_qkv.bias", qd + 2 * kvd, &bias);
                if (!rc && bias) e.wq_bias = bias, e.wk_bias = bias + qd, e.wv_bias = bias + qd + kvd;
            }
        } else if (!rc) {
            rc = L.matrix(b + "attn_q.weight", qd, c.hidden, &w.wq) || L.matrix(b + "attn_k.weight", kvd, c.hidden, &w.wk) ||
                 L.matrix(b + "attn_v.weight", kvd, c.hidden, &w.wv);
            if (!rc && (qkv_bias || all_bias))
                rc = L.opt_f32(b + "attn_q.bias", qd, &e.wq_bias) || L.opt_f32(b + "attn_k.bias", kvd, &e.wk_bias) ||
                     L.opt_f32(b + "attn_v.bias", kvd, &e.wv_bias);
        }
        if (!rc && a.mlp_type == VH_MLP_GELU) {  // fc1 = ffn_up, fc2 = ffn_down (pkg/gguf/loader.go:190-198)
            rc = L.matrix(b + "ffn_up.weight", c.ffn, c.hidden, &w.w1);
        } else if (!rc && fused_gate_up) {
            // Phi-3's gate+up matrix [2 ffn rows, hidden], gate rows first: W1 and W3 are its halves, in place
            // (splitGateUpWeight, loader.go:1147-1218, which the reference reaches under the tensor's safetensors
            // name mlp.gate_up_proj; GGUF files of the architecture carry it as ffn_up)
            vh_qweight both;
            memset(&both, 0, sizeof both);
            rc = L.matrix(b + "ffn_up.weight", 2 * c.ffn, c.hidden, &both);
            if (!rc) {
                vh_gguf_tensor t;
                L.find(b + "ffn_up.weight", &t);
                const size_t row_bytes = (size_t)t.n_bytes / (size_t)(2 * c.ffn);
                const uint8_t *base = (const uint8_t *)both.data;
                w.w1 = vh_qweight{both.fmt, base, c.ffn, c.hidden};
                w.w3 = vh_qweight{both.fmt, base + (size_t)c.ffn * row_bytes, c.ffn, c.hidden};
            }
        } else if (!rc) {
            rc = L.matrix(b + "ffn_gate.weight", c.ffn, c.hidden, &w.w1) || L.matrix(b + "ffn_up.weight", c.ffn, c.hidden, &w.w3);
        }
        if (!rc && !a.parallel_residual) rc = L.as_f32(b + "ffn_norm.weight", c.hidden, &w.ffn_norm);
        if (!rc && all_bias)
            rc = L.opt_f32(b + "attn_norm.bias", c.hidden, &e.attn_norm_bias) || L.opt_f32(b + "attn_output.bias", c.hidden, &e.wo_bias) ||
                 L.opt_f32(b + "ffn_up.bias", c.ffn, &e.w1_bias) || L.opt_f32(b + "ffn_down.bias", c.hidden, &e.w2_bias) ||
                 (a.parallel_residual ? (int)VH_OK : L.opt_f32(b + "ffn_norm.bias", c.hidden, &e.ffn_norm_bias));
        if (!rc && a.post_norms)  // loader.go:366-371
            rc = L.as_f32(b + "post_attention_norm.weight", c.hidden, &e.post_attn_norm) ||
                 L.as_f32(b + "post_ffw_norm.weight", c.hidden, &e.post_ffn_norm);
        adopt_all();
        if (rc) return done(VH_ERR);
        if (vh_model_set_layer(L.m, l, &w) != VH_OK || vh_model_set_layer_extras(L.m, l, &e) != VH_OK) return done(VH_ERR);
    }
    if (a.norm_type == VH_NORM_LAYER) {  // model.norm.bias (pkg/gguf/loader.go:126)
        const float *fb = nullptr;
        const int rc = L.opt_f32("output_norm.bias", c.hidden, &fb);
        adopt_all();
        if (rc) return done(VH_ERR);
        if (fb && vh_model_set_final_norm_bias(L.m, fb) != VH_OK) return done(VH_ERR);
    }
    const float *embedding = nullptr, *final_norm = nullptr;
    if (L.as_f32("token_embd.weight", (int64_t)c.vocab * c.hidden, &embedding) || L.as_f32("output_norm.weight", c.hidden, &final_norm)) {
        adopt_all();
        return done(VH_ERR);
    }
    vh_qweight head;
    memset(&head, 0, sizeof head);
    vh_gguf_tensor ot;
    const bool has_out = vh_gguf_find_tensor(g, "output.weight", &ot) == VH_OK;
    const vh_gguf_tensor &src = has_out ? ot : embd;  // weight tying: loader.go:596-600
    int rc = VH_OK;
    if (quant_fmt(src.type)) {
        rc = L.matrix(has_out ? "output.weight" : "token_embd.weight", c.vocab, c.hidden, &head);
    } else if (!has_out) {
        head.fmt = VH_F32;  // the float32 embedding itself
        head.data = embedding;
        head.n = c.vocab;
        head.k = c.hidden;
    } else {
        const float *hf = nullptr;
        rc = L.as_f32("output.weight", (int64_t)c.vocab * c.hidden, &hf);
        head.fmt = VH_F32;
        head.data = hf;
        head.n = c.vocab;
        head.k = c.hidden;
    }
    adopt_all();
    if (rc) return done(VH_ERR);
    if (vh_model_set_head(L.m, embedding, final_norm, &head) != VH_OK) return done(VH_ERR);
    *out = L.m;
    L.m = nullptr;
    vh_gguf_close(g);
    return VH_OK;
}
