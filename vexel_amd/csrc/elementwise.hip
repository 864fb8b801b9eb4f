// Elementwise, normalisation, embedding, argmax, dequantisation and dense F32 matmul
// kernels. Each entry point cites the Go method it replaces (include/vexel_hip.h).
//
// Arithmetic notes: where the reference CPU backend goes through float64 (sqrt, exp,
// pow, cos, sin: backend/cpu/cpu.go:214,256-260,397,508) these kernels do the same in
// double on the device, so the only differences from the CPU result are float32
// summation order in reductions. Dequantisation is bit-exact: its products are written
// with explicit round-to-nearest intrinsics so no multiply-add is fused.
#include <float.h>

#include "common.h"

using namespace vx;

namespace {

constexpr int kThreads = 256;

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

// Block-wide sum for blockDim.x == kThreads; every thread gets the result.
__device__ __forceinline__ float block_sum(float v, float *sm) {
    v = wave_sum(v);
    int w = threadIdx.x >> 6, l = threadIdx.x & 63;
    __syncthreads();
    if (l == 0) sm[w] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < (int)(blockDim.x >> 6); i++) t += sm[i];
    return t;
}

__device__ __forceinline__ float block_max(float v, float *sm) {
    v = wave_max(v);
    int w = threadIdx.x >> 6, l = threadIdx.x & 63;
    __syncthreads();
    if (l == 0) sm[w] = v;
    __syncthreads();
    float t = sm[0];
    for (int i = 1; i < (int)(blockDim.x >> 6); i++) t = fmaxf(t, sm[i]);
    return t;
}

// ---------------------------------------------------------------- RMSNorm (cpu.go:200-220)
__global__ void __launch_bounds__(kThreads) rmsnorm_kernel(const float *x, const float *w, float *out, int cols,
                                                           float eps) {
    __shared__ float sm[kThreads / 64];
    const float *xr = x + (size_t)blockIdx.x * cols;
    float *orow = out + (size_t)blockIdx.x * cols;
    float ss = 0.f;
    for (int j = threadIdx.x; j < cols; j += kThreads) {
        float v = xr[j];
        ss += v * v;
    }
    ss = block_sum(ss, sm);
    float mean = ss / (float)cols;
    float rms = (float)sqrt((double)(mean + eps));
    for (int j = threadIdx.x; j < cols; j += kThreads) orow[j] = (xr[j] / rms) * w[j];
}

// ---------------------------------------------------------------- RoPE (cpu.go:226-303)
struct RopeCS {
    float c, s;
};

__device__ __forceinline__ RopeCS rope_cs(int pos, int j, int eff_dim, float theta) {
    double ex = (double)(2 * j) / (double)eff_dim;
    float freq = (float)(1.0 / pow((double)theta, ex));
    float angle = __fmul_rn((float)pos, freq);
    RopeCS r;
    r.c = (float)cos((double)angle);
    r.s = (float)sin((double)angle);
    return r;
}

__device__ __forceinline__ void rope_pair(float &a, float &b, RopeCS cs) {
    float v1 = a, v2 = b;
    a = __fsub_rn(__fmul_rn(v1, cs.c), __fmul_rn(v2, cs.s));
    b = __fadd_rn(__fmul_rn(v1, cs.s), __fmul_rn(v2, cs.c));
}

// grid.x = seq row, threads over rotation pairs j.
__global__ void rope_kernel(float *q, float *k, int head_dim, int num_heads, int num_kv_heads, int start_pos,
                            int eff_dim, float theta, int neox, const int32_t *positions, int row_step) {
    int row = blockIdx.x;
    int half = eff_dim / 2;
    int pos = positions ? positions[row] : start_pos + row * row_step;  // row_step 0: one position for every row
    for (int j = threadIdx.x; j < half; j += blockDim.x) {
        RopeCS cs = rope_cs(pos, j, eff_dim, theta);
        int i0 = neox ? j : 2 * j;
        int i1 = neox ? j + half : 2 * j + 1;
        float *qr = q + (size_t)row * num_heads * head_dim;
        for (int h = 0; h < num_heads; h++) rope_pair(qr[h * head_dim + i0], qr[h * head_dim + i1], cs);
        if (k) {
            float *kr = k + (size_t)row * num_kv_heads * head_dim;
            for (int h = 0; h < num_kv_heads; h++) rope_pair(kr[h * head_dim + i0], kr[h * head_dim + i1], cs);
        }
    }
}

// RoPE + paged scatter of K and V. The first eff_dim dimensions of a head turn, in pairs (2j, 2j+1) or, neox,
// (j, j + eff_dim/2); the rest is copied. Thread j of a head handles rotation pair j, or past the rotated part the
// two elements eff_dim + 2(j - eff_dim/2) and the one after: head_dim/2 threads cover the head either way.
template <bool F16>
__global__ void rope_store_paged_kernel(float *q, const float *k, const float *v, const int32_t *positions,
                                        const int32_t *slot_mapping, void *pool, int num_q_heads, int num_kv_heads,
                                        int head_dim, int block_size, float theta, int eff_dim, int neox) {
    // grid = (rows, head groups); thread = (pair j, head lane); heads are strided over
    // head lanes and head groups so the float64 cos/sin of a pair is computed once per thread.
    int row = blockIdx.x;
    int half = head_dim / 2, he = eff_dim / 2;
    int pos = positions[row];
    int slot = slot_mapping[row];
    int blk = slot / block_size, off = slot % block_size;
    size_t hs = (size_t)num_kv_heads * head_dim;
    size_t part = (size_t)block_size * hs;
    size_t kbase = (size_t)blk * 2 * part + (size_t)off * hs;
    size_t vbase = kbase + part;
    const int lanes = blockDim.x / half;              // head lanes per block (>= 1)
    const int hl = threadIdx.x / half;
    const int hstride = lanes * gridDim.y;
    const int h0 = blockIdx.y * lanes + hl;
    for (int j = threadIdx.x % half; j < half && hl < lanes; j += half) {
        const bool turn = j < he;
        const int i0 = turn ? (neox ? j : 2 * j) : eff_dim + 2 * (j - he);
        const int i1 = turn ? (neox ? j + he : 2 * j + 1) : i0 + 1;
        RopeCS cs = {1.f, 0.f};
        if (turn) cs = rope_cs(pos, j, eff_dim, theta);
        float *qr = q + (size_t)row * num_q_heads * head_dim;
        if (turn)
            for (int h = h0; h < num_q_heads; h += hstride) rope_pair(qr[h * head_dim + i0], qr[h * head_dim + i1], cs);
        const float *kr = k + (size_t)row * hs;
        const float *vr = v + (size_t)row * hs;
        for (int h = h0; h < num_kv_heads; h += hstride) {
            float a = kr[h * head_dim + i0], b = kr[h * head_dim + i1];
            if (turn) rope_pair(a, b, cs);
            float va = vr[h * head_dim + i0], vb = vr[h * head_dim + i1];
            size_t o0 = (size_t)h * head_dim + i0, o1 = (size_t)h * head_dim + i1;
            if (F16) {
                _Float16 *p = (_Float16 *)pool;
                p[kbase + o0] = (_Float16)a;
                p[kbase + o1] = (_Float16)b;
                p[vbase + o0] = (_Float16)va;
                p[vbase + o1] = (_Float16)vb;
            } else {
                float *p = (float *)pool;
                p[kbase + o0] = a;
                p[kbase + o1] = b;
                p[vbase + o0] = va;
                p[vbase + o1] = vb;
            }
        }
    }
}

// ---------------------------------------------------------------- SiLU / SiLUMul / Add / Mul
__device__ __forceinline__ float sigmoid_ref(float v) {  // cpu.go:384,397
    return 1.0f / (1.0f + (float)exp((double)(-v)));
}

__global__ void silu_kernel(const float *x, float *out, int n) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = __fmul_rn(x[i], sigmoid_ref(x[i]));
}

__global__ void silu_mul_kernel(const float *g, const float *u, float *out, int n) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = __fmul_rn(__fmul_rn(g[i], sigmoid_ref(g[i])), u[i]);
}

__global__ void add_kernel(const float *a, const float *b, float *out, int n) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = a[i] + b[i];
}

__global__ void mul_kernel(const float *a, const float *b, float *out, int n) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = a[i] * b[i];
}

// ---------------------------------------------------------------- LayerNorm (cpu.go:404-436)
__global__ void __launch_bounds__(kThreads) layernorm_kernel(const float *x, const float *w, const float *b, float *out,
                                                             int cols, float eps) {
    __shared__ float sm[kThreads / 64];
    const float *xr = x + (size_t)blockIdx.x * cols;
    float *orow = out + (size_t)blockIdx.x * cols;
    float s = 0.f;
    for (int j = threadIdx.x; j < cols; j += kThreads) s += xr[j];
    const float mean = block_sum(s, sm) / (float)cols;
    float vs = 0.f;
    for (int j = threadIdx.x; j < cols; j += kThreads) {
        const float d = xr[j] - mean;
        vs = fmaf(d, d, vs);
    }
    const float variance = block_sum(vs, sm) / (float)cols;
    const float inv_std = 1.0f / (float)sqrt((double)(variance + eps));
    for (int j = threadIdx.x; j < cols; j += kThreads) orow[j] = (xr[j] - mean) * inv_std * w[j] + b[j];
}

// ---------------------------------------------------------------- GELU, tanh form (cpu.go:440-473)
__device__ __forceinline__ float gelu_ref(float v) {
    // plain operators under contract(off): v + 0.044715 x^3 stays a product and a sum as in the reference (the
    // __f*_rn helpers are ordinary inline functions whose operations the compiler still fuses)
#pragma clang fp contract(off)
    const float x3 = v * v * v;
    const float arg = 0.7978845608f * (v + 0.044715f * x3);
    const float th = (float)tanh((double)arg);
    return 0.5f * v * (1.0f + th);
}

__global__ void gelu_kernel(const float *x, float *out, int n) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = gelu_ref(x[i]);
}

__global__ void gelu_mul_kernel(const float *g, const float *u, float *out, int n) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = __fmul_rn(gelu_ref(g[i]), u[i]);
}

// cpu.go:476-487: out[r][c] = x[r][c] + bias[c]; n = rows * cols
__global__ void add_bias_kernel(const float *x, const float *bias, float *out, int cols, int n) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = x[i] + bias[i % cols];
}

// cpu.go:558-563
__global__ void scale_kernel(float *buf, float scale, int n) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) buf[i] = __fmul_rn(buf[i], scale);
}

// model.go:336-350: float32(float64(cap) * tanh(float64(x) / cap)) with the quotient as a product by 1 / float64(cap)
__global__ void logit_softcap_kernel(float *x, double cap, double inv_cap, int n) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] = (float)(cap * tanh((double)x[i] * inv_cap));
}

// cpu.go:308-375: RoPE over the whole head, pair j turning by position * freqs[j]. grid.x = row.
__global__ void rope_freqs_kernel(float *q, float *k, const float *freqs, int head_dim, int num_heads, int num_kv_heads,
                                  int start_pos, int neox) {
    const int row = blockIdx.x, half = head_dim / 2;
    const int pos = start_pos + row;
    for (int j = threadIdx.x; j < half; j += blockDim.x) {
        const float angle = __fmul_rn((float)pos, freqs[j]);
        RopeCS cs;
        cs.c = (float)cos((double)angle);
        cs.s = (float)sin((double)angle);
        const int i0 = neox ? j : 2 * j, i1 = neox ? j + half : 2 * j + 1;
        float *qr = q + (size_t)row * num_heads * head_dim;
        for (int h = 0; h < num_heads; h++) rope_pair(qr[h * head_dim + i0], qr[h * head_dim + i1], cs);
        if (k) {
            float *kr = k + (size_t)row * num_kv_heads * head_dim;
            for (int h = 0; h < num_kv_heads; h++) rope_pair(kr[h * head_dim + i0], kr[h * head_dim + i1], cs);
        }
    }
}

// ---------------------------------------------------------------- Softmax (cpu.go:490-518)
__global__ void __launch_bounds__(kThreads) softmax_kernel(const float *x, float *out, int cols) {
    __shared__ float sm[kThreads / 64];
    const float *xr = x + (size_t)blockIdx.x * cols;
    float *orow = out + (size_t)blockIdx.x * cols;
    float mx = -INFINITY;
    for (int j = threadIdx.x; j < cols; j += kThreads) mx = fmaxf(mx, xr[j]);
    mx = block_max(mx, sm);
    float s = 0.f;
    for (int j = threadIdx.x; j < cols; j += kThreads) {
        float e = (float)exp((double)(xr[j] - mx));
        orow[j] = e;
        s += e;
    }
    s = block_sum(s, sm);
    float inv = 1.0f / s;
    for (int j = threadIdx.x; j < cols; j += kThreads) orow[j] *= inv;
}

// ---------------------------------------------------------------- Embedding (cpu.go:543-555)
__global__ void embedding_kernel(const int32_t *ids, const float *table, float *out, int vocab, int dim) {
    int t = blockIdx.x;
    int id = ids[t];
    if (id < 0 || id >= vocab) return;  // row left untouched
    const float *src = table + (size_t)id * dim;
    float *dst = out + (size_t)t * dim;
    for (int j = threadIdx.x; j < dim; j += blockDim.x) dst[j] = src[j];
}

// ---------------------------------------------------------------- Argmax (sampler.go:80-91)
// One block per row. Strict '>' from -FLT_MAX; ties resolve to the lowest index; NaN never wins.
__global__ void __launch_bounds__(1024) argmax_rows_kernel(const float *x, int n, int32_t *out) {
    __shared__ float sv[16];
    __shared__ int si[16];
    const float *xr = x + (size_t)blockIdx.x * n;
    float bv = -FLT_MAX;
    int bi = 0;
    if (((uintptr_t)xr % 16) == 0 && n % 4 == 0) {
        // four pieces of four columns in flight per thread (the comparisons form a chain; the loads need not wait for
        // it), a thread's columns in rising order, so that its first maximum is the one with the lowest index
        const int n4 = n / 4, step = (int)blockDim.x;
        for (int j0 = threadIdx.x; j0 < n4; j0 += 4 * step) {
            float4 v[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int j = j0 + u * step;
                v[u] = j < n4 ? ((const float4 *)xr)[j] : make_float4(-FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX);
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int j = 4 * (j0 + u * step);
                const float e[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (e[i] > bv) {
                        bv = e[i];
                        bi = j + i;
                    }
            }
        }
    } else {
        for (int j = threadIdx.x; j < n; j += blockDim.x) {
            float v = xr[j];
            if (v > bv) {
                bv = v;
                bi = j;
            }
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        float ov = __shfl_xor(bv, off, 64);
        int oi = __shfl_xor(bi, off, 64);
        if (ov > bv || (ov == bv && oi < bi)) {
            bv = ov;
            bi = oi;
        }
    }
    int w = threadIdx.x >> 6, l = threadIdx.x & 63;
    if (l == 0) {
        sv[w] = bv;
        si[w] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int i = 1; i < (int)(blockDim.x >> 6); i++)
            if (sv[i] > bv || (sv[i] == bv && si[i] < bi)) {
                bv = sv[i];
                bi = si[i];
            }
        // an index found through a tie on -FLT_MAX is not a strict improvement: the reference returns 0
        out[blockIdx.x] = (bv > -FLT_MAX) ? bi : 0;
    }
}

// ---------------------------------------------------------------- Dequantise (dequant.go), bit-exact
__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) {
    // IEEE half -> float is exact; matches dequant.go:231-261 for every non-NaN pattern.
    _Float16 v;
    __builtin_memcpy(&v, &h, 2);
    return (float)v;
}

__device__ __forceinline__ uint16_t ld_u16(const uint8_t *p) { return (uint16_t)(p[0] | ((uint16_t)p[1] << 8)); }

// one thread per block of 32 (Q4_0 / Q8_0)
__global__ void dequant_q4_0_kernel(const uint8_t *src, float *dst, int64_t nblk) {
    int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblk) return;
    const uint8_t *p = src + b * 18;
    float d = f16_bits_to_f32(ld_u16(p));
    float *o = dst + b * 32;
    for (int i = 0; i < 16; i++) {
        uint8_t bv = p[2 + i];
        o[i] = __fmul_rn(d, (float)((int)(bv & 0xF) - 8));
        o[i + 16] = __fmul_rn(d, (float)((int)(bv >> 4) - 8));
    }
}

__global__ void dequant_q8_0_kernel(const uint8_t *src, float *dst, int64_t nblk) {
    int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblk) return;
    const uint8_t *p = src + b * 34;
    float d = f16_bits_to_f32(ld_u16(p));
    float *o = dst + b * 32;
    for (int i = 0; i < 32; i++) o[i] = __fmul_rn(d, (float)(int8_t)p[2 + i]);
}

__device__ __forceinline__ void scale_min_k4(int j, const uint8_t *q, uint8_t &sc, uint8_t &mn) {  // dequant.go:400-409
    if (j < 4) {
        sc = q[j] & 63;
        mn = q[j + 4] & 63;
    } else {
        sc = (uint8_t)((q[j + 4] & 0x0F) | ((q[j - 4] >> 6) << 4));
        mn = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

// one 64-thread group per super-block of 256; thread t handles elements t, t+64, ...
__global__ void dequant_q4_k_kernel(const uint8_t *src, float *dst, int64_t nblk) {
    int64_t b = (int64_t)blockIdx.x * (blockDim.x / 64) + (threadIdx.x >> 6);
    if (b >= nblk) return;
    int t = threadIdx.x & 63;
    const uint8_t *p = src + b * 144;
    float d = f16_bits_to_f32(ld_u16(p)), dmin = f16_bits_to_f32(ld_u16(p + 2));
    const uint8_t *scales = p + 4, *qs = p + 16;
    float *o = dst + b * 256;
    for (int e = t; e < 256; e += 64) {
        int grp = e >> 6, l = e & 31, hi = (e >> 5) & 1;
        uint8_t sc, mn;
        scale_min_k4(grp * 2 + hi, scales, sc, mn);
        float d1 = __fmul_rn(d, (float)sc), dm1 = __fmul_rn(dmin, (float)mn);
        uint8_t bv = qs[grp * 32 + l];
        int q = hi ? (bv >> 4) : (bv & 0xF);
        o[e] = __fsub_rn(__fmul_rn(d1, (float)q), dm1);
    }
}

// pkg/gguf/dequant.go:423-500: Q4_K's arithmetic with a fifth bit from qh
__global__ void dequant_q5_k_kernel(const uint8_t *src, float *dst, int64_t nblk) {
    int64_t b = (int64_t)blockIdx.x * (blockDim.x / 64) + (threadIdx.x >> 6);
    if (b >= nblk) return;
    int t = threadIdx.x & 63;
    const uint8_t *p = src + b * 176;
    float d = f16_bits_to_f32(ld_u16(p)), dmin = f16_bits_to_f32(ld_u16(p + 2));
    const uint8_t *scales = p + 4, *qh = p + 16, *qs = p + 48;
    float *o = dst + b * 256;
    for (int e = t; e < 256; e += 64) {
        int grp = e >> 6, l = e & 31, hi = (e >> 5) & 1;
        uint8_t sc, mn;
        scale_min_k4(grp * 2 + hi, scales, sc, mn);
        float d1 = __fmul_rn(d, (float)sc), dm1 = __fmul_rn(dmin, (float)mn);
        uint8_t bv = qs[grp * 32 + l];
        int q = (hi ? (bv >> 4) : (bv & 0xF)) + (((qh[l] >> (grp * 2 + hi)) & 1) << 4);
        o[e] = __fsub_rn(__fmul_rn(d1, (float)q), dm1);
    }
}

// pkg/gguf/dequant.go:100-145; thread = one block of 32
__global__ void dequant_q5_0_kernel(const uint8_t *src, float *dst, int64_t nblk) {
    int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblk) return;
    const uint8_t *p = src + b * 22;
    float d = f16_bits_to_f32(ld_u16(p));
    uint32_t qh = (uint32_t)ld_u16(p + 2) | ((uint32_t)ld_u16(p + 4) << 16);
    float *o = dst + b * 32;
    for (int j = 0; j < 16; j++) {
        uint8_t bv = p[6 + j];
        int q0 = (int)(bv & 0xF) | (int)(((qh >> j) & 1) << 4);
        int q1 = (int)(bv >> 4) | (int)(((qh >> (j + 16)) & 1) << 4);
        o[j] = __fmul_rn((float)(q0 - 16), d);
        o[j + 16] = __fmul_rn((float)(q1 - 16), d);
    }
}

// pkg/gguf/dequant.go:215-228
__global__ void dequant_bf16_kernel(const uint8_t *src, float *dst, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = __uint_as_float((uint32_t)ld_u16(src + 2 * i) << 16);
}

__global__ void dequant_q6_k_kernel(const uint8_t *src, float *dst, int64_t nblk) {
    int64_t b = (int64_t)blockIdx.x * (blockDim.x / 64) + (threadIdx.x >> 6);
    if (b >= nblk) return;
    int t = threadIdx.x & 63;
    const uint8_t *p = src + b * 210;
    const uint8_t *ql = p, *qh = p + 128, *sc = p + 192;
    float d = f16_bits_to_f32(ld_u16(p + 208));
    float *o = dst + b * 256;
    int nn = t >> 5, l = t & 31, is = l >> 4;  // dequant.go:294-326
    const uint8_t *qlp = ql + nn * 64, *qhp = qh + nn * 32;
    const int8_t *scp = (const int8_t *)sc + nn * 8;
    int q1 = (int)((qlp[l] & 0xF) | (((qhp[l] >> 0) & 3) << 4)) - 32;
    int q2 = (int)((qlp[l + 32] & 0xF) | (((qhp[l] >> 2) & 3) << 4)) - 32;
    int q3 = (int)((qlp[l] >> 4) | (((qhp[l] >> 4) & 3) << 4)) - 32;
    int q4 = (int)((qlp[l + 32] >> 4) | (((qhp[l] >> 6) & 3) << 4)) - 32;
    float *y = o + nn * 128;
    y[l] = __fmul_rn(__fmul_rn(d, (float)scp[is + 0]), (float)q1);
    y[l + 32] = __fmul_rn(__fmul_rn(d, (float)scp[is + 2]), (float)q2);
    y[l + 64] = __fmul_rn(__fmul_rn(d, (float)scp[is + 4]), (float)q3);
    y[l + 96] = __fmul_rn(__fmul_rn(d, (float)scp[is + 6]), (float)q4);
}

// ---------------------------------------------------------------- dense F32 matmul (cpu.go:106-197)
// C[M,N] = A[M,K] * op(B); 32x32 output tile per block, k ascending inside each output.
template <bool BT>
__global__ void __launch_bounds__(256) matmul_f32_kernel(const float *a, const float *b, float *c, int m, int n,
                                                         int k) {
    __shared__ float as[32][33];
    __shared__ float bs[32][33];
    int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
    int row0 = blockIdx.y * 32, col0 = blockIdx.x * 32;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < k; k0 += 32) {
        for (int r = ty; r < 32; r += 8) {
            int gr = row0 + r, gk = k0 + tx;
            as[r][tx] = (gr < m && gk < k) ? a[(size_t)gr * k + gk] : 0.f;
            if (BT) {  // B is [N,K]
                int gn = col0 + r;
                bs[tx][r] = (gn < n && gk < k) ? b[(size_t)gn * k + gk] : 0.f;
            } else {  // B is [K,N]
                int gkk = k0 + r, gn = col0 + tx;
                bs[r][tx] = (gkk < k && gn < n) ? b[(size_t)gkk * n + gn] : 0.f;
            }
        }
        __syncthreads();
#pragma unroll 8
        for (int kk = 0; kk < 32; kk++) {
            float bv = bs[kk][tx];
#pragma unroll
            for (int i = 0; i < 4; i++) acc[i] = fmaf(as[ty + 8 * i][kk], bv, acc[i]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        int gr = row0 + ty + 8 * i, gn = col0 + tx;
        if (gr < m && gn < n) c[(size_t)gr * n + gn] = acc[i];
    }
}

// ---------------------------------------------------------------- paged scatter (metal_bridge_darwin.m:8539-8642)
template <bool F16>
__global__ void reshape_paged_kv_kernel(const float *src, void *dst, const int32_t *blk_idx, const int32_t *blk_off,
                                        int num_tokens, int num_kv_heads, int head_dim, int block_size, int is_value) {
    size_t hs = (size_t)num_kv_heads * head_dim;
    size_t total = (size_t)num_tokens * hs;
    size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= total) return;
    int t = (int)(gid / hs);
    size_t r = gid % hs;
    size_t part = (size_t)block_size * hs;
    size_t di = (size_t)blk_idx[t] * 2 * part + (is_value ? part : 0) + (size_t)blk_off[t] * hs + r;
    if (F16)
        ((_Float16 *)dst)[di] = (_Float16)src[gid];  // round to nearest even, like Metal's (half)x
    else
        ((float *)dst)[di] = src[gid];
}

// Moves token rows inside a paged pool. Chain c holds the moves chain_offsets[c] .. chain_offsets[c+1]-1, applied
// in that order; a thread owns the same words of every row, so a move may read a row an earlier move of its
// chain wrote. grid = (chains, 2: K rows, V rows).
__global__ void move_paged_kv_kernel(uint32_t *pool, const int32_t *chain_offsets, const int32_t *src_slots,
                                     const int32_t *dst_slots, int row_words, int block_size) {
    const int c = blockIdx.x, half = blockIdx.y;
    const size_t part = (size_t)block_size * row_words;
    for (int i = chain_offsets[c]; i < chain_offsets[c + 1]; i++) {
        const int s = src_slots[i], d = dst_slots[i];
        const uint32_t *src = pool + (size_t)(s / block_size) * 2 * part + half * part + (size_t)(s % block_size) * row_words;
        uint32_t *dst = pool + (size_t)(d / block_size) * 2 * part + half * part + (size_t)(d % block_size) * row_words;
        for (int w = threadIdx.x; w < row_words; w += blockDim.x) dst[w] = src[w];
    }
}


// Copies token rows between slots of one layer's paged pool (K and V of every KV head); the K rows are rotated by
// the angle of position `shift` on the way (interleaved pairs), which turns RoPE(p) into RoPE(p + shift):
// backend/cpu/backend.go:244-276 applied to pool rows. cs: [head_dim/2] (cos, sin) pairs of the shift, worked out
// on the host in the reference's precision chain. The products are rounded before they are added, as the
// reference's separate float32 operations are. grid = tokens, block = 256.
template <typename T>
__global__ void __launch_bounds__(256) copy_shift_paged_kv_kernel(T *pool, const int32_t *__restrict__ src_slots,
                                                                  const int32_t *__restrict__ dst_slots,
                                                                  const float2 *__restrict__ cs, int num_kv_heads,
                                                                  int head_dim, int block_size, int rotate) {
    const int i = blockIdx.x;
    const int s = src_slots[i], d = dst_slots[i];
    const int row = num_kv_heads * head_dim, half = head_dim / 2;
    const size_t part = (size_t)block_size * row;
    const T *ks = pool + (size_t)(s / block_size) * 2 * part + (size_t)(s % block_size) * row;
    T *kd = pool + (size_t)(d / block_size) * 2 * part + (size_t)(d % block_size) * row;
    for (int p = threadIdx.x; p < num_kv_heads * half; p += blockDim.x) {
        const int h = p / half, j = p % half;
        const float v1 = (float)ks[h * head_dim + 2 * j], v2 = (float)ks[h * head_dim + 2 * j + 1];
        float o1 = v1, o2 = v2;
        if (rotate) {
            const float2 c = cs[j];
            // Every product and every sum has to exist as a rounded float32 of its own, as in the reference's
            // separate operations: left alone, the compiler fuses a product into the sum, and the sum into the
            // conversion to half precision (one mixed-precision instruction that rounds once, from the unrounded
            // sum, and lands on the other side of a tie now and then).
            float p1 = v1 * c.x, p2 = v2 * c.y, p3 = v1 * c.y, p4 = v2 * c.x;
            asm volatile("" : "+v"(p1), "+v"(p2), "+v"(p3), "+v"(p4));
            o1 = p1 - p2;
            o2 = p3 + p4;
            asm volatile("" : "+v"(o1), "+v"(o2));
        }
        kd[h * head_dim + 2 * j] = (T)o1;
        kd[h * head_dim + 2 * j + 1] = (T)o2;
    }
    for (int e = threadIdx.x; e < row; e += blockDim.x) kd[part + e] = ks[part + e];  // the V row, as it is
}

inline int grid1d(int64_t n, int threads) { return (int)((n + threads - 1) / threads); }

}  // namespace

extern "C" {

int vx_rmsnorm(vx_backend *be, const float *x, const float *weight, float *out, int rows, int cols, float eps) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(x && weight && out && rows >= 0 && cols > 0, "vx_rmsnorm: bad arguments");
    if (rows == 0) return VX_OK;
    rmsnorm_kernel<<<rows, kThreads, 0, be->stream>>>(x, weight, out, cols, eps);
    VX_CHECK_LAUNCH();
    return VX_OK;
}

int vx_rope(vx_backend *be, float *q, float *k, int head_dim, int num_heads, int num_kv_heads, int seq_len,
            int start_pos, int rope_dim, float theta, int rope_neox) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(q && head_dim > 0 && num_heads > 0 && seq_len >= 0, "vx_rope: bad arguments");
    int eff = rope_dim == 0 ? head_dim : rope_dim;
    VX_REQUIRE(eff <= head_dim && eff % 2 == 0, "vx_rope: rope_dim %d invalid for head_dim %d", rope_dim, head_dim);
    if (seq_len == 0) return VX_OK;
    int threads = eff / 2 < 64 ? 64 : (eff / 2 > 256 ? 256 : eff / 2);
    rope_kernel<<<seq_len, threads, 0, be->stream>>>(q, k, head_dim, num_heads, num_kv_heads, start_pos, eff, theta,
                                                      rope_neox, nullptr, 1);
    VX_CHECK_LAUNCH();
    return VX_OK;
}

int vx_rope_shift(vx_backend *be, float *k, int head_dim, int num_kv_heads, int num_tokens, int shift, float theta) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(k && head_dim > 0 && head_dim % 2 == 0 && num_kv_heads > 0 && num_tokens >= 0, "vx_rope_shift: bad arguments");
    if (shift == 0 || num_tokens == 0) return VX_OK;  // backend/cpu/backend.go:248-250
    int threads = head_dim / 2 < 64 ? 64 : (head_dim / 2 > 256 ? 256 : head_dim / 2);
    rope_kernel<<<num_tokens, threads, 0, be->stream>>>(nullptr, k, head_dim, 0, num_kv_heads, shift, head_dim, theta, 0,
                                                         nullptr, 0);
    VX_CHECK_LAUNCH();
    return VX_OK;
}

int vx_paged_kv_copy_shifted(vx_backend *be, void *kv_pool, int pool_is_f16, const int32_t *src_slots,
                             const int32_t *dst_slots, int num_tokens, int num_kv_heads, int head_dim, int block_size,
                             int shift, float theta) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(kv_pool && src_slots && dst_slots && num_tokens >= 0, "vx_paged_kv_copy_shifted: bad arguments");
    VX_REQUIRE(head_dim > 0 && head_dim % 2 == 0 && num_kv_heads > 0 && block_size > 0, "vx_paged_kv_copy_shifted: bad shape");
    if (num_tokens == 0) return VX_OK;
    const int half = head_dim / 2;
    VX_REQUIRE(half <= VX_ROPE_TAB_PAIRS * 2, "vx_paged_kv_copy_shifted: head_dim %d too large", head_dim);
    if (shift != 0 && !(be->shift_tab && be->shift_tab_shift == shift && be->shift_tab_theta == theta && be->shift_tab_dim == head_dim)) {
        // The angles depend on (shift, theta, head_dim) only: worked out and uploaded when that changes (once per
        // fragment insertion, not once per layer), into a table of their own that nothing else writes.
        VX_REQUIRE(!be->capturing, "vx_paged_kv_copy_shifted: a new shift table during graph capture");
        if (!be->shift_tab) VX_CHECK_HIP(hipMalloc(&be->shift_tab, (size_t)VX_ROPE_TAB_PAIRS * 2 * sizeof(float2)));
        std::vector<float2> t(half);
        for (int j = 0; j < half; j++) {                       // backend/cpu/backend.go:262-266
            const double ex = (double)(2 * j) / (double)head_dim;
            const float freq = (float)(1.0 / pow((double)theta, ex));
            const float angle = (float)shift * freq;
            // through volatile doubles: the compiler may otherwise shrink (float)cos((double)x) to cosf(x), whose
            // last bit is not the correctly rounded double result's
            volatile double cd = cos((double)angle), sd = sin((double)angle);
            t[j] = make_float2((float)cd, (float)sd);
        }
        VX_CHECK_HIP(hipStreamSynchronize(be->stream));        // a copy in flight may still read the previous table
        VX_CHECK_HIP(hipMemcpy(be->shift_tab, t.data(), (size_t)half * sizeof(float2), hipMemcpyHostToDevice));
        be->shift_tab_shift = shift;
        be->shift_tab_theta = theta;
        be->shift_tab_dim = head_dim;
    }
    if (pool_is_f16)
        copy_shift_paged_kv_kernel<_Float16><<<num_tokens, 256, 0, be->stream>>>((_Float16 *)kv_pool, src_slots, dst_slots,
                                                                                 (const float2 *)be->shift_tab, num_kv_heads,
                                                                                 head_dim, block_size, shift != 0);
    else
        copy_shift_paged_kv_kernel<float><<<num_tokens, 256, 0, be->stream>>>((float *)kv_pool, src_slots, dst_slots,
                                                                              (const float2 *)be->shift_tab, num_kv_heads,
                                                                              head_dim, block_size, shift != 0);
    VX_CHECK_LAUNCH();
    return VX_OK;
}

int vx_rope_store_paged_ex(vx_backend *be, float *q, const float *k, const float *v, const int32_t *positions,
                           const int32_t *slot_mapping, void *kv_pool, int pool_is_f16, int rows, int num_q_heads,
                           int num_kv_heads, int head_dim, int block_size, float theta, int rope_dim, int rope_neox) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(q && k && v && positions && slot_mapping && kv_pool, "vx_rope_store_paged: null pointer");
    VX_REQUIRE(head_dim > 0 && head_dim % 2 == 0 && block_size > 0 && num_q_heads > 0 && num_kv_heads > 0,
               "vx_rope_store_paged: bad shape");
    const int eff = rope_dim == 0 ? head_dim : rope_dim;
    VX_REQUIRE(eff > 0 && eff <= head_dim && eff % 2 == 0, "vx_rope_store_paged: rope_dim %d invalid for head_dim %d", rope_dim,
               head_dim);
    if (rows == 0) return VX_OK;
    VX_REQUIRE(head_dim <= 512, "vx_rope_store_paged: head_dim %d too large", head_dim);
    const int half = head_dim / 2;
    const int lanes = 256 / half > 0 ? 256 / half : 1;
    const int threads = lanes * half;
    const int max_heads = num_q_heads > num_kv_heads ? num_q_heads : num_kv_heads;
    int groups = ceil_div(max_heads, lanes * 2);  // about two heads per thread
    if (groups < 1) groups = 1;
    dim3 grid(rows, groups);
    if (pool_is_f16)
        rope_store_paged_kernel<true><<<grid, threads, 0, be->stream>>>(q, k, v, positions, slot_mapping, kv_pool,
                                                                        num_q_heads, num_kv_heads, head_dim,
                                                                        block_size, theta, eff, rope_neox);
    else
        rope_store_paged_kernel<false><<<grid, threads, 0, be->stream>>>(q, k, v, positions, slot_mapping, kv_pool,
                                                                         num_q_heads, num_kv_heads, head_dim,
                                                                         block_size, theta, eff, rope_neox);
    VX_CHECK_LAUNCH();
    return VX_OK;
}

int vx_rope_store_paged(vx_backend *be, float *q, const float *k, const float *v, const int32_t *positions,
                        const int32_t *slot_mapping, void *kv_pool, int pool_is_f16, int rows, int num_q_heads,
                        int num_kv_heads, int head_dim, int block_size, float theta) {
    return vx_rope_store_paged_ex(be, q, k, v, positions, slot_mapping, kv_pool, pool_is_f16, rows, num_q_heads,
                                  num_kv_heads, head_dim, block_size, theta, 0, 0);
}

#define VX_EW(name, kernel, ...)                                                \
    int rc = enter(be);                                                         \
    if (rc) return rc;                                                          \
    VX_REQUIRE(n >= 0, name ": negative n");                                    \
    if (n == 0) return VX_OK;                                                   \
    kernel<<<grid1d(n, kThreads), kThreads, 0, be->stream>>>(__VA_ARGS__, n);   \
    VX_CHECK_LAUNCH();                                                          \
    return VX_OK;

int vx_silu(vx_backend *be, const float *x, float *out, int n) {
    VX_REQUIRE(x && out, "vx_silu: null pointer");
    VX_EW("vx_silu", silu_kernel, x, out)
}

int vx_silu_mul(vx_backend *be, const float *gate, const float *up, float *out, int n) {
    VX_REQUIRE(gate && up && out, "vx_silu_mul: null pointer");
    VX_EW("vx_silu_mul", silu_mul_kernel, gate, up, out)
}

int vx_gelu(vx_backend *be, const float *x, float *out, int n) {
    VX_REQUIRE(x && out, "vx_gelu: null pointer");
    VX_EW("vx_gelu", gelu_kernel, x, out)
}

int vx_gelu_mul(vx_backend *be, const float *gate, const float *up, float *out, int n) {
    VX_REQUIRE(gate && up && out, "vx_gelu_mul: null pointer");
    VX_EW("vx_gelu_mul", gelu_mul_kernel, gate, up, out)
}

int vx_scale_buffer(vx_backend *be, float *buf, float scale, int n) {
    VX_REQUIRE(buf, "vx_scale_buffer: null pointer");
    VX_EW("vx_scale_buffer", scale_kernel, buf, scale)
}

int vx_logit_softcap(vx_backend *be, float *logits, int n, float cap) {
    VX_REQUIRE(logits, "vx_logit_softcap: null pointer");
    if (cap <= 0.f) return enter(be);  // disabled (model.go:342-344)
    VX_EW("vx_logit_softcap", logit_softcap_kernel, logits, (double)cap, 1.0 / (double)cap)
}

int vx_add_bias(vx_backend *be, const float *x, const float *bias, float *out, int rows, int cols) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(x && bias && out && rows >= 0 && cols > 0, "vx_add_bias: bad arguments");
    VX_REQUIRE((int64_t)rows * cols <= INT32_MAX, "vx_add_bias: %d x %d elements exceed 2^31", rows, cols);
    const int n = rows * cols;
    if (n == 0) return VX_OK;
    add_bias_kernel<<<grid1d(n, kThreads), kThreads, 0, be->stream>>>(x, bias, out, cols, n);
    VX_CHECK_LAUNCH();
    return VX_OK;
}

int vx_layernorm(vx_backend *be, const float *x, const float *weight, const float *bias, float *out, int rows, int cols,
                 float eps) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(x && weight && bias && out && rows >= 0 && cols > 0, "vx_layernorm: bad arguments");
    if (rows == 0) return VX_OK;
    layernorm_kernel<<<rows, kThreads, 0, be->stream>>>(x, weight, bias, out, cols, eps);
    VX_CHECK_LAUNCH();
    return VX_OK;
}

int vx_rope_with_freqs(vx_backend *be, float *q, float *k, const float *freqs, int head_dim, int num_heads,
                       int num_kv_heads, int seq_len, int start_pos, int rope_neox) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(q && freqs && head_dim > 0 && head_dim % 2 == 0 && num_heads > 0 && seq_len >= 0 && (!k || num_kv_heads > 0),
               "vx_rope_with_freqs: bad arguments");
    if (seq_len == 0) return VX_OK;
    int threads = head_dim / 2 < 64 ? 64 : (head_dim / 2 > 256 ? 256 : head_dim / 2);
    rope_freqs_kernel<<<seq_len, threads, 0, be->stream>>>(q, k, freqs, head_dim, num_heads, num_kv_heads, start_pos,
                                                           rope_neox);
    VX_CHECK_LAUNCH();
    return VX_OK;
}

int vx_add(vx_backend *be, const float *a, const float *b, float *out, int n) {
    VX_REQUIRE(a && b && out, "vx_add: null pointer");
    VX_EW("vx_add", add_kernel, a, b, out)
}

int vx_mul(vx_backend *be, const float *a, const float *b, float *out, int n) {
    VX_REQUIRE(a && b && out, "vx_mul: null pointer");
    VX_EW("vx_mul", mul_kernel, a, b, out)
}

int vx_softmax(vx_backend *be, const float *x, float *out, int rows, int cols) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(x && out && rows >= 0 && cols > 0, "vx_softmax: bad arguments");
    if (rows == 0) return VX_OK;
    softmax_kernel<<<rows, kThreads, 0, be->stream>>>(x, out, cols);
    VX_CHECK_LAUNCH();
    return VX_OK;
}

int vx_embedding(vx_backend *be, const int32_t *ids, int num_tokens, const float *table, float *out, int vocab_size,
                 int dim) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(ids && table && out && num_tokens >= 0 && dim > 0, "vx_embedding: bad arguments");
    if (num_tokens == 0) return VX_OK;
    embedding_kernel<<<num_tokens, kThreads, 0, be->stream>>>(ids, table, out, vocab_size, dim);
    VX_CHECK_LAUNCH();
    return VX_OK;
}

int vx_argmax_rows(vx_backend *be, const float *logits, int rows, int n, int32_t *out_idx) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(logits && out_idx && rows >= 0 && n > 0, "vx_argmax_rows: bad arguments");
    if (rows == 0) return VX_OK;
    argmax_rows_kernel<<<rows, 1024, 0, be->stream>>>(logits, n, out_idx);
    VX_CHECK_LAUNCH();
    return VX_OK;
}

int vx_argmax(vx_backend *be, const float *input, int n, int *out_index) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(input && out_index && n > 0, "vx_argmax: bad arguments");
    VX_REQUIRE(!be->capturing, "vx_argmax during graph capture");
    int32_t *dev = (int32_t *)be->misc_ws;
    argmax_rows_kernel<<<1, 1024, 0, be->stream>>>(input, n, dev);
    VX_CHECK_LAUNCH();
    VX_CHECK_HIP(hipMemcpyAsync(be->host_stage, dev, 4, hipMemcpyDeviceToHost, be->stream));
    VX_CHECK_HIP(hipStreamSynchronize(be->stream));
    *out_index = *(int32_t *)be->host_stage;
    return VX_OK;
}

int vx_dequantize(vx_backend *be, int fmt, const void *src, float *dst, int64_t n) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(src && dst && n >= 0, "vx_dequantize: bad arguments");
    if (n == 0) return VX_OK;
    const uint8_t *s = (const uint8_t *)src;
    switch (fmt) {
    case VX_Q4_0:
        VX_REQUIRE(n % 32 == 0, "vx_dequantize: n must be a multiple of 32");
        dequant_q4_0_kernel<<<grid1d(n / 32, kThreads), kThreads, 0, be->stream>>>(s, dst, n / 32);
        break;
    case VX_Q8_0:
        VX_REQUIRE(n % 32 == 0, "vx_dequantize: n must be a multiple of 32");
        dequant_q8_0_kernel<<<grid1d(n / 32, kThreads), kThreads, 0, be->stream>>>(s, dst, n / 32);
        break;
    case VX_Q4_K:
        VX_REQUIRE(n % 256 == 0, "vx_dequantize: n must be a multiple of 256");
        dequant_q4_k_kernel<<<grid1d(n / 256, 4), 256, 0, be->stream>>>(s, dst, n / 256);
        break;
    case VX_Q6_K:
        VX_REQUIRE(n % 256 == 0, "vx_dequantize: n must be a multiple of 256");
        dequant_q6_k_kernel<<<grid1d(n / 256, 4), 256, 0, be->stream>>>(s, dst, n / 256);
        break;
    case VX_Q5_0:
        VX_REQUIRE(n % 32 == 0, "vx_dequantize: n must be a multiple of 32");
        dequant_q5_0_kernel<<<grid1d(n / 32, kThreads), kThreads, 0, be->stream>>>(s, dst, n / 32);
        break;
    case VX_Q5_K:
        VX_REQUIRE(n % 256 == 0, "vx_dequantize: n must be a multiple of 256");
        dequant_q5_k_kernel<<<grid1d(n / 256, 4), 256, 0, be->stream>>>(s, dst, n / 256);
        break;
    case VX_BF16:
        dequant_bf16_kernel<<<grid1d(n, kThreads), kThreads, 0, be->stream>>>(s, dst, n);
        break;
    default:
        set_error("vx_dequantize: unknown format %d", fmt);
        return VX_ERR_UNSUPPORTED;
    }
    VX_CHECK_LAUNCH();
    return VX_OK;
}

int vx_matmul(vx_backend *be, const float *a, const float *b, float *out, int m, int n, int k) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(a && b && out && m >= 0 && n >= 0 && k >= 0, "vx_matmul: bad arguments");
    if (m == 0 || n == 0) return VX_OK;
    dim3 grid(ceil_div(n, 32), ceil_div(m, 32));
    matmul_f32_kernel<false><<<grid, 256, 0, be->stream>>>(a, b, out, m, n, k);
    VX_CHECK_LAUNCH();
    return VX_OK;
}

int vx_matmul_transposed(vx_backend *be, const float *a, const float *b, float *out, int m, int n, int k) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(a && b && out && m >= 0 && n >= 0 && k >= 0, "vx_matmul_transposed: bad arguments");
    if (m == 0 || n == 0) return VX_OK;
    dim3 grid(ceil_div(n, 32), ceil_div(m, 32));
    matmul_f32_kernel<true><<<grid, 256, 0, be->stream>>>(a, b, out, m, n, k);
    VX_CHECK_LAUNCH();
    return VX_OK;
}

static int reshape_paged(vx_backend *be, const float *src, void *dst_base, const int32_t *page_table,
                         const int32_t *block_offsets, int num_tokens, int num_kv_heads, int head_dim,
                         int block_size, int is_value, bool f16) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(src && dst_base && page_table && block_offsets, "vx_reshape_paged_kv: null pointer");
    VX_REQUIRE(num_tokens >= 0 && num_kv_heads > 0 && head_dim > 0 && block_size > 0, "vx_reshape_paged_kv: bad shape");
    if (num_tokens == 0) return VX_OK;
    int64_t total = (int64_t)num_tokens * num_kv_heads * head_dim;
    if (f16)
        reshape_paged_kv_kernel<true><<<grid1d(total, kThreads), kThreads, 0, be->stream>>>(
            src, dst_base, page_table, block_offsets, num_tokens, num_kv_heads, head_dim, block_size, is_value);
    else
        reshape_paged_kv_kernel<false><<<grid1d(total, kThreads), kThreads, 0, be->stream>>>(
            src, dst_base, page_table, block_offsets, num_tokens, num_kv_heads, head_dim, block_size, is_value);
    VX_CHECK_LAUNCH();
    return VX_OK;
}

int vx_reshape_paged_kv(vx_backend *be, const float *src, void *dst_base, const int32_t *page_table,
                        const int32_t *block_offsets, int num_tokens, int num_kv_heads, int head_dim, int block_size,
                        int is_value) {
    return reshape_paged(be, src, dst_base, page_table, block_offsets, num_tokens, num_kv_heads, head_dim, block_size,
                         is_value, false);
}

int vx_reshape_paged_kv_f16(vx_backend *be, const float *src, void *dst_base, const int32_t *page_table,
                            const int32_t *block_offsets, int num_tokens, int num_kv_heads, int head_dim,
                            int block_size, int is_value) {
    return reshape_paged(be, src, dst_base, page_table, block_offsets, num_tokens, num_kv_heads, head_dim, block_size,
                         is_value, true);
}

int vx_paged_kv_move(vx_backend *be, void *kv_pool, int pool_is_f16, const int32_t *chain_offsets,
                     const int32_t *src_slots, const int32_t *dst_slots, int num_chains, int num_kv_heads, int head_dim,
                     int block_size) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(kv_pool && chain_offsets && src_slots && dst_slots, "vx_paged_kv_move: null pointer");
    VX_REQUIRE(num_chains >= 0 && num_kv_heads > 0 && head_dim > 0 && block_size > 0, "vx_paged_kv_move: bad shape");
    const int64_t row_bytes = (int64_t)num_kv_heads * head_dim * (pool_is_f16 ? 2 : 4);
    VX_REQUIRE(row_bytes % 4 == 0, "vx_paged_kv_move: a token row must be a whole number of 32-bit words");
    if (num_chains == 0) return VX_OK;
    move_paged_kv_kernel<<<dim3(num_chains, 2), kThreads, 0, be->stream>>>((uint32_t *)kv_pool, chain_offsets, src_slots,
                                                                        dst_slots, (int)(row_bytes / 4), block_size);
    VX_CHECK_LAUNCH();
    return VX_OK;
}

}  // extern "C"
