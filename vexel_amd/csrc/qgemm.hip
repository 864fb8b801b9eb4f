// Quantized matmul C[M,N] = A[M,K] * B^T with B in raw GGUF blocks (Q4_0, Q8_0, Q4_K, Q6_K).
// Replaces QuantizedMatMul.MatMulQ4_0/Q4_K/Q6_K/Q8_0 (inference/backend/backend.go:47-81).
//
// Fast path (Q4_0, Q8_0, Q4_K; K a multiple of 256, 16-byte aligned rows):
//   1. split_act_kernel scales every activation row by a power of two, splits it into
//      hi = f16(x) and lo = f16(x - hi) (together ~22 significant bits, the float32 level)
//      and stores both in the k-order the weight unpacking produces.
//   2. qgemm_kernel: a workgroup owns 16*R weight rows; its 4 waves split K. A wave stages
//      its rows' raw blocks from HBM into LDS with coalesced 16-byte loads, unpacks the
//      integer codes to exact f16 values in registers, and feeds v_mfma_f32_16x16x32_f16
//      twice per 32-element block (hi, lo). The block scale d is applied to the float32
//      MFMA result, never to the f16 operand, so the weight values entering the sum are
//      exactly the integers of the format. The 4 partial sums are added in wave order.
//   Each output element depends only on its own activation row and weight row, and the
//   arithmetic does not depend on M, so a row gives the same bits alone or in a batch
//   (the property the reference keeps by looping M=1 kernels, backend/metal/backend.go:777-779).
// Fallback (Q6_K, odd shapes): one wave per output column, float32 FMAs on the exact
// dequantised values.
#include "common.h"

using namespace vx;

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float h2f(uint16_t h) {
    _Float16 v;
    __builtin_memcpy(&v, &h, 2);
    return (float)v;
}

// ---------------------------------------------------------------- k-order of the MFMA operand
// perm[p] = element index (within a 32-element block) that sits in operand position p, where
// position p = 8*g + j is slot j of lane group g. inv is the inverse.
struct Perm32 {
    int8_t inv[32];
};

constexpr Perm32 make_inv_q4_0() {
    Perm32 r{};
    for (int g = 0; g < 4; g++) {
        const int e[8] = {4 * g, 4 * g + 2, 16 + 4 * g, 16 + 4 * g + 2, 4 * g + 1, 4 * g + 3, 16 + 4 * g + 1, 16 + 4 * g + 3};
        for (int j = 0; j < 8; j++) r.inv[e[j]] = (int8_t)(8 * g + j);
    }
    return r;
}
constexpr Perm32 make_inv_ident() {
    Perm32 r{};
    for (int i = 0; i < 32; i++) r.inv[i] = (int8_t)i;
    return r;
}
constexpr Perm32 make_inv_q4_k() {
    Perm32 r{};
    const int o[8] = {0, 2, 1, 3, 4, 6, 5, 7};
    for (int g = 0; g < 4; g++)
        for (int j = 0; j < 8; j++) r.inv[8 * g + o[j]] = (int8_t)(8 * g + j);
    return r;
}

__constant__ Perm32 c_inv_q4_0 = make_inv_q4_0();
__constant__ Perm32 c_inv_q8_0 = make_inv_ident();
__constant__ Perm32 c_inv_q4_k = make_inv_q4_k();

// ---------------------------------------------------------------- activation split
// grid = Mpad rows, block = 256. Outputs: hi/lo [Mpad,K] f16 (permuted inside each 32-block),
// inv_scale[Mpad], bsum[K/32][Mpad] (block sums of the scaled row; used by Q4_K's min term).
__global__ void __launch_bounds__(256) split_act_kernel(const float *__restrict__ a, int M, int K, int fmt,
                                                        _Float16 *__restrict__ hi, _Float16 *__restrict__ lo,
                                                        float *__restrict__ inv_scale, float *__restrict__ bsum,
                                                        int Mpad) {
    __shared__ float sm[4];
    const int r = blockIdx.x, tid = threadIdx.x;
    const Perm32 *pm = fmt == VX_Q4_0 ? &c_inv_q4_0 : (fmt == VX_Q4_K ? &c_inv_q4_k : &c_inv_q8_0);
    if (r >= M) {
        for (int k = tid; k < K; k += 256) {
            hi[(size_t)r * K + k] = (_Float16)0.f;
            lo[(size_t)r * K + k] = (_Float16)0.f;
        }
        for (int b = tid; b < K / 32; b += 256) bsum[(size_t)b * Mpad + r] = 0.f;
        if (tid == 0) inv_scale[r] = 0.f;
        return;
    }
    const float *ar = a + (size_t)r * K;
    float amax = 0.f;
    for (int k = tid; k < K; k += 256) amax = fmaxf(amax, fabsf(ar[k]));
    for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    if ((tid & 63) == 0) sm[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(sm[0], sm[1]), fmaxf(sm[2], sm[3]));
    float s = 1.f, inv = 1.f;
    if (amax > 0.f && amax < INFINITY) {
        int ex;
        (void)frexpf(amax, &ex);      // amax = f * 2^ex, f in [0.5,1)
        s = ldexpf(1.f, 14 - ex);     // amax*s in [2^13, 2^14)
        inv = ldexpf(1.f, ex - 14);
    }
    if (tid == 0) inv_scale[r] = inv;
    for (int k = tid; k < K; k += 256) {
        float x = ar[k] * s;
        _Float16 h = (_Float16)x;
        _Float16 l = (_Float16)(x - (float)h);
        size_t o = (size_t)r * K + (k & ~31) + pm->inv[k & 31];
        hi[o] = h;
        lo[o] = l;
        // 32 consecutive threads hold one block (256 % 32 == 0 and K % 32 == 0)
        float t = x;
        for (int off = 16; off > 0; off >>= 1) t += __shfl_xor(t, off, 64);
        if ((tid & 31) == 0) bsum[(size_t)(k >> 5) * Mpad + r] = t;
    }
}

// ---------------------------------------------------------------- format policies (fast path)
// CHUNK_STEPS 32-element MFMA steps per staged chunk, CHUNK_BYTES raw bytes per row per chunk.
__device__ __forceinline__ uint32_t lds_u32_unaligned(const uint8_t *p) {
    uintptr_t a = (uintptr_t)p;
    const uint32_t *w = (const uint32_t *)(a & ~(uintptr_t)3);
    return __builtin_amdgcn_alignbyte(w[1], w[0], (uint32_t)(a & 3));
}

__device__ __forceinline__ uint32_t as_u32(half2v v) {
    uint32_t u;
    __builtin_memcpy(&u, &v, 4);
    return u;
}
__device__ __forceinline__ half2v as_h2(uint32_t u) {
    half2v v;
    __builtin_memcpy(&v, &u, 4);
    return v;
}

__device__ __forceinline__ half8 pack8(half2v a, half2v b, half2v c, half2v d) {
    half8 r;
    r[0] = a[0]; r[1] = a[1]; r[2] = b[0]; r[3] = b[1];
    r[4] = c[0]; r[5] = c[1]; r[6] = d[0]; r[7] = d[1];
    return r;
}

struct StepW {   // what one MFMA step needs from the weights
    half8 b;     // exact integer codes as f16
    float d;     // multiplies the MFMA result
    float dm;    // multiplies the activation block sum and is subtracted (Q4_K), else 0
};

struct PQ4_0 {
    static constexpr int CHUNK_STEPS = 16, CHUNK_BYTES = 288;  // sixteen 18-byte blocks
    static constexpr bool HAS_MIN = false;
    static __device__ __forceinline__ size_t row_bytes(int K) { return (size_t)K / 32 * 18; }
    static __device__ __forceinline__ StepW load(const uint8_t *row, int step, int g) {
        const uint8_t *blk = row + step * 18;
        uint32_t w = lds_u32_unaligned(blk + 2 + 4 * g);
        const half2v off = {(_Float16)1032.f, (_Float16)1032.f};
        const uint32_t m = 0x000F000Fu, mg = 0x64006400u;
        half2v x0 = as_h2((w & m) | mg) - off;          // bytes 0,2 low nibbles
        half2v x1 = as_h2(((w >> 4) & m) | mg) - off;   // bytes 0,2 high nibbles
        half2v x2 = as_h2(((w >> 8) & m) | mg) - off;   // bytes 1,3 low nibbles
        half2v x3 = as_h2(((w >> 12) & m) | mg) - off;  // bytes 1,3 high nibbles
        StepW r;
        r.b = pack8(x0, x1, x2, x3);
        r.d = h2f(*(const uint16_t *)blk);
        r.dm = 0.f;
        return r;
    }
};

struct PQ8_0 {
    static constexpr int CHUNK_STEPS = 8, CHUNK_BYTES = 272;
    static constexpr bool HAS_MIN = false;
    static __device__ __forceinline__ size_t row_bytes(int K) { return (size_t)K / 32 * 34; }
    static __device__ __forceinline__ StepW load(const uint8_t *row, int step, int g) {
        const uint8_t *blk = row + step * 34;
        const uint8_t *p = blk + 2 + 8 * g;
        uintptr_t a = (uintptr_t)p;
        const uint32_t *w = (const uint32_t *)(a & ~(uintptr_t)3);
        uint32_t sh = (uint32_t)(a & 3);
        uint32_t w0 = __builtin_amdgcn_alignbyte(w[1], w[0], sh) ^ 0x80808080u;
        uint32_t w1 = __builtin_amdgcn_alignbyte(w[2], w[1], sh) ^ 0x80808080u;
        const half2v off = {(_Float16)1152.f, (_Float16)1152.f};  // 1024 + 128
        const uint32_t c64 = 0x64646464u;
        half2v x0 = as_h2(__builtin_amdgcn_perm(w0, c64, 0x00050004u)) - off;
        half2v x1 = as_h2(__builtin_amdgcn_perm(w0, c64, 0x00070006u)) - off;
        half2v x2 = as_h2(__builtin_amdgcn_perm(w1, c64, 0x00050004u)) - off;
        half2v x3 = as_h2(__builtin_amdgcn_perm(w1, c64, 0x00070006u)) - off;
        StepW r;
        r.b = pack8(x0, x1, x2, x3);
        r.d = h2f(*(const uint16_t *)blk);
        r.dm = 0.f;
        return r;
    }
};

struct PQ4_K {
    static constexpr int CHUNK_STEPS = 16, CHUNK_BYTES = 288;  // two 144-byte super-blocks
    static constexpr bool HAS_MIN = true;
    static __device__ __forceinline__ size_t row_bytes(int K) { return (size_t)K / 256 * 144; }
    static __device__ __forceinline__ StepW load(const uint8_t *row, int step, int g) {
        const uint8_t *sb = row + (step >> 3) * 144;
        const int j = step & 7, gr = j >> 1, hi = j & 1;
        const uint32_t *qp = (const uint32_t *)(sb + 16 + 32 * gr + 8 * g);
        uint32_t w0 = qp[0] >> (4 * hi), w1 = qp[1] >> (4 * hi);
        const half2v off = {(_Float16)1024.f, (_Float16)1024.f};
        const uint32_t m = 0x000F000Fu, mg = 0x64006400u;
        half2v x0 = as_h2((w0 & m) | mg) - off;         // bytes 0,2
        half2v x1 = as_h2(((w0 >> 8) & m) | mg) - off;  // bytes 1,3
        half2v x2 = as_h2((w1 & m) | mg) - off;         // bytes 4,6
        half2v x3 = as_h2(((w1 >> 8) & m) | mg) - off;  // bytes 5,7
        const uint8_t *q = sb + 4;
        uint32_t sc, mn;  // dequant.go:400-409
        if (j < 4) {
            sc = q[j] & 63;
            mn = q[j + 4] & 63;
        } else {
            sc = (q[j + 4] & 0x0F) | ((q[j - 4] >> 6) << 4);
            mn = (q[j + 4] >> 4) | ((q[j] >> 6) << 4);
        }
        uint32_t hd = *(const uint32_t *)sb;
        StepW r;
        r.b = pack8(x0, x1, x2, x3);
        r.d = h2f((uint16_t)(hd & 0xFFFF)) * (float)sc;
        r.dm = h2f((uint16_t)(hd >> 16)) * (float)mn;
        return r;
    }
};

constexpr int PITCH_PAD = 16;

// grid.x = ceil(N / (16*R)); block = 256 (4 waves, K split by chunk index mod 4).
// MT = number of 16-row activation tiles processed per pass over the weights.
template <class F, int R, int MT>
__global__ void __launch_bounds__(256) qgemm_kernel(const uint8_t *__restrict__ W, const _Float16 *__restrict__ ahi,
                                                    const _Float16 *__restrict__ alo,
                                                    const float *__restrict__ inv_scale,
                                                    const float *__restrict__ bsum, float *__restrict__ out,
                                                    const float *__restrict__ residual, int M, int Mpad, int N, int K) {
    constexpr int ROWS = 16 * R;
    constexpr int PITCH = F::CHUNK_BYTES + PITCH_PAD;
    constexpr int PIECES = ROWS * (F::CHUNK_BYTES / 16);
    constexpr int NL = (PIECES + 63) / 64;
    constexpr int WAVE_LDS = ROWS * PITCH;
    constexpr int RED_FLOATS = 4 * R * MT * 4 * 64;
    constexpr int LDS_BYTES = (4 * WAVE_LDS > RED_FLOATS * 4) ? 4 * WAVE_LDS : RED_FLOATS * 4;
    __shared__ __attribute__((aligned(16))) uint8_t smem[LDS_BYTES];

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int ln = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * ROWS;
    const size_t row_bytes = F::row_bytes(K);
    const int steps_total = K / 32;
    const int n_chunks = (steps_total + F::CHUNK_STEPS - 1) / F::CHUNK_STEPS;
    uint8_t *wl = smem + wave * WAVE_LDS;

    for (int m0 = 0; m0 < Mpad; m0 += 16 * MT) {
        float4v run[R][MT];
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int t = 0; t < MT; t++) run[r][t] = (float4v){0.f, 0.f, 0.f, 0.f};

        uint4 stage[NL];
        auto fetch = [&](int chunk) {
            const size_t coff = (size_t)chunk * F::CHUNK_BYTES;
            const int valid_bytes = (int)min((size_t)F::CHUNK_BYTES, row_bytes - coff);
#pragma unroll
            for (int i = 0; i < NL; i++) {
                int pc = i * 64 + lane;
                int row = pc / (F::CHUNK_BYTES / 16), col = pc % (F::CHUNK_BYTES / 16);
                int n = min(n0 + row, N - 1);
                bool ok = pc < PIECES && col * 16 < valid_bytes;
                stage[i] = ok ? *(const uint4 *)(W + (size_t)n * row_bytes + coff + col * 16) : make_uint4(0, 0, 0, 0);
            }
        };
        auto commit = [&]() {
#pragma unroll
            for (int i = 0; i < NL; i++) {
                int pc = i * 64 + lane;
                int row = pc / (F::CHUNK_BYTES / 16), col = pc % (F::CHUNK_BYTES / 16);
                if (pc < PIECES) *(uint4 *)(wl + row * PITCH + col * 16) = stage[i];
            }
        };

        int chunk = wave;
        if (chunk < n_chunks) fetch(chunk);
        for (; chunk < n_chunks; chunk += 4) {
            __builtin_amdgcn_wave_barrier();
            commit();
            __builtin_amdgcn_wave_barrier();
            if (chunk + 4 < n_chunks) fetch(chunk + 4);
            const int s0 = chunk * F::CHUNK_STEPS;
            const int nsteps = min(F::CHUNK_STEPS, steps_total - s0);
            for (int s = 0; s < nsteps; s++) {
                const size_t koff = (size_t)(s0 + s) * 32 + 8 * g;
                half8 ah[MT], al[MT];
#pragma unroll
                for (int t = 0; t < MT; t++) {
                    const size_t ro = (size_t)(m0 + t * 16 + ln) * K + koff;
                    ah[t] = *(const half8 *)(ahi + ro);
                    al[t] = *(const half8 *)(alo + ro);
                }
#pragma unroll
                for (int r = 0; r < R; r++) {
                    StepW sw = F::load(wl + (r * 16 + ln) * PITCH, s, g);
#pragma unroll
                    for (int t = 0; t < MT; t++) {
                        float4v acc = {0.f, 0.f, 0.f, 0.f};
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah[t], sw.b, acc, 0, 0, 0);
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(al[t], sw.b, acc, 0, 0, 0);
                        if (F::HAS_MIN) {
                            const float4v bs = *(const float4v *)(bsum + (size_t)(s0 + s) * Mpad + m0 + t * 16 + 4 * g);
#pragma unroll
                            for (int i = 0; i < 4; i++) run[r][t][i] += sw.d * acc[i] - sw.dm * bs[i];
                        } else {
#pragma unroll
                            for (int i = 0; i < 4; i++) run[r][t][i] += sw.d * acc[i];
                        }
                    }
                }
            }
        }

        // cross-wave reduction in wave order, then scale back, add the residual, store
        __syncthreads();
        float *red = (float *)smem;
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int t = 0; t < MT; t++)
#pragma unroll
                for (int i = 0; i < 4; i++) red[((wave * R + r) * MT + t) * 256 + i * 64 + lane] = run[r][t][i];
        __syncthreads();
        for (int idx = tid; idx < R * MT * 256; idx += 256) {
            const int rt = idx / 256, e = idx % 256, i = e / 64, l2 = e % 64;
            const int r = rt / MT, t = rt % MT;
            float v = red[(0 * R * MT + rt) * 256 + e];
            v += red[(1 * R * MT + rt) * 256 + e];
            v += red[(2 * R * MT + rt) * 256 + e];
            v += red[(3 * R * MT + rt) * 256 + e];
            const int m = m0 + t * 16 + 4 * (l2 >> 4) + i;
            const int n = n0 + r * 16 + (l2 & 15);
            if (m < M && n < N) {
                v *= inv_scale[m];
                if (residual) v = residual[(size_t)m * N + n] + v;
                out[(size_t)m * N + n] = v;
            }
        }
        __syncthreads();
    }
}

// ---------------------------------------------------------------- fallback: exact dequantised values, float32 FMAs
__device__ __forceinline__ float deq_elem(int fmt, const uint8_t *row, int k) {
    if (fmt == VX_Q4_0) {
        const uint8_t *b = row + (size_t)(k >> 5) * 18;
        int i = k & 31;
        uint8_t bv = b[2 + (i & 15)];
        int q = (i < 16) ? (bv & 0xF) : (bv >> 4);
        return __fmul_rn(h2f((uint16_t)(b[0] | (b[1] << 8))), (float)(q - 8));
    }
    if (fmt == VX_Q8_0) {
        const uint8_t *b = row + (size_t)(k >> 5) * 34;
        return __fmul_rn(h2f((uint16_t)(b[0] | (b[1] << 8))), (float)(int8_t)b[2 + (k & 31)]);
    }
    if (fmt == VX_Q4_K) {
        const uint8_t *b = row + (size_t)(k >> 8) * 144;
        int e = k & 255, grp = e >> 6, l = e & 31, hi = (e >> 5) & 1, j = grp * 2 + hi;
        const uint8_t *q = b + 4;
        uint32_t sc, mn;
        if (j < 4) {
            sc = q[j] & 63;
            mn = q[j + 4] & 63;
        } else {
            sc = (q[j + 4] & 0x0F) | ((q[j - 4] >> 6) << 4);
            mn = (q[j + 4] >> 4) | ((q[j] >> 6) << 4);
        }
        float d1 = __fmul_rn(h2f((uint16_t)(b[0] | (b[1] << 8))), (float)sc);
        float dm1 = __fmul_rn(h2f((uint16_t)(b[2] | (b[3] << 8))), (float)mn);
        uint8_t bv = b[16 + grp * 32 + l];
        int qq = hi ? (bv >> 4) : (bv & 0xF);
        return __fsub_rn(__fmul_rn(d1, (float)qq), dm1);
    }
    // Q6_K, dequant.go:272-331
    const uint8_t *b = row + (size_t)(k >> 8) * 210;
    int e = k & 255, nn = e >> 7, r = e & 127, quad = r >> 5, l = r & 31, is = l >> 4;
    const uint8_t *ql = b + nn * 64, *qh = b + 128 + nn * 32;
    const int8_t *sc = (const int8_t *)b + 192 + nn * 8;
    uint8_t qlb = ql[l + ((quad & 1) ? 32 : 0)];
    int lo4 = (quad >= 2) ? (qlb >> 4) : (qlb & 0xF);
    int hi2 = (qh[l] >> (2 * quad)) & 3;
    int q = (lo4 | (hi2 << 4)) - 32;
    float d = h2f((uint16_t)(b[208] | (b[209] << 8)));
    return __fmul_rn(__fmul_rn(d, (float)sc[is + 2 * quad]), (float)q);
}

constexpr int FB_M = 8;
// grid = (N, ceil(M/FB_M)); block = 64 (one wave).
__global__ void __launch_bounds__(64) qgemm_fallback_kernel(int fmt, const uint8_t *__restrict__ W,
                                                            const float *__restrict__ a, float *__restrict__ out,
                                                            const float *__restrict__ residual, int M, int N, int K,
                                                            size_t row_bytes) {
    const int n = blockIdx.x, m0 = blockIdx.y * FB_M, lane = threadIdx.x;
    const uint8_t *row = W + (size_t)n * row_bytes;
    float acc[FB_M];
#pragma unroll
    for (int i = 0; i < FB_M; i++) acc[i] = 0.f;
    for (int k = lane; k < K; k += 64) {
        float w = deq_elem(fmt, row, k);
#pragma unroll
        for (int i = 0; i < FB_M; i++)
            if (m0 + i < M) acc[i] = fmaf(a[(size_t)(m0 + i) * K + k], w, acc[i]);
    }
#pragma unroll
    for (int i = 0; i < FB_M; i++) {
        float v = acc[i];
        for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
        if (lane == 0 && m0 + i < M) {
            if (residual) v = residual[(size_t)(m0 + i) * N + n] + v;
            out[(size_t)(m0 + i) * N + n] = v;
        }
    }
}

size_t fmt_row_bytes(int fmt, int k) {
    switch (fmt) {
    case VX_Q4_0: return (size_t)k / 32 * 18;
    case VX_Q8_0: return (size_t)k / 32 * 34;
    case VX_Q4_K: return (size_t)k / 256 * 144;
    case VX_Q6_K: return (size_t)k / 256 * 210;
    }
    return 0;
}

template <class F, int R>
int launch_fast_r(vx_backend *be, const uint8_t *W, const _Float16 *hi, const _Float16 *lo, const float *inv,
                  const float *bsum, float *out, const float *residual, int M, int Mpad, int N, int K) {
    int grid = ceil_div(N, 16 * R);
    if (Mpad <= 16)
        qgemm_kernel<F, R, 1><<<grid, 256, 0, be->stream>>>(W, hi, lo, inv, bsum, out, residual, M, Mpad, N, K);
    else
        qgemm_kernel<F, R, 2><<<grid, 256, 0, be->stream>>>(W, hi, lo, inv, bsum, out, residual, M, Mpad, N, K);
    VX_CHECK_LAUNCH();
    return VX_OK;
}

template <class F>
int launch_fast(vx_backend *be, const uint8_t *W, const _Float16 *hi, const _Float16 *lo, const float *inv,
                const float *bsum, float *out, const float *residual, int M, int Mpad, int N, int K) {
    // more rows per wave reuse each activation fetch, but the launch still has to fill 256 CUs
    if (N >= 16 * 2 * 512) return launch_fast_r<F, 2>(be, W, hi, lo, inv, bsum, out, residual, M, Mpad, N, K);
    return launch_fast_r<F, 1>(be, W, hi, lo, inv, bsum, out, residual, M, Mpad, N, K);
}

}  // namespace

extern "C" {

int vx_matmul_quant(vx_backend *be, int fmt, const float *a, const void *b, float *out, const float *residual, int m,
                    int n, int k) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(a && b && out, "vx_matmul_quant: null pointer");
    VX_REQUIRE(m >= 0 && n >= 0 && k > 0, "vx_matmul_quant: bad shape %dx%dx%d", m, n, k);
    int blk = (fmt == VX_Q4_0 || fmt == VX_Q8_0) ? 32 : 256;
    if (fmt != VX_Q4_0 && fmt != VX_Q8_0 && fmt != VX_Q4_K && fmt != VX_Q6_K) {
        set_error("vx_matmul_quant: unknown format %d", fmt);
        return VX_ERR_UNSUPPORTED;
    }
    VX_REQUIRE(k % blk == 0, "vx_matmul_quant: K=%d is not a multiple of the block size %d", k, blk);
    if (m == 0 || n == 0) return VX_OK;
    const size_t rb = fmt_row_bytes(fmt, k);
    const bool fast = fmt != VX_Q6_K && (k % 256 == 0) && (rb % 16 == 0) && ((uintptr_t)b % 16 == 0);
    if (!fast) {
        dim3 grid(n, ceil_div(m, FB_M));
        qgemm_fallback_kernel<<<grid, 64, 0, be->stream>>>(fmt, (const uint8_t *)b, a, out, residual, m, n, k, rb);
        VX_CHECK_LAUNCH();
        return VX_OK;
    }
    const int mpad = ceil_div(m, 16) * 16 <= 16 ? 16 : ceil_div(m, 32) * 32;
    const size_t hl = (size_t)mpad * k * sizeof(_Float16);
    const size_t need = 2 * hl + (size_t)mpad * 4 + (size_t)(k / 32) * mpad * 4 + 256;
    rc = ensure_ws(be, &be->gemm_ws, &be->gemm_ws_bytes, need, "quantized matmul");
    if (rc) return rc;
    _Float16 *hi = (_Float16 *)be->gemm_ws;
    _Float16 *lo = (_Float16 *)((char *)be->gemm_ws + hl);
    float *inv = (float *)((char *)be->gemm_ws + 2 * hl);
    float *bsum = inv + mpad + (64 - mpad % 64) % 64;  // keep 16-byte alignment for float4 loads
    split_act_kernel<<<mpad, 256, 0, be->stream>>>(a, m, k, fmt, hi, lo, inv, bsum, mpad);
    VX_CHECK_LAUNCH();
    const uint8_t *W = (const uint8_t *)b;
    switch (fmt) {
    case VX_Q4_0: return launch_fast<PQ4_0>(be, W, hi, lo, inv, bsum, out, residual, m, mpad, n, k);
    case VX_Q8_0: return launch_fast<PQ8_0>(be, W, hi, lo, inv, bsum, out, residual, m, mpad, n, k);
    default: return launch_fast<PQ4_K>(be, W, hi, lo, inv, bsum, out, residual, m, mpad, n, k);
    }
}

int vx_matmul_q4_0(vx_backend *be, const float *a, const void *b, float *out, int m, int n, int k) {
    return vx_matmul_quant(be, VX_Q4_0, a, b, out, nullptr, m, n, k);
}
int vx_matmul_q4_k(vx_backend *be, const float *a, const void *b, float *out, int m, int n, int k) {
    return vx_matmul_quant(be, VX_Q4_K, a, b, out, nullptr, m, n, k);
}
int vx_matmul_q6_k(vx_backend *be, const float *a, const void *b, float *out, int m, int n, int k) {
    return vx_matmul_quant(be, VX_Q6_K, a, b, out, nullptr, m, n, k);
}
int vx_matmul_q8_0(vx_backend *be, const float *a, const void *b, float *out, int m, int n, int k) {
    return vx_matmul_quant(be, VX_Q8_0, a, b, out, nullptr, m, n, k);
}

static int unsupported(const char *name) {
    set_error("%s: format not implemented by this backend", name);
    return VX_ERR_UNSUPPORTED;
}
int vx_matmul_q5_k(vx_backend *, const float *, const void *, float *, int, int, int) { return unsupported("vx_matmul_q5_k"); }
int vx_matmul_q5_0(vx_backend *, const float *, const void *, float *, int, int, int) { return unsupported("vx_matmul_q5_0"); }
int vx_matmul_bf16(vx_backend *, const float *, const void *, float *, int, int, int) { return unsupported("vx_matmul_bf16"); }

}  // extern "C"
