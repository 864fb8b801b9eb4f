// Quantized matmul C[M,N] = A[M,K] * B^T with B in raw GGUF blocks (Q4_0, Q8_0, Q4_K, Q6_K, Q5_0, Q5_K) or BF16.
// Replaces QuantizedMatMul.MatMulQ4_0/Q4_K/Q6_K/Q8_0/Q5_0/Q5_K/BF16 (inference/backend/backend.go:47-81).
//
// Fast path (the six block formats; K a multiple of 256, the matrix on a 16-byte boundary), two phases:
//
//  1. prepare: every activation row is scaled by a power of two and split into
//     hi = f16(x), lo = f16(x - hi) (together ~22 significant bits, the float32 level). Both are
//     written as ready-made MFMA operand tiles A[kstep][mtile][hi|lo][lane][8]: lane (g, r) of
//     tile `mtile` holds row 16*mtile + r and the eight k-slots 8g..8g+7 of 32-element block
//     `kstep`. Slot p of a block holds element PERM[p], the order in which every format's
//     unpacking produces its eight values per lane, so one prepared activation serves any weight
//     format. RMSNorm and SiLU*up have fused prepare variants; a prepared activation can be
//     multiplied by several weights (Q/K/V, gate/up).
//  2. qgemm_kernel: a workgroup owns 64*R weight rows (a wave 16*R of them) and one K slice.
//     Per 256-element chunk the workgroup copies the activation tiles (contiguous, coalesced)
//     into LDS once for its 4 waves, each wave stages its rows' raw blocks into LDS with 16-byte
//     loads, unpacks the integer codes to exact f16 values in registers and issues
//     v_mfma_f32_16x16x32_f16 twice per block (hi, lo). The block scale multiplies the float32
//     MFMA result, never the f16 operand, so the weights entering the sum are exactly the
//     format's integers. With KS > 1 slices the partial sums go to scratch and
//     qgemm_reduce_kernel adds them in slice order (deterministic), applies the row scale and
//     the optional residual.
//     Decode batches (2 to 64 rows) of Q4_0, Q8_0 and Q4_K take qgemm_wave_kernel (qgemm_wave.h)
//     instead: one workgroup per compute unit, its waves split K, activation tiles go from L2
//     straight to registers (up to 32 rows: matrices whose rows fit one round of workgroups; 33 to
//     64 rows: four activation tiles a step, several rounds); BF16 matrices take it at any batch size.
//     Q8_0 batches of more than 96 rows take qgemm_rows_kernel (same header): the waves split the
//     weight rows and share 64 activation rows' tiles through LDS.
//  Each output element depends only on its own activation row and weight row and the launch
//  shape depends on (N, K) and on which of these kernels the batch size selects, so a row gives
//  the same bits in any two batches of one range (the property the reference keeps by looping
//  M=1 kernels, backend/metal/backend.go:777-779).
//
// Fallback (odd shapes): one wave per output column, float32 FMAs on the exact dequantised values.
#include <stdlib.h>

#include "common.h"
#include <cstring>
#include <algorithm>

#include "prep_tiles.h"
#include "qgemm_shared.h"

using namespace vx;

namespace {

typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float h2f(uint16_t h) {
    _Float16 v;
    __builtin_memcpy(&v, &h, 2);
    return (float)v;
}

// Slot j of lane group g (operand position p = 8g+j) holds block element
//   {4g, 4g+2, 16+4g, 16+4g+2, 4g+1, 4g+3, 16+4g+1, 16+4g+3}[j]:
// a lane needs elements 4g..4g+3 and 16+4g..16+4g+3, i.e. two aligned float4 of the source row.

// ---------------------------------------------------------------- activation prepare
// (PrepView, the workspace layout and write_chunk: prep_tiles.h)

enum { PREP_PLAIN = 0, PREP_RMSNORM = 1, PREP_SILU_MUL = 2, PREP_GELU_MUL = 3, PREP_GELU = 4 };

__device__ __forceinline__ float sigmoid_ref(float v) { return 1.0f / (1.0f + (float)exp((double)(-v))); }
// GELU, tanh form, with the reference's operation order (backend/cpu/cpu.go:440-473; the arithmetic of vx_gelu)
__device__ __forceinline__ float gelu_tanh_ref(float v) {
#pragma clang fp contract(off)
    const float x3 = v * v * v;
    const float arg = 0.7978845608f * (v + 0.044715f * x3);
    const float th = (float)tanh((double)arg);
    return 0.5f * v * (1.0f + th);
}
// the activation modes: SiLU(a) * b, GELU(a) * b, or GELU(a) alone (b unused)
template <int MODE> __device__ __forceinline__ float gated(float a, float b) {
    if (MODE == PREP_GELU) return gelu_tanh_ref(a);
    return MODE == PREP_GELU_MUL ? __fmul_rn(gelu_tanh_ref(a), b) : __fmul_rn(__fmul_rn(a, sigmoid_ref(a)), b);
}
template <int MODE> constexpr bool is_act_mode() { return MODE == PREP_SILU_MUL || MODE == PREP_GELU_MUL || MODE == PREP_GELU; }

// grid = Mpad rows, block = 256.
//   PREP_PLAIN:    y = a
//   PREP_RMSNORM:  y = (a / rms) * w            (backend/cpu/cpu.go:200-220), optional f32 copy to `fout`
//   PREP_SILU_MUL: y = (a*sigmoid(a)) * b       (backend/cpu/cpu.go:390-400), optional f32 copy to `fout`
//   PREP_GELU_MUL: y = gelu(a) * b              (backend/cpu/cpu.go:462-473), optional f32 copy to `fout`
//   PREP_GELU:     y = gelu(a)                  (backend/cpu/cpu.go:440-460), optional f32 copy to `fout`
// STAGE: keep the row's output values in LDS between the two passes (K*4 bytes of dynamic LDS);
// otherwise pass 2 recomputes them.
constexpr int PREP_THREADS = 1024;  // shared by every kernel that writes prepared tiles: the row statistics
                                    // are summed in an order that depends on it, and fused and unfused
                                    // producers must agree bit for bit

// ss + a^2 + b^2 + c^2 + d^2 in one fixed order of fused multiply-adds
__device__ __forceinline__ float sumsq4(float ss, float a, float b, float c, float d) {
    return __fmaf_rn(d, d, __fmaf_rn(c, c, __fmaf_rn(b, b, __fmaf_rn(a, a, ss))));
}

// amax / sum of squares over the workgroup; every thread gets the totals
__device__ __forceinline__ void row_stats(float &amax, float &ss, float *sm) {
    constexpr int NW = PREP_THREADS / 64;
    for (int off = 32; off > 0; off >>= 1) {
        amax = fmaxf(amax, __shfl_xor(amax, off, 64));
        ss += __shfl_xor(ss, off, 64);
    }
    const int tid = threadIdx.x;
    if ((tid & 63) == 0) {
        sm[tid >> 6] = amax;
        sm[NW + (tid >> 6)] = ss;
    }
    __syncthreads();
    amax = sm[0];
    ss = sm[NW];
    for (int i = 1; i < NW; i++) {
        amax = fmaxf(amax, sm[i]);
        ss += sm[NW + i];
    }
}

template <int MODE, bool STAGE>
__global__ void __launch_bounds__(PREP_THREADS) prepare_kernel(const float *__restrict__ a, const float *__restrict__ b,
                                                      float *__restrict__ fout, int M, int K, float eps,
                                                      PrepView pv, int Mpad) {
    extern __shared__ __attribute__((aligned(16))) float ybuf[];
    __shared__ float sm[2 * (PREP_THREADS / 64)];
    const int r = blockIdx.x, tid = threadIdx.x;
    const int mtiles = Mpad / 16, mt = r >> 4, ln = r & 15;
    const int npairs = K / 8;  // (kstep, g) pairs: 8 output slots each
    if (r >= M) {
        const half8 z = {0, 0, 0, 0, 0, 0, 0, 0};
        for (int p = tid; p < npairs; p += PREP_THREADS) {
            const int ks = p >> 2, g = p & 3;
            half8 *t = pv.tiles + ((size_t)(ks * mtiles + mt) * 2) * 64 + g * 16 + ln;
            t[0] = z;
            t[64] = z;
            if (g == 0) pv.bsum[(size_t)ks * Mpad + r] = 0.f;
        }
        if (tid == 0) pv.inv_scale[r] = 0.f;
        for (int c = tid; c < K / 256; c += blockDim.x) pv.cscale[(size_t)c * Mpad + r] = 0.f;
        return;
    }
    const float *ar = a + (size_t)r * K;
    const float *br = (MODE == PREP_RMSNORM) ? b : (b ? b + (size_t)r * K : nullptr);
    // pass 1: row statistics (SiLU*up values are staged in LDS for pass 2 when STAGE)
    float amax = 0.f, ss = 0.f;
    for (int k = tid * 4; k < K; k += PREP_THREADS * 4) {
        const float4 x = *(const float4 *)(ar + k);
        float y[4] = {x.x, x.y, x.z, x.w};
        if (MODE == PREP_RMSNORM) {
            ss = sumsq4(ss, x.x, x.y, x.z, x.w);
        } else if (is_act_mode<MODE>()) {
            const float4 u = MODE == PREP_GELU ? make_float4(0.f, 0.f, 0.f, 0.f) : *(const float4 *)(br + k);
            y[0] = gated<MODE>(x.x, u.x);
            y[1] = gated<MODE>(x.y, u.y);
            y[2] = gated<MODE>(x.z, u.z);
            y[3] = gated<MODE>(x.w, u.w);
        }
        if (STAGE && is_act_mode<MODE>()) *(float4 *)(ybuf + k) = make_float4(y[0], y[1], y[2], y[3]);
        if (MODE == PREP_RMSNORM) {
            const float4 w = *(const float4 *)(br + k);
            y[0] *= w.x; y[1] *= w.y; y[2] *= w.z; y[3] *= w.w;
        }
        amax = fmaxf(amax, fmaxf(fmaxf(fabsf(y[0]), fabsf(y[1])), fmaxf(fabsf(y[2]), fabsf(y[3]))));
    }
    row_stats(amax, ss, sm);
    float rms = 1.f;
    if (MODE == PREP_RMSNORM) {
        rms = (float)sqrt((double)(ss / (float)K + eps));
        amax = amax / rms * 1.0001f;  // bound of |(x/rms)*w| up to rounding
    }
    float s = 1.f, inv = 1.f;
    if (amax > 0.f && amax < INFINITY) {
        int ex;
        (void)frexpf(amax, &ex);   // amax = f * 2^ex, f in [0.5,1)
        s = ldexpf(1.f, 13 - ex);  // amax*s in [2^12, 2^13): far from the f16 limit 65504
        inv = ldexpf(1.f, ex - 13);
    }
    if (tid == 0) pv.inv_scale[r] = inv;
    for (int c = tid; c < K / 256; c += blockDim.x) pv.cscale[(size_t)c * Mpad + r] = 1.f;
    // pass 2: one (kstep, g) pair per iteration = elements 4g..4g+3 and 16+4g..16+4g+3 of the block
    for (int p = tid; p < npairs; p += PREP_THREADS) {
        const int ks = p >> 2, g = p & 3;
        const int k0 = ks * 32 + 4 * g;
        const float *src = (STAGE && is_act_mode<MODE>()) ? ybuf : ar;
        float4 xa = *(const float4 *)(src + k0), xb = *(const float4 *)(src + k0 + 16);
        float ya[4] = {xa.x, xa.y, xa.z, xa.w}, yb[4] = {xb.x, xb.y, xb.z, xb.w};
        if (MODE == PREP_RMSNORM) {
            const float4 wa = *(const float4 *)(br + k0), wb = *(const float4 *)(br + k0 + 16);
            const float wv[8] = {wa.x, wa.y, wa.z, wa.w, wb.x, wb.y, wb.z, wb.w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                ya[i] = __fmul_rn(ya[i] / rms, wv[i]);
                yb[i] = __fmul_rn(yb[i] / rms, wv[4 + i]);
            }
        } else if (is_act_mode<MODE>() && !STAGE) {
            const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
            const float4 ua = MODE == PREP_GELU ? zero4 : *(const float4 *)(br + k0), ub = MODE == PREP_GELU ? zero4 : *(const float4 *)(br + k0 + 16);
            const float uv[8] = {ua.x, ua.y, ua.z, ua.w, ub.x, ub.y, ub.z, ub.w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                ya[i] = gated<MODE>(ya[i], uv[i]);
                yb[i] = gated<MODE>(yb[i], uv[4 + i]);
            }
        }
        if (MODE != PREP_PLAIN && fout) {
            *(float4 *)(fout + (size_t)r * K + k0) = make_float4(ya[0], ya[1], ya[2], ya[3]);
            *(float4 *)(fout + (size_t)r * K + k0 + 16) = make_float4(yb[0], yb[1], yb[2], yb[3]);
        }
        // slots: {4g, 4g+2, 16+4g, 16+4g+2, 4g+1, 4g+3, 16+4g+1, 16+4g+3}
        const float v[8] = {ya[0] * s, ya[2] * s, yb[0] * s, yb[2] * s, ya[1] * s, ya[3] * s, yb[1] * s, yb[3] * s};
        half8 h, l;
        float bs = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            h[i] = (_Float16)v[i];
            l[i] = (_Float16)(v[i] - (float)h[i]);
            bs += v[i];
        }
        half8 *t = pv.tiles + ((size_t)(ks * mtiles + mt) * 2) * 64 + g * 16 + ln;
        t[0] = h;
        t[64] = l;
        // the 4 lanes g = 0..3 of one kstep are adjacent threads (p = 4*ks + g)
        bs += __shfl_xor(bs, 1, 64);
        bs += __shfl_xor(bs, 2, 64);
        if (g == 0) pv.bsum[(size_t)ks * Mpad + r] = bs;
    }
}

// ---------------------------------------------------------------- weight unpacking per format
// 4 bytes at byte offset `off` (any alignment) of an LDS array. Indexing the array keeps the access
// in the LDS address space (ds_read2_b32); a pointer rebuilt from an integer would become a flat load.
__device__ __forceinline__ uint32_t lds_u32_unaligned(const uint8_t *base, int off) {
    const uint32_t *w = (const uint32_t *)base;
    const int i = off >> 2;
    return __builtin_amdgcn_alignbyte(w[i + 1], w[i], (uint32_t)(off & 3));
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

typedef _Float16 half4v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ half4v first16(half8 v) { return __builtin_shufflevector(v, v, 0, 1, 4, 5); }
__device__ __forceinline__ half4v second16(half8 v) { return __builtin_shufflevector(v, v, 2, 3, 6, 7); }

struct StepW {  // what one MFMA step needs from the weights
    half8 b;    // exact integer codes as f16, in slot order
    float d;    // multiplies the MFMA result
    float dm;   // multiplies the activation block sum and is subtracted (Q4_K); Q6_K: the scale of the
                // step's second 16 elements (d is that of the first 16); else 0
};

// CHUNK_BYTES = raw bytes per weight row for 8 steps (256 elements). ROW_PIECES = 16-byte pieces staged per
// row and chunk: CHUNK_BYTES / 16 where rows start on 16-byte boundaries (ALIGNED), else enough to cover the
// chunk from the aligned address below its first byte. TWO_SCALES: a step's two halves of 16 elements carry
// different scales, so a step is two 16x16x16 MFMAs per activation half instead of one 16x16x32.
struct PQ4_0 {
    static constexpr int CHUNK_BYTES = 144;
    static constexpr int ROW_PIECES = CHUNK_BYTES / 16;
    static constexpr bool ALIGNED = true, TWO_SCALES = false;
    // Rows sit back to back in LDS: 144 bytes = 36 dwords, and 36*row mod 64 takes 16 distinct multiples of 4
    // for the 16 rows of a tile, so the 4 lane groups of every row read 64 different banks.
    static constexpr int PITCH = 144;
    static constexpr int MIN_WAVES = 2;
    static constexpr bool HAS_MIN = false;
    static __host__ __device__ size_t row_bytes(int K) { return (size_t)K / 32 * 18; }
    struct Raw { uint32_t lo, hi, sh; uint16_t d; };
    // LDS reads of one step (no arithmetic on the loaded values): two dwords around the 4 nibble bytes, the scale
    static __device__ __forceinline__ Raw read(const uint8_t *base, int row_off, int step, int g) {
        const int bo = row_off + step * 18, off = bo + 2 + 4 * g;  // bytes 4g..4g+3 of the block
        const uint32_t *w = (const uint32_t *)base;
        Raw r;
        r.lo = w[off >> 2];
        r.hi = w[(off >> 2) + 1];
        r.sh = (uint32_t)(off & 3);
        r.d = *(const uint16_t *)(base + bo);
        return r;
    }
    static __device__ __forceinline__ StepW unpack(const Raw &x, int) {
        const uint32_t w = __builtin_amdgcn_alignbyte(x.hi, x.lo, x.sh);
        const half2v off = {(_Float16)1032.f, (_Float16)1032.f};  // 1024 + 8
        const uint32_t lo = w & 0x0F0F0F0Fu, hi = (w >> 4) & 0x0F0F0F0Fu, c64 = 0x64646464u;
        StepW r;  // byte b next to a 0x64 byte is the f16 1024 + b
        r.b = pack8(as_h2(__builtin_amdgcn_perm(lo, c64, 0x00060004u)) - off,   // low nibbles of bytes 0,2  -> 4g, 4g+2
                    as_h2(__builtin_amdgcn_perm(hi, c64, 0x00060004u)) - off,   // high nibbles of bytes 0,2 -> 16+4g, 16+4g+2
                    as_h2(__builtin_amdgcn_perm(lo, c64, 0x00070005u)) - off,   // low nibbles of bytes 1,3  -> 4g+1, 4g+3
                    as_h2(__builtin_amdgcn_perm(hi, c64, 0x00070005u)) - off);  // high nibbles of bytes 1,3 -> 16+4g+1, 16+4g+3
        r.d = h2f(x.d);
        r.dm = 0.f;
        return r;
    }
};

struct PQ8_0 {
    static constexpr int CHUNK_BYTES = 272;
    static constexpr int ROW_PIECES = CHUNK_BYTES / 16;
    static constexpr bool ALIGNED = true, TWO_SCALES = false;
    static constexpr int PITCH = 272;  // 68 dwords: (PITCH/4) % 8 == 4, conflict free like Q4_0's 36
    static constexpr int MIN_WAVES = 2;
    static constexpr bool HAS_MIN = false;
    static __host__ __device__ size_t row_bytes(int K) { return (size_t)K / 32 * 34; }
    struct Raw { uint32_t a0, a1, b0, b1, sh; uint16_t d; };
    static __device__ __forceinline__ Raw read(const uint8_t *base, int row_off, int step, int g) {
        const int bo = row_off + step * 34, off = bo + 2 + 4 * g;  // elements 4g..4g+3; 16+4g.. are 16 bytes on
        const uint32_t *w = (const uint32_t *)base;
        Raw r;
        r.a0 = w[off >> 2];
        r.a1 = w[(off >> 2) + 1];
        r.b0 = w[(off >> 2) + 4];
        r.b1 = w[(off >> 2) + 5];
        r.sh = (uint32_t)(off & 3);
        r.d = *(const uint16_t *)(base + bo);
        return r;
    }
    static __device__ __forceinline__ StepW unpack(const Raw &x, int) {
        const uint32_t w0 = __builtin_amdgcn_alignbyte(x.a1, x.a0, x.sh) ^ 0x80808080u;
        const uint32_t w1 = __builtin_amdgcn_alignbyte(x.b1, x.b0, x.sh) ^ 0x80808080u;
        const half2v off = {(_Float16)1152.f, (_Float16)1152.f};  // 1024 + 128
        const uint32_t c64 = 0x64646464u;
        StepW r;
        r.b = pack8(as_h2(__builtin_amdgcn_perm(w0, c64, 0x00060004u)) - off,   // bytes 0,2 of w0
                    as_h2(__builtin_amdgcn_perm(w1, c64, 0x00060004u)) - off,   // bytes 0,2 of w1
                    as_h2(__builtin_amdgcn_perm(w0, c64, 0x00070005u)) - off,   // bytes 1,3 of w0
                    as_h2(__builtin_amdgcn_perm(w1, c64, 0x00070005u)) - off);  // bytes 1,3 of w1
        r.d = h2f(x.d);
        r.dm = 0.f;
        return r;
    }
};

struct PQ4_K {
    static constexpr int CHUNK_BYTES = 144;  // one super-block = 8 sub-blocks of 32
    static constexpr int ROW_PIECES = CHUNK_BYTES / 16;
    static constexpr bool ALIGNED = true, TWO_SCALES = false;
    static constexpr int PITCH = 144;
    static constexpr int MIN_WAVES = 2;  // the min-term bookkeeping needs more registers than 3 waves leave
    static constexpr bool HAS_MIN = true;
    static __host__ __device__ size_t row_bytes(int K) { return (size_t)K / 256 * 144; }
    struct Raw { uint32_t w0, w1, hd, s0, s1, s2; };
    static __device__ __forceinline__ Raw read(const uint8_t *base, int row_off, int j, int g) {
        const uint32_t *sb = (const uint32_t *)(base + row_off);
        const uint32_t *qp = sb + 4 + 8 * (j >> 1);
        Raw r;
        r.w0 = qp[g];      // elements 4g..4g+3 of both sub-blocks of the pair (low / high nibbles)
        r.w1 = qp[4 + g];  // elements 16+4g..
        r.hd = sb[0];      // d, dmin
        r.s0 = sb[1];      // the 12 bytes of 6-bit scales and mins
        r.s1 = sb[2];
        r.s2 = sb[3];
        return r;
    }
    static __device__ __forceinline__ StepW unpack(const Raw &x, int j) {
        const uint32_t w0 = (x.w0 >> (4 * (j & 1))) & 0x0F0F0F0Fu, w1 = (x.w1 >> (4 * (j & 1))) & 0x0F0F0F0Fu;
        const half2v off = {(_Float16)1024.f, (_Float16)1024.f};
        const uint32_t c64 = 0x64646464u;
        auto q = [&](int i) -> uint32_t {  // byte i of the scales field
            const uint32_t wd = i < 4 ? x.s0 : (i < 8 ? x.s1 : x.s2);
            return (wd >> (8 * (i & 3))) & 0xFFu;
        };
        uint32_t sc, mn;  // pkg/gguf/dequant.go:400-409
        if (j < 4) {
            sc = q(j) & 63;
            mn = q(j + 4) & 63;
        } else {
            sc = (q(j + 4) & 0x0F) | ((q(j - 4) >> 6) << 4);
            mn = (q(j + 4) >> 4) | ((q(j) >> 6) << 4);
        }
        StepW r;
        r.b = pack8(as_h2(__builtin_amdgcn_perm(w0, c64, 0x00060004u)) - off, as_h2(__builtin_amdgcn_perm(w1, c64, 0x00060004u)) - off,
                    as_h2(__builtin_amdgcn_perm(w0, c64, 0x00070005u)) - off, as_h2(__builtin_amdgcn_perm(w1, c64, 0x00070005u)) - off);
        r.d = h2f((uint16_t)(x.hd & 0xFFFF)) * (float)sc;
        r.dm = h2f((uint16_t)(x.hd >> 16)) * (float)mn;
        return r;
    }
};

// bit i of the 4 low bits of b into bit 4 of byte i
__device__ __forceinline__ uint32_t fifth_bits4(uint32_t b) { return ((b * 0x00204081u) & 0x01010101u) << 4; }

// Q5_0 (dequant.go:100-145): 22-byte blocks [f16 d][u32 qh][16 nibble bytes]; element i = nibble | bit i of qh << 4,
// value (q - 16) d. Eight blocks are 176 bytes, so rows and chunks start on 16-byte boundaries.
struct PQ5_0 {
    static constexpr int CHUNK_BYTES = 176;
    static constexpr int ROW_PIECES = CHUNK_BYTES / 16;
    static constexpr bool ALIGNED = true, TWO_SCALES = false;
    static constexpr int PITCH = 176;  // 44 dwords: (PITCH/4) % 8 == 4
    static constexpr int MIN_WAVES = 2;
    static constexpr bool HAS_MIN = false;
    static __host__ __device__ size_t row_bytes(int K) { return (size_t)K / 32 * 22; }
    struct Raw { uint32_t lo, hi, sh, q0, q1, qsh, g; uint16_t d; };
    static __device__ __forceinline__ Raw read(const uint8_t *base, int row_off, int step, int g) {
        const int bo = row_off + step * 22, off = bo + 6 + 4 * g;  // nibble bytes 4g..4g+3; qh sits at bo + 2
        const uint32_t *w = (const uint32_t *)base;
        Raw r;
        r.lo = w[off >> 2];
        r.hi = w[(off >> 2) + 1];
        r.sh = (uint32_t)(off & 3);
        r.q0 = w[(bo + 2) >> 2];
        r.q1 = w[((bo + 2) >> 2) + 1];
        r.qsh = (uint32_t)((bo + 2) & 3);
        r.g = (uint32_t)g;
        r.d = *(const uint16_t *)(base + bo);
        return r;
    }
    static __device__ __forceinline__ StepW unpack(const Raw &x, int) {
        const uint32_t w = __builtin_amdgcn_alignbyte(x.hi, x.lo, x.sh);
        const uint32_t qh = __builtin_amdgcn_alignbyte(x.q1, x.q0, x.qsh);
        const half2v off = {(_Float16)1040.f, (_Float16)1040.f};  // 1024 + 16
        const uint32_t lo = (w & 0x0F0F0F0Fu) | fifth_bits4((qh >> (4 * x.g)) & 15u);
        const uint32_t hi = ((w >> 4) & 0x0F0F0F0Fu) | fifth_bits4((qh >> (16 + 4 * x.g)) & 15u);
        const uint32_t c64 = 0x64646464u;
        StepW r;
        r.b = pack8(as_h2(__builtin_amdgcn_perm(lo, c64, 0x00060004u)) - off, as_h2(__builtin_amdgcn_perm(hi, c64, 0x00060004u)) - off,
                    as_h2(__builtin_amdgcn_perm(lo, c64, 0x00070005u)) - off, as_h2(__builtin_amdgcn_perm(hi, c64, 0x00070005u)) - off);
        r.d = h2f(x.d);
        r.dm = 0.f;
        return r;
    }
};

// Q5_K (dequant.go:423-500): Q4_K's header and 6-bit scales, then qh[32] and qs[128]; bit j of qh byte l is the
// fifth bit of element l of sub-block j.
struct PQ5_K {
    static constexpr int CHUNK_BYTES = 176;
    static constexpr int ROW_PIECES = CHUNK_BYTES / 16;
    static constexpr bool ALIGNED = true, TWO_SCALES = false;
    static constexpr int PITCH = 176;
    static constexpr int MIN_WAVES = 2;
    static constexpr bool HAS_MIN = true;
    static __host__ __device__ size_t row_bytes(int K) { return (size_t)K / 256 * 176; }
    // what a step keeps between its LDS reads and its MFMA: the sub-block's fifth bits (bit 0 of each byte: elements
    // 4g.., bit 1: 16+4g..) and its 6-bit scale and min are picked out at once, so that fewer registers stay live
    struct Raw { uint32_t w0, w1, h, hd, scmn; };
    static __device__ __forceinline__ Raw read(const uint8_t *base, int row_off, int j, int g) {
        const uint32_t *sb = (const uint32_t *)(base + row_off);
        const uint32_t *qp = sb + 12 + 8 * (j >> 1);
        Raw r;
        r.w0 = qp[g];      // elements 4g..4g+3 of both sub-blocks of the pair (low / high nibbles)
        r.w1 = qp[4 + g];  // elements 16+4g..
        r.h = ((sb[4 + g] >> j) & 0x01010101u) | (((sb[8 + g] >> j) & 0x01010101u) << 1);
        r.hd = sb[0];
        const uint8_t *q = base + row_off + 4;  // pkg/gguf/dequant.go:400-409
        uint32_t sc, mn;
        if (j < 4) {
            sc = q[j] & 63;
            mn = q[j + 4] & 63;
        } else {
            sc = (q[j + 4] & 0x0F) | ((q[j - 4] >> 6) << 4);
            mn = (q[j + 4] >> 4) | ((q[j] >> 6) << 4);
        }
        r.scmn = sc | (mn << 8);
        return r;
    }
    static __device__ __forceinline__ StepW unpack(const Raw &x, int j) {
        const uint32_t w0 = ((x.w0 >> (4 * (j & 1))) & 0x0F0F0F0Fu) | ((x.h & 0x01010101u) << 4);
        const uint32_t w1 = ((x.w1 >> (4 * (j & 1))) & 0x0F0F0F0Fu) | ((x.h & 0x02020202u) << 3);
        const half2v off = {(_Float16)1024.f, (_Float16)1024.f};
        const uint32_t c64 = 0x64646464u;
        StepW r;
        r.b = pack8(as_h2(__builtin_amdgcn_perm(w0, c64, 0x00060004u)) - off, as_h2(__builtin_amdgcn_perm(w1, c64, 0x00060004u)) - off,
                    as_h2(__builtin_amdgcn_perm(w0, c64, 0x00070005u)) - off, as_h2(__builtin_amdgcn_perm(w1, c64, 0x00070005u)) - off);
        r.d = h2f((uint16_t)(x.hd & 0xFFFF)) * (float)(x.scmn & 0xFFu);
        r.dm = h2f((uint16_t)(x.hd >> 16)) * (float)(x.scmn >> 8);
        return r;
    }
};

constexpr int CH = 8;  // MFMA steps (32 elements each) per chunk

// Up to three weight matrices that share K and the activation (Q/K/V, gate/up) multiplied in one
// launch: output column n belongs to segment sg = first with n < n_end[sg], local row n - n_end[sg-1].
// Q6_K: 210-byte super-blocks (ql[128] | qh[64] | int8 scales[16] | f16 d), so rows start on 2-byte
// boundaries only. Element e = 128n + 32qt + p of a super-block: low nibble source ql[64n + 32(qt&1) + p]
// >> 4(qt>>1), high two bits qh[32n + p] >> 2qt, scale[8n + 2qt + p/16] (inference/pkg/gguf/dequant.go:272-331).
struct PQ6_K {
    static constexpr int CHUNK_BYTES = 210;
    static constexpr int ROW_PIECES = 14;  // shift <= 14 bytes, 14 + 210 = 224
    static constexpr bool ALIGNED = false, TWO_SCALES = true;
    static constexpr int PITCH = 240;  // 60 dwords: (PITCH/4) % 8 == 4
    static constexpr int MIN_WAVES = 2;
    static constexpr bool HAS_MIN = false;
    static __host__ __device__ size_t row_bytes(int K) { return (size_t)K / 256 * 210; }
    struct Raw { uint32_t l0, l1, l2, l3, h0, h1, h2, h3, sh; uint16_t sc, d; };
    static __device__ __forceinline__ Raw read(const uint8_t *base, int row_off, int j, int g) {
        const int n = j >> 2, qt = j & 3;
        const int lo = row_off + 64 * n + 32 * (qt & 1) + 4 * g;  // positions 4g..4g+3; 16+4g.. are 16 bytes on
        const int ho = row_off + 128 + 32 * n + 4 * g;
        const uint32_t *w = (const uint32_t *)base;
        Raw r;
        r.l0 = w[lo >> 2];
        r.l1 = w[(lo >> 2) + 1];
        r.l2 = w[(lo >> 2) + 4];
        r.l3 = w[(lo >> 2) + 5];
        r.h0 = w[ho >> 2];
        r.h1 = w[(ho >> 2) + 1];
        r.h2 = w[(ho >> 2) + 4];
        r.h3 = w[(ho >> 2) + 5];
        r.sh = (uint32_t)(row_off & 3);  // every offset above differs from row_off by a multiple of 4
        r.sc = *(const uint16_t *)(base + row_off + 192 + 8 * n + 2 * qt);
        r.d = *(const uint16_t *)(base + row_off + 208);
        return r;
    }
    static __device__ __forceinline__ StepW unpack(const Raw &x, int j) {
        const int qt = j & 3;
        const uint32_t ql0 = __builtin_amdgcn_alignbyte(x.l1, x.l0, x.sh), ql1 = __builtin_amdgcn_alignbyte(x.l3, x.l2, x.sh);
        const uint32_t qh0 = __builtin_amdgcn_alignbyte(x.h1, x.h0, x.sh), qh1 = __builtin_amdgcn_alignbyte(x.h3, x.h2, x.sh);
        const uint32_t w0 = ((ql0 >> (4 * (qt >> 1))) & 0x0F0F0F0Fu) | (((qh0 >> (2 * qt)) & 0x03030303u) << 4);
        const uint32_t w1 = ((ql1 >> (4 * (qt >> 1))) & 0x0F0F0F0Fu) | (((qh1 >> (2 * qt)) & 0x03030303u) << 4);
        const half2v off = {(_Float16)1056.f, (_Float16)1056.f};  // 1024 + 32
        const uint32_t c64 = 0x64646464u;
        StepW r;
        r.b = pack8(as_h2(__builtin_amdgcn_perm(w0, c64, 0x00060004u)) - off, as_h2(__builtin_amdgcn_perm(w1, c64, 0x00060004u)) - off,
                    as_h2(__builtin_amdgcn_perm(w0, c64, 0x00070005u)) - off, as_h2(__builtin_amdgcn_perm(w1, c64, 0x00070005u)) - off);
        const float d = h2f(x.d);
        r.d = d * (float)(int8_t)(x.sc & 0xFF);
        r.dm = d * (float)(int8_t)(x.sc >> 8);
        return r;
    }
};

struct Segs {
    const uint8_t *w[3];
    int n_end[3];
};
// Selects over values read once from the kernel arguments; indexing the arrays with a per-lane index
// would turn every row lookup into dependent memory loads.
__device__ __forceinline__ const uint8_t *seg_row(const Segs &sg, int n, size_t row_bytes) {
    const uint8_t *w0 = sg.w[0], *w1 = sg.w[1], *w2 = sg.w[2];
    const int e0 = sg.n_end[0], e1 = sg.n_end[1];
    const uint8_t *base = n < e0 ? w0 : (n < e1 ? w1 : w2);
    const int local = n < e0 ? n : (n < e1 ? n - e0 : n - e1);
    return base + (size_t)local * row_bytes;
}

// grid = (row groups of 64*R rows, KS k-slices, groups of MT activation tiles); block = 256.
template <class F, int R, int MT, bool SERIAL>
__global__ void __launch_bounds__(256, F::MIN_WAVES) qgemm_kernel(Segs segs, PrepView pv, float *__restrict__ out,
                                                    const float *__restrict__ residual, float *__restrict__ partial,
                                                    int M, int Mpad, int N, int K, int n_slices, int flags) {
    constexpr int ROWS_W = 16 * R;
    constexpr int PITCH = F::PITCH;
    constexpr int WPIECES = ROWS_W * F::ROW_PIECES;
    constexpr int WNL = (WPIECES + 63) / 64;
    constexpr int APIECES = CH * MT * 2 * 64;  // 16-byte pieces of one activation chunk
    constexpr int ANL = APIECES / 256;
    __shared__ __attribute__((aligned(16))) half8 a_lds[APIECES];
    __shared__ __attribute__((aligned(16))) uint8_t w_lds[4][ROWS_W * PITCH + 16];  // +16: the unaligned dword read may touch 4 bytes past the last row
    // formats with a min term: the chunk's activation block sums, [step][tile][row], staged with the tiles
    constexpr int NBS = CH * MT * 16;
    static_assert(NBS <= 256, "one block sum per thread");
    __shared__ __attribute__((aligned(16))) float bs_lds[F::HAS_MIN ? NBS : 4];

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int ln = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * (64 * R) + wave * ROWS_W;
    const int ks = blockIdx.y, mg = blockIdx.z;
    const int m0 = mg * 16 * MT;
    const int mtiles = Mpad / 16;
    const size_t row_bytes = F::row_bytes(K);
    const int steps_total = K / 32;
    const int n_chunks = (steps_total + CH - 1) / CH;
    // balanced slices: the first n_chunks % n_slices slices hold one chunk more
    const int sl_base = n_chunks / n_slices, sl_rem = n_chunks % n_slices;
    // SERIAL: this workgroup walks all slices itself, one after the other, and adds their sums in slice order:
    // the same bits as one workgroup per slice plus the reduction, without the partial sums' round trip
    constexpr bool serial = SERIAL;
    const int c_begin = serial ? 0 : ks * sl_base + min(ks, sl_rem);
    const int c_end = serial ? n_chunks : c_begin + sl_base + (ks < sl_rem ? 1 : 0);

    float4v run[R][MT];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int t = 0; t < MT; t++) run[r][t] = (float4v){0.f, 0.f, 0.f, 0.f};

    half8 a_stage[ANL];
    u32x4 w_stage[WNL];
    float4v cs_stage[MT], cs_cur[MT];  // the chunk's factors for this lane's rows m0 + 16t + 4g + (0..3)
    float bs_stage = 0.f;
    // K is a multiple of 256, so every chunk has CH full steps and CHUNK_BYTES bytes per row. Every load is
    // unconditional (addresses are clamped instead): a load under a branch makes the compiler wait for it
    // inside the branch, which serialises the whole prefetch.
    auto fetch = [&](int chunk) __attribute__((always_inline)) {
        const int s0 = chunk * CH;
#pragma unroll
        for (int i = 0; i < ANL; i++) {
            const int p = i * 256 + tid;              // (s, t, hl, l)
            const int l = p & 63, hl = (p >> 6) & 1, t = (p >> 7) % MT, s = p / (128 * MT);
            a_stage[i] = pv.tiles[((size_t)((s0 + s) * mtiles + mg * MT + t) * 2 + hl) * 64 + l];
        }
#pragma unroll
        for (int t = 0; t < MT; t++) cs_stage[t] = *(const float4v *)(pv.cscale + (size_t)chunk * Mpad + m0 + t * 16 + 4 * g);
        if (F::HAS_MIN) {
            const int i = tid % NBS;  // (step, tile, row); threads past NBS repeat a load and store nothing
            bs_stage = pv.bsum[(size_t)(s0 + i / (MT * 16)) * Mpad + m0 + i % (MT * 16)];
        }
        const size_t coff = (size_t)chunk * F::CHUNK_BYTES;
#pragma unroll
        for (int i = 0; i < WNL; i++) {
            const int pc = min(i * 64 + lane, WPIECES - 1);
            const int row = pc / F::ROW_PIECES, col = pc % F::ROW_PIECES;
            const int n = min(n0 + row, N - 1);
            const uint8_t *src = seg_row(segs, n, row_bytes) + coff;
            // Unaligned rows are staged from the 16-byte boundary below their first byte; the pieces then end
            // at the boundary at or above the chunk's last byte, which is inside the matrix because its size
            // is a multiple of 16 (checked on the host).
            if (!F::ALIGNED) src = (const uint8_t *)((uintptr_t)src & ~(uintptr_t)15);
            w_stage[i] = *(const u32x4 *)(src + col * 16);
        }
    };
    auto commit = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < MT; t++) cs_cur[t] = cs_stage[t];
        if (F::HAS_MIN && tid < NBS) bs_lds[tid] = bs_stage;
#pragma unroll
        for (int i = 0; i < ANL; i++) a_lds[i * 256 + tid] = a_stage[i];
#pragma unroll
        for (int i = 0; i < WNL; i++) {
            const int pc = i * 64 + lane;
            const int row = pc / F::ROW_PIECES, col = pc % F::ROW_PIECES;
            if (pc < WPIECES) *(u32x4 *)(&w_lds[wave][row * PITCH + col * 16]) = w_stage[i];
        }
    };
    // One chunk = CH steps, software-pipelined by hand. A SIMD issues a wave's instructions in order and a
    // 16x16x32 MFMA keeps the matrix pipe busy for 16 cycles, so eight MFMAs back to back stall the wave for
    // most of a step while its ~60 vector instructions (nibble unpacking, block-scale FMAs) wait their turn.
    // Each step therefore issues its MFMAs interleaved with vector work that does not depend on them: the
    // scale FMAs of the previous step and the unpacking of the next step's weights, whose LDS reads were
    // issued a step earlier. sched_group_barrier pins that interleaving.
    struct StepA { half8 h[MT], l[MT]; };
    auto lds_a = [&](int s) __attribute__((always_inline)) {
        StepA a;
#pragma unroll
        for (int t = 0; t < MT; t++) {
            a.h[t] = a_lds[((s * MT + t) * 2 + 0) * 64 + lane];
            a.l[t] = a_lds[((s * MT + t) * 2 + 1) * 64 + lane];
        }
        return a;
    };
    float4v crun[R][MT];  // the chunk's own sum, folded into run with the chunk's factors at its end
    auto scale_add = [&](const float4v (&acc)[R][MT], const StepW (&w)[R], const float4v (&bs)[MT]) __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int t = 0; t < MT; t++) {
                if (F::HAS_MIN) {
#pragma unroll
                    for (int i = 0; i < 4; i++)  // two fused multiply-adds per output (one expression would cost three operations)
                        crun[r][t][i] = __builtin_fmaf(-w[r].dm, bs[t][i], __builtin_fmaf(w[r].d, acc[r][t][i], crun[r][t][i]));
                } else {
#pragma unroll
                    for (int i = 0; i < 4; i++) crun[r][t][i] += w[r].d * acc[r][t][i];
                }
            }
    };
    auto compute = [&](int chunk) __attribute__((always_inline)) {
        const uint8_t *wl = &w_lds[wave][0];
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int t = 0; t < MT; t++) crun[r][t] = (float4v){0.f, 0.f, 0.f, 0.f};
        StepA a_cur = lds_a(0), a_nxt = a_cur;
        typename F::Raw raw_n[R], raw_nn[R];
        StepW w_cur[R], w_nxt[R], w_old[R];
        float4v acc_old[R][MT], bs_old[MT] = {}, bs_cur[MT] = {};
        int roff[R];  // where this lane's row of tile r starts in the wave's staging area
#pragma unroll
        for (int r = 0; r < R; r++) {
            roff[r] = (r * 16 + ln) * PITCH;
            if (!F::ALIGNED) {
                const int n = min(n0 + r * 16 + ln, N - 1);
                roff[r] += (int)((uintptr_t)(seg_row(segs, n, row_bytes) + (size_t)chunk * F::CHUNK_BYTES) & 15);
            }
            raw_n[r] = F::read(wl, roff[r], 0, g);
            w_old[r] = w_nxt[r] = w_cur[r] = F::unpack(raw_n[r], 0);
            raw_nn[r] = raw_n[r] = F::read(wl, roff[r], 1, g);
#pragma unroll
            for (int t = 0; t < MT; t++) acc_old[r][t] = (float4v){0.f, 0.f, 0.f, 0.f};
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < CH; s++) {
            // LDS reads for later steps go out first
            if (s + 1 < CH) a_nxt = lds_a(s + 1);
            if (s + 2 < CH) {
#pragma unroll
                for (int r = 0; r < R; r++) raw_nn[r] = F::read(wl, roff[r], s + 2, g);
            }
            if (F::HAS_MIN) {
#pragma unroll
                for (int t = 0; t < MT; t++) bs_cur[t] = *(const float4v *)&bs_lds[(s * MT + t) * 16 + 4 * g];
            }
            float4v acc[R][MT];
#pragma unroll
            for (int r = 0; r < R; r++)
#pragma unroll
                for (int t = 0; t < MT; t++)
                    acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_cur.h[t], w_cur[r].b, (float4v){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < R; r++)
#pragma unroll
                for (int t = 0; t < MT; t++)
                    acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_cur.l[t], w_cur[r].b, acc[r][t], 0, 0, 0);
            // vector work independent of this step's MFMAs
            if (s > 0) scale_add(acc_old, w_old, bs_old);
            if (s + 1 < CH) {
#pragma unroll
                for (int r = 0; r < R; r++) w_nxt[r] = F::unpack(raw_n[r], s + 1);
            }
            // one MFMA, then a share of the vector instructions
#pragma unroll
            for (int i = 0; i < 2 * R * MT; i++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int r = 0; r < R; r++) {
                w_old[r] = w_cur[r];
                w_cur[r] = w_nxt[r];
                raw_n[r] = raw_nn[r];
#pragma unroll
                for (int t = 0; t < MT; t++) acc_old[r][t] = acc[r][t];
            }
#pragma unroll
            for (int t = 0; t < MT; t++) bs_old[t] = bs_cur[t];
            a_cur = a_nxt;
        }
        scale_add(acc_old, w_old, bs_old);
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int t = 0; t < MT; t++)
#pragma unroll
                for (int i = 0; i < 4; i++) run[r][t][i] += cs_cur[t][i] * crun[r][t][i];
    };

    // The same for formats whose step has two scales: four 16x16x16 MFMAs per tile and step, scaled as
    // soon as the next tile's MFMAs have been issued, so that only two tiles' results are live at a time
    // (the staging of unaligned rows and the wider raw reads leave fewer registers for pipelining).
    auto compute_two_scales = [&](int chunk) __attribute__((always_inline)) {
        const uint8_t *wl = &w_lds[wave][0];
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int t = 0; t < MT; t++) crun[r][t] = (float4v){0.f, 0.f, 0.f, 0.f};
        int roff[R];
        typename F::Raw raw_n[R];
        StepW w_cur[R], w_nxt[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int n = min(n0 + r * 16 + ln, N - 1);
            roff[r] = (r * 16 + ln) * PITCH +
                      (int)((uintptr_t)(seg_row(segs, n, row_bytes) + (size_t)chunk * F::CHUNK_BYTES) & 15);
            raw_n[r] = F::read(wl, roff[r], 0, g);
            w_nxt[r] = w_cur[r] = F::unpack(raw_n[r], 0);
            raw_n[r] = F::read(wl, roff[r], 1, g);
        }
        StepA a_cur = lds_a(0), a_nxt = a_cur;
        const float4v z = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < CH; s++) {
            if (s + 1 < CH) {
                a_nxt = lds_a(s + 1);
#pragma unroll
                for (int r = 0; r < R; r++) w_nxt[r] = F::unpack(raw_n[r], s + 1);
            }
            if (s + 2 < CH) {
#pragma unroll
                for (int r = 0; r < R; r++) raw_n[r] = F::read(wl, roff[r], s + 2, g);
            }
            float4v p1 = z, p2 = z;  // the previous tile's two sums
            int pr = 0, pt = 0;
#pragma unroll
            for (int i = 0; i <= R * MT; i++) {
                float4v c1 = z, c2 = z;
                const int r = i / MT, t = i % MT;
                if (i < R * MT) {
                    // slots 0,1,4,5 of an operand are the step's first 16 elements, slots 2,3,6,7 its second 16
                    c1 = __builtin_amdgcn_mfma_f32_16x16x16f16(first16(a_cur.h[t]), first16(w_cur[r].b), z, 0, 0, 0);
                    c2 = __builtin_amdgcn_mfma_f32_16x16x16f16(second16(a_cur.h[t]), second16(w_cur[r].b), z, 0, 0, 0);
                    c1 = __builtin_amdgcn_mfma_f32_16x16x16f16(first16(a_cur.l[t]), first16(w_cur[r].b), c1, 0, 0, 0);
                    c2 = __builtin_amdgcn_mfma_f32_16x16x16f16(second16(a_cur.l[t]), second16(w_cur[r].b), c2, 0, 0, 0);
                }
                if (i > 0) {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        crun[pr][pt][e] = __builtin_fmaf(w_cur[pr].dm, p2[e], __builtin_fmaf(w_cur[pr].d, p1[e], crun[pr][pt][e]));
                }
                p1 = c1, p2 = c2, pr = r, pt = t;
            }
#pragma unroll
            for (int r = 0; r < R; r++) w_cur[r] = w_nxt[r];
            a_cur = a_nxt;
        }
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int t = 0; t < MT; t++)
#pragma unroll
                for (int i = 0; i < 4; i++) run[r][t][i] += cs_cur[t][i] * crun[r][t][i];
    };

    float4v total[SERIAL ? R : 1][SERIAL ? MT : 1];  // serial mode: the finished slices' sum (touched at slice ends only)
    int slice = 0, slice_end = sl_base + (0 < sl_rem ? 1 : 0);
    if (c_begin < c_end) fetch(c_begin);
    for (int chunk = c_begin; chunk < c_end; chunk++) {
        if constexpr (SERIAL) if (chunk == slice_end) {  // a slice is complete: fold it in, start the next from zero
#pragma unroll
            for (int r = 0; r < R; r++)
#pragma unroll
                for (int t = 0; t < MT; t++) {
#pragma unroll
                    for (int i = 0; i < 4; i++) total[r][t][i] = slice == 0 ? run[r][t][i] : total[r][t][i] + run[r][t][i];
                    run[r][t] = (float4v){0.f, 0.f, 0.f, 0.f};
                }
            slice++;
            slice_end += sl_base + (slice < sl_rem ? 1 : 0);
        }
        __syncthreads();  // previous chunk's reads are done
        commit();
        __syncthreads();
        if (chunk + 1 < c_end) fetch(chunk + 1);  // in flight while this chunk is computed
        if constexpr (F::TWO_SCALES)
            compute_two_scales(chunk);
        else
            compute(chunk);
    }
    if constexpr (SERIAL) if (slice > 0) {
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int t = 0; t < MT; t++)
#pragma unroll
                for (int i = 0; i < 4; i++) run[r][t][i] = total[r][t][i] + run[r][t][i];
    }

    // lane (g, ln) of tile (r, t) holds C[m = m0 + 16t + 4g + i][n = n0 + 16r + ln], i = 0..3. Each wave
    // transposes its [16*MT x ROWS_W] block through LDS (the activation buffer is free now) so that global
    // memory sees 16-byte accesses covering whole 128-byte row segments.
    constexpr int TP = ROWS_W + 4;  // floats per transposed row: rows 4 apart land 16 banks apart
    static_assert(4 * 16 * MT * TP * 4 <= (int)sizeof(a_lds), "transpose area must fit the activation buffer");
    __syncthreads();  // every wave is done reading a_lds
    float *T = (float *)a_lds + wave * (16 * MT * TP);
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int t = 0; t < MT; t++)
#pragma unroll
            for (int i = 0; i < 4; i++) T[(t * 16 + 4 * g + i) * TP + r * 16 + ln] = run[r][t][i];
    __syncthreads();
    constexpr int LPR = ROWS_W / 4;   // lanes per row of the block
    constexpr int RPI = 64 / LPR;     // rows per access
    const bool vec = (flags & 1) != 0;  // N % 4 == 0 and 16-byte aligned bases
    const int nl = (lane % LPR) * 4, n = n0 + nl;
#pragma unroll
    for (int j = 0; j < 16 * MT / RPI; j++) {
        const int ml = j * RPI + lane / LPR, m = m0 + ml;
        const float4 c = *(const float4 *)(T + ml * TP + nl);
        float v[4] = {c.x, c.y, c.z, c.w};
        if (m >= M || n >= N) continue;
        if (partial) {
            float *dst = partial + ((size_t)ks * M + m) * N + n;
            if (vec) {
                *(float4 *)dst = c;
            } else {
                for (int e = 0; e < 4; e++)
                    if (n + e < N) dst[e] = v[e];
            }
            continue;
        }
        const float inv = pv.inv_scale[m];
        float *dst = out + (size_t)m * N + n;
        const float *rs = residual ? residual + (size_t)m * N + n : nullptr;
        if (vec) {
            float4 o;
            o.x = __fmul_rn(v[0], inv); o.y = __fmul_rn(v[1], inv); o.z = __fmul_rn(v[2], inv); o.w = __fmul_rn(v[3], inv);
            if (rs) {
                const float4 q = *(const float4 *)rs;
                o.x = __fadd_rn(q.x, o.x); o.y = __fadd_rn(q.y, o.y); o.z = __fadd_rn(q.z, o.z); o.w = __fadd_rn(q.w, o.w);
            }
            *(float4 *)dst = o;
        } else {
            for (int e = 0; e < 4; e++)
                if (n + e < N) {
                    float o = __fmul_rn(v[e], inv);
                    if (rs) o = __fadd_rn(rs[e], o);
                    dst[e] = o;
                }
        }
    }
}

// out[m][n] = residual + inv_scale[m] * (P[0] + P[1] + ... + P[KS-1]) in that order.
__global__ void __launch_bounds__(256) qgemm_reduce_kernel(const float *__restrict__ partial,
                                                           const float *__restrict__ inv_scale,
                                                           float *__restrict__ out, const float *__restrict__ residual,
                                                           int M, int N, int KS) {
    const size_t total = (size_t)M * N;
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    float v = partial[i];
    for (int s = 1; s < KS; s++) v += partial[(size_t)s * total + i];
    v = __fmul_rn(v, inv_scale[i / N]);
    if (residual) v = __fadd_rn(residual[i], v);
    out[i] = v;
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
    if (fmt == VX_Q5_0) {  // pkg/gguf/dequant.go:100-145
        const uint8_t *b = row + (size_t)(k >> 5) * 22;
        const int i = k & 31;
        const uint32_t qh = (uint32_t)b[2] | ((uint32_t)b[3] << 8) | ((uint32_t)b[4] << 16) | ((uint32_t)b[5] << 24);
        const uint8_t bv = b[6 + (i & 15)];
        const int q = (int)((i < 16) ? (bv & 0xF) : (bv >> 4)) | (int)(((qh >> i) & 1) << 4);
        return __fmul_rn((float)(q - 16), h2f((uint16_t)(b[0] | (b[1] << 8))));
    }
    if (fmt == VX_Q5_K) {  // pkg/gguf/dequant.go:423-500
        const uint8_t *b = row + (size_t)(k >> 8) * 176;
        const int e = k & 255, grp = e >> 6, l = e & 31, hi = (e >> 5) & 1, j = grp * 2 + hi;
        const uint8_t *q = b + 4;
        uint32_t sc, mn;
        if (j < 4) {
            sc = q[j] & 63;
            mn = q[j + 4] & 63;
        } else {
            sc = (q[j + 4] & 0x0F) | ((q[j - 4] >> 6) << 4);
            mn = (q[j + 4] >> 4) | ((q[j] >> 6) << 4);
        }
        const float d1 = __fmul_rn(h2f((uint16_t)(b[0] | (b[1] << 8))), (float)sc);
        const float dm1 = __fmul_rn(h2f((uint16_t)(b[2] | (b[3] << 8))), (float)mn);
        const uint8_t bv = b[48 + grp * 32 + l];
        const int qq = (int)(hi ? (bv >> 4) : (bv & 0xF)) + (int)(((b[16 + l] >> j) & 1) << 4);
        return __fsub_rn(__fmul_rn(d1, (float)qq), dm1);
    }
    if (fmt == VX_BF16) {  // pkg/gguf/dequant.go:215-228
        const uint32_t u = ((uint32_t)row[2 * (size_t)k] | ((uint32_t)row[2 * (size_t)k + 1] << 8)) << 16;
        return __uint_as_float(u);
    }
    // Q6_K, pkg/gguf/dequant.go:272-331
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

// Formats without a tiled path (Q5_0, Q5_K, BF16): one wave per weight row, lane l takes elements 4l..4l+3 of every
// 256-element stretch (coalesced float4 activation loads, the row's bytes shared through the cache), exact
// dequantised values, float32 FMAs, a butterfly sum. grid = (N, ceil(M/FB_M)); block = 64.
template <int FMT>
__device__ __forceinline__ void deq4(const uint8_t *row, int k0, float (&w)[4]) {
    if (FMT == VX_BF16) {
        const uint16_t *p = (const uint16_t *)(row + 2 * (size_t)k0);
#pragma unroll
        for (int i = 0; i < 4; i++) w[i] = __uint_as_float((uint32_t)p[i] << 16);
    } else if (FMT == VX_Q5_0) {
        const uint8_t *b = row + (size_t)(k0 >> 5) * 22;
        const uint16_t *h = (const uint16_t *)b;  // blocks start on even addresses
        const int i0 = k0 & 31, j0 = i0 & 15;
        const float d = h2f(h[0]);
        const uint32_t qh = ((uint32_t)h[1] | ((uint32_t)h[2] << 16)) >> i0;
        const uint32_t qs = ((uint32_t)h[3 + (j0 >> 1)] | ((uint32_t)h[4 + (j0 >> 1)] << 16)) >> (i0 & 16 ? 4 : 0);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int q = (int)((qs >> (8 * i)) & 0xF) | (int)(((qh >> i) & 1) << 4);
            w[i] = __fmul_rn((float)(q - 16), d);
        }
    } else {  // Q5_K
        const uint8_t *b = row + (size_t)(k0 >> 8) * 176;
        const int e = k0 & 255, grp = e >> 6, l = e & 31, hi = (e >> 5) & 1, j = grp * 2 + hi;
        const uint8_t *q = b + 4;
        uint32_t sc, mn;
        if (j < 4) {
            sc = q[j] & 63;
            mn = q[j + 4] & 63;
        } else {
            sc = (q[j + 4] & 0x0F) | ((q[j - 4] >> 6) << 4);
            mn = (q[j + 4] >> 4) | ((q[j] >> 6) << 4);
        }
        const uint16_t *h = (const uint16_t *)b;
        const float d1 = __fmul_rn(h2f(h[0]), (float)sc), dm1 = __fmul_rn(h2f(h[1]), (float)mn);
        const uint16_t *qs16 = (const uint16_t *)(b + 48 + grp * 32 + l), *qh16 = (const uint16_t *)(b + 16 + l);
        const uint32_t qs = ((uint32_t)qs16[0] | ((uint32_t)qs16[1] << 16)) >> (hi ? 4 : 0);
        const uint32_t qh = ((uint32_t)qh16[0] | ((uint32_t)qh16[1] << 16)) >> j;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int qq = (int)((qs >> (8 * i)) & 0xF) + (int)(((qh >> (8 * i)) & 1) << 4);
            w[i] = __fsub_rn(__fmul_rn(d1, (float)qq), dm1);
        }
    }
}

template <int FMT>
__global__ void __launch_bounds__(64) qrow4_kernel(const uint8_t *__restrict__ W, const float *__restrict__ a,
                                                   float *__restrict__ out, const float *__restrict__ residual, int M, int N,
                                                   int K, size_t row_bytes) {
    const int n = blockIdx.x, m0 = blockIdx.y * FB_M, lane = threadIdx.x;
    const uint8_t *row = W + (size_t)n * row_bytes;
    float acc[FB_M];
#pragma unroll
    for (int i = 0; i < FB_M; i++) acc[i] = 0.f;
    for (int k0 = lane * 4; k0 < K; k0 += 256) {
        float w[4];
        deq4<FMT>(row, k0, w);
#pragma unroll
        for (int i = 0; i < FB_M; i++) {
            const int m = min(m0 + i, M - 1);  // rows past M repeat the last one; their sums are dropped
            const float4 x = *(const float4 *)(a + (size_t)m * K + k0);
            acc[i] = fmaf(x.w, w[3], fmaf(x.z, w[2], fmaf(x.y, w[1], fmaf(x.x, w[0], acc[i]))));
        }
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

// ---------------------------------------------------------------- consumers of split-K partial sums
// Sum of the KS slices of four consecutive columns, in slice order, times the activation row scale:
// exactly what qgemm_reduce_kernel computes.
__device__ __forceinline__ float4 psum4(const float *__restrict__ P, int KS, size_t slice_elems, size_t idx, float inv) {
    float4 v = *(const float4 *)(P + idx);
    for (int s = 1; s < KS; s++) {
        const float4 t = *(const float4 *)(P + (size_t)s * slice_elems + idx);
        v.x += t.x; v.y += t.y; v.z += t.z; v.w += t.w;
    }
    v.x = __fmul_rn(v.x, inv); v.y = __fmul_rn(v.y, inv); v.z = __fmul_rn(v.z, inv); v.w = __fmul_rn(v.w, inv);
    return v;
}

enum { FUSE_ADD_RMSNORM = 0, FUSE_SILU_MUL = 1 };
constexpr int FP_THREADS = PREP_THREADS;

// grid = Mpad rows, block = FP_THREADS, dynamic LDS = K floats.
//  FUSE_ADD_RMSNORM: v = x + inv_in * sum_ks P[ks][r][:K]  (the residual add of runtime/block.go:990,1077),
//                    x <- v, prepared <- (v / rms) * w      (backend/cpu/cpu.go:200-220)
//  FUSE_SILU_MUL:    g = inv_in * sum P[..][r][:K], u = inv_in * sum P[..][r][K:2K],
//                    prepared <- (g*sigmoid(g)) * u          (backend/cpu/cpu.go:390-400)
// inv_in is the row scale of the activation that produced P; it is read before this row's new
// scale overwrites it. Values are bit-identical to reduce + RMSNorm/SiLUMul + prepare run separately.
template <int MODE>
__global__ void __launch_bounds__(FP_THREADS) fused_prepare_kernel(float *__restrict__ x, const float *__restrict__ P,
                                                                   int KS, int M, int K, const float *__restrict__ w,
                                                                   float eps, PrepView pv, int Mpad,
                                                                   const float *__restrict__ inv_in_rows) {
    extern __shared__ __attribute__((aligned(16))) float ybuf[];
    __shared__ float sm[2 * (FP_THREADS / 64)];
    const int r = blockIdx.x, tid = threadIdx.x;
    const int mtiles = Mpad / 16, mt = r >> 4, ln = r & 15;
    const int npairs = K / 8;
    if (r >= M) {
        const half8 z = {0, 0, 0, 0, 0, 0, 0, 0};
        for (int p = tid; p < npairs; p += FP_THREADS) {
            const int ks = p >> 2, g = p & 3;
            half8 *t = pv.tiles + ((size_t)(ks * mtiles + mt) * 2) * 64 + g * 16 + ln;
            t[0] = z;
            t[64] = z;
            if (g == 0) pv.bsum[(size_t)ks * Mpad + r] = 0.f;
        }
        if (tid == 0) pv.inv_scale[r] = 0.f;
        for (int c = tid; c < K / 256; c += blockDim.x) pv.cscale[(size_t)c * Mpad + r] = 0.f;
        return;
    }
    const float inv_in = inv_in_rows[r];
    const int ncols = (MODE == FUSE_SILU_MUL) ? 2 * K : K;
    const size_t slice_elems = (size_t)M * ncols;
    float amax = 0.f, ss = 0.f;
    for (int k = tid * 4; k < K; k += FP_THREADS * 4) {
        float y[4];
        if (MODE == FUSE_ADD_RMSNORM) {
            const float4 d = psum4(P, KS, slice_elems, (size_t)r * ncols + k, inv_in);
            const float4 xo = *(const float4 *)(x + (size_t)r * K + k);
            y[0] = __fadd_rn(xo.x, d.x); y[1] = __fadd_rn(xo.y, d.y); y[2] = __fadd_rn(xo.z, d.z); y[3] = __fadd_rn(xo.w, d.w);
            *(float4 *)(x + (size_t)r * K + k) = make_float4(y[0], y[1], y[2], y[3]);
            *(float4 *)(ybuf + k) = make_float4(y[0], y[1], y[2], y[3]);
            ss = sumsq4(ss, y[0], y[1], y[2], y[3]);
            const float4 wv = *(const float4 *)(w + k);
            y[0] *= wv.x; y[1] *= wv.y; y[2] *= wv.z; y[3] *= wv.w;
        } else {
            // two column groups per trip, their loads issued together: the trip count is what this
            // latency-bound loop pays for (the second group is clamped and dropped past the row's end)
            const int k2 = k + FP_THREADS * 4;
            const bool has2 = k2 < K;
            const int kb = has2 ? k2 : k;
            const float4 gt = psum4(P, KS, slice_elems, (size_t)r * ncols + k, inv_in);
            const float4 up = psum4(P, KS, slice_elems, (size_t)r * ncols + K + k, inv_in);
            const float4 gt2 = psum4(P, KS, slice_elems, (size_t)r * ncols + kb, inv_in);
            const float4 up2 = psum4(P, KS, slice_elems, (size_t)r * ncols + K + kb, inv_in);
            y[0] = __fmul_rn(__fmul_rn(gt.x, sigmoid_ref(gt.x)), up.x);
            y[1] = __fmul_rn(__fmul_rn(gt.y, sigmoid_ref(gt.y)), up.y);
            y[2] = __fmul_rn(__fmul_rn(gt.z, sigmoid_ref(gt.z)), up.z);
            y[3] = __fmul_rn(__fmul_rn(gt.w, sigmoid_ref(gt.w)), up.w);
            *(float4 *)(ybuf + k) = make_float4(y[0], y[1], y[2], y[3]);
            if (has2) {
                float z[4];
                z[0] = __fmul_rn(__fmul_rn(gt2.x, sigmoid_ref(gt2.x)), up2.x);
                z[1] = __fmul_rn(__fmul_rn(gt2.y, sigmoid_ref(gt2.y)), up2.y);
                z[2] = __fmul_rn(__fmul_rn(gt2.z, sigmoid_ref(gt2.z)), up2.z);
                z[3] = __fmul_rn(__fmul_rn(gt2.w, sigmoid_ref(gt2.w)), up2.w);
                *(float4 *)(ybuf + k2) = make_float4(z[0], z[1], z[2], z[3]);
                amax = fmaxf(amax, fmaxf(fmaxf(fabsf(z[0]), fabsf(z[1])), fmaxf(fabsf(z[2]), fabsf(z[3]))));
            }
            k += FP_THREADS * 4;  // the second group is done
        }
        amax = fmaxf(amax, fmaxf(fmaxf(fabsf(y[0]), fabsf(y[1])), fmaxf(fabsf(y[2]), fabsf(y[3]))));
    }
    row_stats(amax, ss, sm);  // also orders the ybuf writes before pass 2
    float rms = 1.f;
    if (MODE == FUSE_ADD_RMSNORM) {
        rms = (float)sqrt((double)(ss / (float)K + eps));
        amax = amax / rms * 1.0001f;
    }
    float s = 1.f, inv = 1.f;
    if (amax > 0.f && amax < INFINITY) {
        int ex;
        (void)frexpf(amax, &ex);
        s = ldexpf(1.f, 13 - ex);
        inv = ldexpf(1.f, ex - 13);
    }
    if (tid == 0) pv.inv_scale[r] = inv;
    for (int c = tid; c < K / 256; c += blockDim.x) pv.cscale[(size_t)c * Mpad + r] = 1.f;
    for (int p = tid; p < npairs; p += FP_THREADS) {
        const int ks = p >> 2, g = p & 3;
        const int k0 = ks * 32 + 4 * g;
        const float4 xa = *(const float4 *)(ybuf + k0), xb = *(const float4 *)(ybuf + k0 + 16);
        float ya[4] = {xa.x, xa.y, xa.z, xa.w}, yb[4] = {xb.x, xb.y, xb.z, xb.w};
        if (MODE == FUSE_ADD_RMSNORM) {
            const float4 wa = *(const float4 *)(w + k0), wb = *(const float4 *)(w + k0 + 16);
            const float wv[8] = {wa.x, wa.y, wa.z, wa.w, wb.x, wb.y, wb.z, wb.w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                ya[i] = __fmul_rn(ya[i] / rms, wv[i]);
                yb[i] = __fmul_rn(yb[i] / rms, wv[4 + i]);
            }
        }
        const float v[8] = {ya[0] * s, ya[2] * s, yb[0] * s, yb[2] * s, ya[1] * s, ya[3] * s, yb[1] * s, yb[3] * s};
        half8 h, l;
        float bs = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            h[i] = (_Float16)v[i];
            l[i] = (_Float16)(v[i] - (float)h[i]);
            bs += v[i];
        }
        half8 *t = pv.tiles + ((size_t)(ks * mtiles + mt) * 2) * 64 + g * 16 + ln;
        t[0] = h;
        t[64] = l;
        bs += __shfl_xor(bs, 1, 64);
        bs += __shfl_xor(bs, 2, 64);
        if (g == 0) pv.bsum[(size_t)ks * Mpad + r] = bs;
    }
}

// Merges the split-KV attention partials (m, l, acc[D]) of row r (one sequence) exactly as the stand-alone merge
// kernel does (out = sum_s acc_s*2^(m_s-M) / sum_s l_s*2^(m_s-M)) and prepares the [Hq*D] result as the Wo
// projection's activation. grid = Mpad rows, block = PREP_THREADS, dynamic LDS = K floats.
__global__ void __launch_bounds__(PREP_THREADS) merge_prepare_kernel(const float *__restrict__ part,
                                                                     const int32_t *__restrict__ kv_lens, int M, int K,
                                                                     int D, int max_splits, int tokens_per_split,
                                                                     PrepView pv, int Mpad) {
    extern __shared__ __attribute__((aligned(16))) float ybuf[];
    __shared__ float sm[2 * (PREP_THREADS / 64)];
    const int r = blockIdx.x, tid = threadIdx.x;
    const int mtiles = Mpad / 16, mt = r >> 4, ln = r & 15;
    const int npairs = K / 8;
    if (r >= M) {
        const half8 z = {0, 0, 0, 0, 0, 0, 0, 0};
        for (int p = tid; p < npairs; p += PREP_THREADS) {
            const int ks = p >> 2, g = p & 3;
            half8 *t = pv.tiles + ((size_t)(ks * mtiles + mt) * 2) * 64 + g * 16 + ln;
            t[0] = z;
            t[64] = z;
            if (g == 0) pv.bsum[(size_t)ks * Mpad + r] = 0.f;
        }
        if (tid == 0) pv.inv_scale[r] = 0.f;
        for (int c = tid; c < K / 256; c += blockDim.x) pv.cscale[(size_t)c * Mpad + r] = 0.f;
        return;
    }
    const int ns = min((kv_lens[r] + tokens_per_split - 1) / tokens_per_split, max_splits);
    const int P = D + 2;
    float amax = 0.f, ss = 0.f;
    for (int k = tid * 4; k < K; k += PREP_THREADS * 4) {
        const int h = k / D, d = k % D;
        const float *pb = part + ((size_t)r * (K / D) + h) * max_splits * P;
        float Mx = -INFINITY;
        for (int s = 0; s < ns; s++) Mx = fmaxf(Mx, pb[(size_t)s * P]);
        float L = 0.f, A[4] = {0.f, 0.f, 0.f, 0.f};
        for (int s = 0; s < ns; s++) {
            const float *ps = pb + (size_t)s * P;
            const float f = exp2f(ps[0] - Mx);
            L += ps[1] * f;
            const float2 a = *(const float2 *)(ps + 2 + d), b = *(const float2 *)(ps + 4 + d);
            A[0] += a.x * f; A[1] += a.y * f; A[2] += b.x * f; A[3] += b.y * f;
        }
        float y[4];
#pragma unroll
        for (int e = 0; e < 4; e++) y[e] = (L > 0.f) ? A[e] / L : 0.f;
        *(float4 *)(ybuf + k) = make_float4(y[0], y[1], y[2], y[3]);
        amax = fmaxf(amax, fmaxf(fmaxf(fabsf(y[0]), fabsf(y[1])), fmaxf(fabsf(y[2]), fabsf(y[3]))));
    }
    row_stats(amax, ss, sm);  // also orders the ybuf writes before pass 2
    float s = 1.f, inv = 1.f;
    if (amax > 0.f && amax < INFINITY) {
        int ex;
        (void)frexpf(amax, &ex);
        s = ldexpf(1.f, 13 - ex);
        inv = ldexpf(1.f, ex - 13);
    }
    if (tid == 0) pv.inv_scale[r] = inv;
    for (int c = tid; c < K / 256; c += blockDim.x) pv.cscale[(size_t)c * Mpad + r] = 1.f;
    for (int p = tid; p < npairs; p += PREP_THREADS) {
        const int ks = p >> 2, g = p & 3;
        const int k0 = ks * 32 + 4 * g;
        const float4 xa = *(const float4 *)(ybuf + k0), xb = *(const float4 *)(ybuf + k0 + 16);
        const float v[8] = {xa.x * s, xa.z * s, xb.x * s, xb.z * s, xa.y * s, xa.w * s, xb.y * s, xb.w * s};
        half8 h, l;
        float bs = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            h[i] = (_Float16)v[i];
            l[i] = (_Float16)(v[i] - (float)h[i]);
            bs += v[i];
        }
        half8 *t = pv.tiles + ((size_t)(ks * mtiles + mt) * 2) * 64 + g * 16 + ln;
        t[0] = h;
        t[64] = l;
        bs += __shfl_xor(bs, 1, 64);
        bs += __shfl_xor(bs, 2, 64);
        if (g == 0) pv.bsum[(size_t)ks * Mpad + r] = bs;
    }
}

// ---------------------------------------------------------------- chunk-parallel prepares (decode batches)
// One wave per (256-column chunk, row): lane l owns columns 4l..4l+3 of the chunk. Nothing spans the row except
// RMSNorm's sum of squares, which goes through per-chunk partial sums and an arrival counter: the last wave of
// a row to arrive adds the partials in chunk order (so the result does not depend on who arrives last) and
// writes the row factor 1/rms; nobody waits for anybody. The prepared values are x*w (not yet divided by rms)
// scaled per chunk; the GEMM multiplies each chunk's dot product by cscale and the row's result by inv_scale.
// Writes inv_scale[r] *= 1/rms for every row, for consumers that read plain row factors. grid = rows, block = 64.
__global__ void __launch_bounds__(64) finalize_row_norm_kernel(float *__restrict__ inv_rows, RowNorm rn) {
    const float f = row_factor(inv_rows, rn, blockIdx.x);
    if (threadIdx.x == 0) inv_rows[blockIdx.x] = f;
}

#include "qgemm_wave.h"

// grid = (K/256, Mpad), block = 64.
//   x_new = x + inv_in[r] * sum_s P[s][r][:]   (P may be NULL: x_new = x), x <- x_new when P is given,
//   prepared <- x_new * w, its chunks' sums of squares to ss_out for the pending 1/rms (backend/cpu/cpu.go:200-220)
__global__ void __launch_bounds__(64) chunk_add_norm_kernel(float *__restrict__ x, const float *__restrict__ P, int KS, int M,
                                                            int K, const float *__restrict__ w, float eps, PrepView pv,
                                                            int Mpad, const float *__restrict__ inv_in_rows, RowNorm rn_in,
                                                            float *__restrict__ ss_out) {
    const int c = blockIdx.x, r = blockIdx.y, lane = threadIdx.x;
    const int k = c * 256 + lane * 4;
    float y[4] = {0.f, 0.f, 0.f, 0.f};
    float ss = 0.f;
    if (r < M) {
        float4 v = *(const float4 *)(x + (size_t)r * K + k);
        if (P) {
            const float4 d = psum4(P, KS, (size_t)M * K, (size_t)r * K + k, row_factor(inv_in_rows, rn_in, r));
            v.x = __fadd_rn(v.x, d.x); v.y = __fadd_rn(v.y, d.y); v.z = __fadd_rn(v.z, d.z); v.w = __fadd_rn(v.w, d.w);
            *(float4 *)(x + (size_t)r * K + k) = v;
        }
        ss = wave_sum(sumsq4(0.f, v.x, v.y, v.z, v.w));
        const float4 wv = *(const float4 *)(w + k);
        y[0] = v.x * wv.x; y[1] = v.y * wv.y; y[2] = v.z * wv.z; y[3] = v.w * wv.w;
    }
    write_chunk(pv, r, c, y, Mpad);
    if (lane == 0) {
        ss_out[c * VX_PREP_SYNC_ROWS + r] = ss;
        if (c == 0) pv.inv_scale[r] = r < M ? 1.f : 0.f;
    }
}

//   g = inv_in[r] * sum_s P[s][r][:K], u = inv_in[r] * sum_s P[s][r][K:2K], prepared <- (g*sigmoid(g)) * u, row factor 1
__global__ void __launch_bounds__(64) chunk_silu_kernel(const float *__restrict__ P, int KS, int M, int K, PrepView pv, int Mpad,
                                                        const float *__restrict__ inv_in_rows, RowNorm rn_in) {
    const int c = blockIdx.x, r = blockIdx.y, lane = threadIdx.x;
    const int k = c * 256 + lane * 4;
    float y[4] = {0.f, 0.f, 0.f, 0.f};
    if (r < M) {
        const float inv_in = row_factor(inv_in_rows, rn_in, r);
        const size_t slice = (size_t)M * 2 * K;
        const float4 gt = psum4(P, KS, slice, (size_t)r * 2 * K + k, inv_in);
        const float4 up = psum4(P, KS, slice, (size_t)r * 2 * K + K + k, inv_in);
        y[0] = __fmul_rn(__fmul_rn(gt.x, sigmoid_ref(gt.x)), up.x);
        y[1] = __fmul_rn(__fmul_rn(gt.y, sigmoid_ref(gt.y)), up.y);
        y[2] = __fmul_rn(__fmul_rn(gt.z, sigmoid_ref(gt.z)), up.z);
        y[3] = __fmul_rn(__fmul_rn(gt.w, sigmoid_ref(gt.w)), up.w);
    }
    write_chunk(pv, r, c, y, Mpad);
    if (c == 0 && lane == 0) pv.inv_scale[r] = r < M ? 1.f : 0.f;
}

//   merged split-KV attention output of row r (as paged_merge_kernel computes it), row factor 1
__global__ void __launch_bounds__(64) chunk_merge_kernel(const float *__restrict__ part, const int32_t *__restrict__ kv_lens,
                                                         int M, int K, int D, int max_splits, int tokens_per_split,
                                                         PrepView pv, int Mpad) {
    const int c = blockIdx.x, r = blockIdx.y, lane = threadIdx.x;
    const int k = c * 256 + lane * 4;
    float y[4] = {0.f, 0.f, 0.f, 0.f};
    if (r < M) {
        const int ns = min((kv_lens[r] + tokens_per_split - 1) / tokens_per_split, max_splits);
        split_merge4(part, ns, K / D, D, max_splits, r, k, y);
    }
    write_chunk(pv, r, c, y, Mpad);
    if (c == 0 && lane == 0) pv.inv_scale[r] = r < M ? 1.f : 0.f;
}

//   a plain activation row by row and chunk by chunk, row factor 1 (big prompt chunks: see vx_prepare_act)
__global__ void __launch_bounds__(64) chunk_plain_kernel(const float *__restrict__ a, int M, int K, PrepView pv, int Mpad) {
    const int c = blockIdx.x, r = blockIdx.y, lane = threadIdx.x;
    float y[4] = {0.f, 0.f, 0.f, 0.f};
    if (r < M) {
        const float4 v = *(const float4 *)(a + (size_t)r * K + c * 256 + lane * 4);
        y[0] = v.x; y[1] = v.y; y[2] = v.z; y[3] = v.w;
    }
    write_chunk(pv, r, c, y, Mpad);
    if (c == 0 && lane == 0) pv.inv_scale[r] = r < M ? 1.f : 0.f;
}

// x <- x + inv_in * sum_ks P (residual add only; used after the last layer's down projection)
__global__ void __launch_bounds__(256) add_partials_kernel(float *__restrict__ x, const float *__restrict__ P, int KS,
                                                           int M, int K, const float *__restrict__ inv_scale) {
    const size_t i4 = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i4 >= (size_t)M * K) return;
    const float4 d = psum4(P, KS, (size_t)M * K, i4, inv_scale[i4 / K]);
    float4 v = *(const float4 *)(x + i4);
    v.x = __fadd_rn(v.x, d.x); v.y = __fadd_rn(v.y, d.y); v.z = __fadd_rn(v.z, d.z); v.w = __fadd_rn(v.w, d.w);
    *(float4 *)(x + i4) = v;
}

// RoPE (backend/cpu/cpu.go:226-303, interleaved pairs, one position per row) + paged K/V scatter
// (metal_bridge_darwin.m:8607-8642) reading the fused Q|K|V projection from its split-K partials.
// grid = (rows, head groups); thread = (pair j, head lane).
// GEN: the general form (biases added to the projections before the rotation as matMulTransposedWithBias +
// applyRoPE do, block.go:497-503,555-560; rope_dim of the head's dimensions rotated, in split pairs when neox).
// Where the V projection's partial sums are when V was a launch of its own (a weight format other than Q's and K's):
// [KS][M][ncols], the head vectors from column 0. P == NULL: behind Q and K in the common buffer.
struct VSrc {
    const float *P;
    int KS, ncols;
};
struct QkvExtra {
    const float *q_bias, *k_bias, *v_bias;  // [qd], [kvd], [kvd] or nullptr
    int eff_dim, neox;
};

template <bool F16, bool GEN>
__global__ void rope_store_general_kernel(const float *__restrict__ P, int KS, int M, const float *__restrict__ inv_scale, RowNorm rn,
                                          float *__restrict__ q_out, const int32_t *__restrict__ positions,
                                          const int32_t *__restrict__ slot_mapping, void *__restrict__ pool,
                                          int num_q_heads, int num_kv_heads, int head_dim, int block_size, float theta,
                                          QkvExtra ex, VSrc vs, float *__restrict__ k_out = nullptr,
                                          float *__restrict__ v_out = nullptr) {
    static_assert(GEN, "the interleaved whole-head form is rope_store_partials_kernel");
    const int row = blockIdx.x, half = head_dim / 2, he = ex.eff_dim / 2;
    const int qd = num_q_heads * head_dim, kvd = num_kv_heads * head_dim, ncols = vs.P ? qd + kvd : qd + 2 * kvd;
    const size_t slice_elems = (size_t)M * ncols;
    const float inv = row_factor(inv_scale, rn, row);  // every wave of the block, before any lane leaves
    const int pos = positions[row], slot = slot_mapping[row];
    const int blk = slot / block_size, off = slot % block_size;
    const size_t part = (size_t)block_size * kvd;
    const size_t kbase = (size_t)blk * 2 * part + (size_t)off * kvd, vbase = kbase + part;
    const int lanes = blockDim.x / half, hl = threadIdx.x / half, j = threadIdx.x % half;
    if (hl >= lanes) return;
    const int hstride = lanes * gridDim.y, h0 = blockIdx.y * lanes + hl;
    // thread j: rotation pair j, or past the rotated part two neighbouring dimensions that are only carried over
    const bool turn = j < he;
    const int i0 = turn ? (ex.neox ? j : 2 * j) : ex.eff_dim + 2 * (j - he);
    const int i1 = turn ? (ex.neox ? j + he : 2 * j + 1) : i0 + 1;
    float c = 1.f, sn = 0.f;
    if (turn) {
        const double e = (double)(2 * j) / (double)ex.eff_dim;
        const float freq = (float)(1.0 / pow((double)theta, e));
        const float angle = __fmul_rn((float)pos, freq);
        c = (float)cos((double)angle);
        sn = (float)sin((double)angle);
    }
    auto elem = [&](int col, const float *bias, int bcol) {
        const float *p0 = P + (size_t)row * ncols + col;
        float v = *p0;
        for (int s = 1; s < KS; s++) v += p0[(size_t)s * slice_elems];
        v = __fmul_rn(v, inv);
        return bias ? __fadd_rn(v, bias[bcol]) : v;
    };
    auto velem = [&](int bcol) {
        if (!vs.P) return elem(qd + kvd + bcol, ex.v_bias, bcol);
        const float *p0 = vs.P + (size_t)row * vs.ncols + bcol;
        float v = *p0;
        for (int s = 1; s < vs.KS; s++) v += p0[(size_t)s * M * vs.ncols];
        v = __fmul_rn(v, inv);
        return ex.v_bias ? __fadd_rn(v, ex.v_bias[bcol]) : v;
    };
    for (int h = h0; h < num_q_heads; h += hstride) {
        const int b0 = h * head_dim + i0, b1 = h * head_dim + i1;
        const float a = elem(b0, ex.q_bias, b0), b = elem(b1, ex.q_bias, b1);
        q_out[(size_t)row * qd + b0] = turn ? __fsub_rn(__fmul_rn(a, c), __fmul_rn(b, sn)) : a;
        q_out[(size_t)row * qd + b1] = turn ? __fadd_rn(__fmul_rn(a, sn), __fmul_rn(b, c)) : b;
    }
    for (int h = h0; h < num_kv_heads; h += hstride) {
        const int b0 = h * head_dim + i0, b1 = h * head_dim + i1;
        const float a = elem(qd + b0, ex.k_bias, b0), b = elem(qd + b1, ex.k_bias, b1);
        const float va = velem(b0), vb = velem(b1);
        const float ka = turn ? __fsub_rn(__fmul_rn(a, c), __fmul_rn(b, sn)) : a;
        const float kb = turn ? __fadd_rn(__fmul_rn(a, sn), __fmul_rn(b, c)) : b;
        if (k_out) {  // (a prompt's first chunk: the rows also as dense floats for the attention that follows)
            k_out[(size_t)row * kvd + b0] = ka;
            k_out[(size_t)row * kvd + b1] = kb;
            v_out[(size_t)row * kvd + b0] = va;
            v_out[(size_t)row * kvd + b1] = vb;
        }
        if (F16) {
            _Float16 *pp = (_Float16 *)pool;
            pp[kbase + b0] = (_Float16)ka;
            pp[kbase + b1] = (_Float16)kb;
            pp[vbase + b0] = (_Float16)va;
            pp[vbase + b1] = (_Float16)vb;
        } else {
            float *pp = (float *)pool;
            pp[kbase + b0] = ka;
            pp[kbase + b1] = kb;
            pp[vbase + b0] = va;
            pp[vbase + b1] = vb;
        }
    }
}

template <bool F16>
__global__ void rope_store_partials_kernel(const float *__restrict__ P, int KS, int M, const float *__restrict__ inv_scale, RowNorm rn,
                                           float *__restrict__ q_out, const int32_t *__restrict__ positions,
                                           const int32_t *__restrict__ slot_mapping, void *__restrict__ pool,
                                           int num_q_heads, int num_kv_heads, int head_dim, int block_size, float theta,
                                           VSrc vs, const float2 *__restrict__ cs_tab = nullptr, float *__restrict__ k_out = nullptr,
                                           float *__restrict__ v_out = nullptr) {
    const int row = blockIdx.x, half = head_dim / 2;
    const int qd = num_q_heads * head_dim, kvd = num_kv_heads * head_dim, ncols = vs.P ? qd + kvd : qd + 2 * kvd;
    const size_t slice_elems = (size_t)M * ncols;
    const float inv = row_factor(inv_scale, rn, row);  // every wave of the block, before any lane leaves
    const int pos = positions[row], slot = slot_mapping[row];
    const int blk = slot / block_size, off = slot % block_size;
    const size_t part = (size_t)block_size * kvd;
    const size_t kbase = (size_t)blk * 2 * part + (size_t)off * kvd, vbase = kbase + part;
    const int lanes = blockDim.x / half, hl = threadIdx.x / half, j = threadIdx.x % half;
    if (hl >= lanes) return;
    const int hstride = lanes * gridDim.y, h0 = blockIdx.y * lanes + hl;
    float c, sn;
    if (cs_tab) {  // the step's table of angles (rope_table_kernel: the arithmetic below, once per row and pair)
        const float2 cs = cs_tab[(size_t)row * half + j];
        c = cs.x;
        sn = cs.y;
    } else {
        const double ex = (double)(2 * j) / (double)head_dim;
        const float freq = (float)(1.0 / pow((double)theta, ex));
        const float angle = __fmul_rn((float)pos, freq);
        c = (float)cos((double)angle);
        sn = (float)sin((double)angle);
    }
    auto pair = [&](int col, float &a, float &b) {
        const float *p0 = P + (size_t)row * ncols + col;
        float2 v = *(const float2 *)p0;
        for (int s = 1; s < KS; s++) {
            const float2 t = *(const float2 *)(p0 + (size_t)s * slice_elems);
            v.x += t.x;
            v.y += t.y;
        }
        a = __fmul_rn(v.x, inv);
        b = __fmul_rn(v.y, inv);
    };
    auto vpair = [&](int col, float &a, float &b) {
        if (!vs.P) {
            pair(qd + kvd + col, a, b);
            return;
        }
        const float *p0 = vs.P + (size_t)row * vs.ncols + col;
        float2 v = *(const float2 *)p0;
        for (int s = 1; s < vs.KS; s++) {
            const float2 t = *(const float2 *)(p0 + (size_t)s * M * vs.ncols);
            v.x += t.x;
            v.y += t.y;
        }
        a = __fmul_rn(v.x, inv);
        b = __fmul_rn(v.y, inv);
    };
    for (int h = h0; h < num_q_heads; h += hstride) {
        float a, b;
        pair(h * head_dim + 2 * j, a, b);
        float2 o;
        o.x = __fsub_rn(__fmul_rn(a, c), __fmul_rn(b, sn));
        o.y = __fadd_rn(__fmul_rn(a, sn), __fmul_rn(b, c));
        *(float2 *)(q_out + (size_t)row * qd + h * head_dim + 2 * j) = o;
    }
    for (int h = h0; h < num_kv_heads; h += hstride) {
        float a, b, va, vb;
        pair(qd + h * head_dim + 2 * j, a, b);
        vpair(h * head_dim + 2 * j, va, vb);
        const float ka = __fsub_rn(__fmul_rn(a, c), __fmul_rn(b, sn));
        const float kb = __fadd_rn(__fmul_rn(a, sn), __fmul_rn(b, c));
        const size_t o = (size_t)h * head_dim + 2 * j;
        if (k_out) {  // (a prompt's first chunk: the rows also as dense floats for the attention that follows)
            *(float2 *)(k_out + (size_t)row * kvd + o) = make_float2(ka, kb);
            *(float2 *)(v_out + (size_t)row * kvd + o) = make_float2(va, vb);
        }
        if (F16) {
            _Float16 *pp = (_Float16 *)pool;
            pp[kbase + o] = (_Float16)ka;
            pp[kbase + o + 1] = (_Float16)kb;
            pp[vbase + o] = (_Float16)va;
            pp[vbase + o + 1] = (_Float16)vb;
        } else {
            float *pp = (float *)pool;
            pp[kbase + o] = ka;
            pp[kbase + o + 1] = kb;
            pp[vbase + o] = va;
            pp[vbase + o + 1] = vb;
        }
    }
}

// (cos, sin) of every (row, pair): rope_store_partials_kernel's angle arithmetic (backend/cpu/cpu.go:226-303 for one
// position per row), once per step instead of once per layer. grid = rows, block = head_dim / 2.
__global__ void rope_table_kernel(const int32_t *__restrict__ positions, float2 *__restrict__ tab, int head_dim, float theta) {
    const int row = blockIdx.x, j = threadIdx.x, half = head_dim / 2;
    const double ex = (double)(2 * j) / (double)head_dim;
    const float freq = (float)(1.0 / pow((double)theta, ex));
    const float angle = __fmul_rn((float)positions[row], freq);
    tab[(size_t)row * half + j] = make_float2((float)cos((double)angle), (float)sin((double)angle));
}

size_t fmt_row_bytes(int fmt, int k) {
    switch (fmt) {
    case VX_Q4_0: return (size_t)k / 32 * 18;
    case VX_Q8_0: return (size_t)k / 32 * 34;
    case VX_Q4_K: return (size_t)k / 256 * 144;
    case VX_Q6_K: return (size_t)k / 256 * 210;
    case VX_Q5_0: return (size_t)k / 32 * 22;
    case VX_Q5_K: return (size_t)k / 256 * 176;
    case VX_BF16: return (size_t)k * 2;
    }
    return 0;
}

int mpad_for(int m) { return m <= 16 ? 16 : ceil_div(m, 32) * 32; }

PrepView prep_view(vx_backend *be, int mpad, int k) {
    PrepView pv;
    // the row scales sit first, at an address that does not depend on K: a fused consumer reads the
    // scales of the activation that produced its input while it prepares an activation of another width
    // two arrays, used alternately (prep_begin switches): the kernel that prepares the next activation writes
    // the new factors while it still reads the previous ones
    char *base = (char *)be->gemm_ws;
    const size_t rf = (size_t)ceil_div(mpad, 64) * 64 * 4;
    pv.inv_scale = (float *)(base + be->rowfac_slot * rf);
    pv.tiles = (half8 *)(base + 2 * rf);
    pv.bsum = (float *)((char *)pv.tiles + prep_tiles_bytes(mpad, k));
    pv.cscale = pv.bsum + (size_t)(k / 32) * mpad;
    return pv;
}

// Makes the prepared-activation workspace hold an [m,k] activation; returns its view.
int prep_begin(vx_backend *be, int m, int k, PrepView *pv) {
    VX_REQUIRE(m >= 1 && k >= 256 && k % 256 == 0, "prepare: bad shape %dx%d (K must be a multiple of 256)", m, k);
    const int mpad = mpad_for(m);
    const size_t need = prep_tiles_bytes(mpad, k) + 2 * (size_t)ceil_div(mpad, 64) * 64 * 4 + (size_t)(k / 32) * mpad * 4 +
                        (size_t)(k / 256) * mpad * 4;
    int rc = ensure_ws(be, &be->gemm_ws, &be->gemm_ws_bytes, need, "prepared activations");
    if (rc) return rc;
    be->rowfac_slot ^= 1;
    be->prep_norm_k = 0;
    be->split.merged = 0;  // whatever the attention kernel prepared is overwritten
    *pv = prep_view(be, mpad, k);
    be->prep_m = m;
    be->prep_k = k;
    return VX_OK;
}

// Number of k-slices for a GEMM of rg row groups (128 weight rows each) and n_chunks 256-column chunks: the count
// that minimises a small model of the kernel's critical path, fitted to measurements of the 7B shapes at 32
// rows. A compute unit holds two workgroups at a time; two together take about 1.4 times as long as one alone,
// a third waits. Each slice costs a fixed 0.2 chunk times (the consumer's pass over it) plus its [M,N] float32
// partial sums' trip through memory, which grows with the matrix' height.
// VEXEL_HIP_KS="NxK:slices,..." (row groups x chunks, e.g. "96x16:4") overrides the choice for tuning.
int gemm_cus(vx_backend *be) {
    static int cus = 0;
    if (cus == 0) {
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, be->device) != hipSuccess || cus <= 0) cus = 256;
    }
    return cus;
}

int gemm_slices(vx_backend *be, int rg, int n_chunks) {
    const int cus = gemm_cus(be);
    static const char *env = getenv("VEXEL_HIP_KS");
    if (env) {
        char key[64];
        snprintf(key, sizeof key, "%dx%d:", rg, n_chunks);
        const char *p = strstr(env, key);
        if (p) return std::max(1, std::min(n_chunks, atoi(p + strlen(key))));
    }
    int best = 1;
    float best_cost = 0.f;
    for (int ks = 1; ks <= std::min(n_chunks, 32); ks++) {
        const int per_cu = ceil_div(rg * ks, cus);  // workgroups on the busiest compute unit
        const float rounds = (float)(per_cu / 2) * 1.4f + (float)(per_cu % 2);
        const float per_slice = 0.2f + 0.8f * (float)rg / (float)cus;
        const float cost = (float)ceil_div(n_chunks, ks) * rounds + per_slice * (float)ks;
        if (ks == 1 || cost < best_cost) {
            best = ks;
            best_cost = cost;
        }
    }
    return best;
}

// Grows the prepared-activation workspace for an [m, kmax] activation now, so that later prepares
// of narrower activations inside one fused sequence cannot reallocate it (and lose the row scales).
int prep_reserve(vx_backend *be, int m, int kmax) {
    const int mpad = mpad_for(m);
    const size_t need = prep_tiles_bytes(mpad, kmax) + 2 * (size_t)ceil_div(mpad, 64) * 64 * 4 + (size_t)(kmax / 32) * mpad * 4 +
                        (size_t)(kmax / 256) * mpad * 4;
    return ensure_ws(be, &be->gemm_ws, &be->gemm_ws_bytes, need, "prepared activations");
}

template <class F>
int launch_gemm(vx_backend *be, const Segs &segs, int N, float *out, const float *residual, bool to_partials, int M,
                int K, int *ks_out) {
    const int mpad = mpad_for(M);
    const PrepView pv = prep_view(be, mpad, K);
    constexpr int R = 2;
    const int rg = ceil_div(N, 64 * R);
    const int mgroups = mpad <= 16 ? 1 : mpad / 32;
    const int n_chunks = ceil_div(K / 32, CH);
    // How many slices to cut K into depends on (N, K) and the device only, never on M: a row has the same bits
    // alone or in a batch. With few rows every slice is a workgroup of its own (grid.y) and the slices' sums go
    // through memory; once the row groups and 32-row activation groups alone fill the device twice over, one
    // workgroup per (row group, activation group) walks the slices in order instead (no partial sums). Both
    // forms add the same numbers in the same order.
    const int n_slices = gemm_slices(be, rg, n_chunks);
    const bool serial = mgroups > 1 && n_slices > 1 && rg * mgroups >= 2 * gemm_cus(be);
    const int ks = serial ? 1 : n_slices;
    float *partial = nullptr;
    if (ks > 1 || to_partials) {
        const size_t need = (size_t)ks * M * N * sizeof(float);
        int rc = ensure_ws(be, &be->part_ws, &be->part_ws_bytes, need, "split-K partial sums");
        if (rc) return rc;
        partial = (float *)be->part_ws;
    }
    dim3 grid(rg, ks, mgroups);
    const bool vec = N % 4 == 0 && ((uintptr_t)out % 16) == 0 && ((uintptr_t)residual % 16) == 0;
    const int flags = vec ? 1 : 0;
    if (mpad <= 16)
        qgemm_kernel<F, R, 1, false><<<grid, 256, 0, be->stream>>>(segs, pv, out, residual, partial, M, mpad, N, K, n_slices, flags);
    else if (!serial)
        qgemm_kernel<F, R, 2, false><<<grid, 256, 0, be->stream>>>(segs, pv, out, residual, partial, M, mpad, N, K, n_slices, flags);
    else
        qgemm_kernel<F, R, 2, true><<<grid, 256, 0, be->stream>>>(segs, pv, out, residual, partial, M, mpad, N, K, n_slices, flags);
    VX_CHECK_LAUNCH();
    if (ks_out) *ks_out = ks;
    if (partial && !to_partials) {
        const size_t total = (size_t)M * N;
        qgemm_reduce_kernel<<<(unsigned)((total + 255) / 256), 256, 0, be->stream>>>(partial, pv.inv_scale, out,
                                                                                      residual, M, N, ks);
        VX_CHECK_LAUNCH();
    }
    return VX_OK;
}

// ---- the wave-private kernel (qgemm_wave.h): which shapes take it, and how the matrix is cut
struct WavePlan {
    int r;   // weight tiles (16 rows) per workgroup; 0: the shape stays on qgemm_kernel
    int ks;  // K slices
};

// Depends on the format, the matrix and on whether M is above 32 only, so that a row's bits do not depend on the
// batch it sits in within 2 .. 32 and within 33 .. 64 rows. One workgroup per compute unit: the plan with the shortest modelled time among those whose workgroups all
// run at once. VEXEL_HIP_WPLAN="NxK:R,KS;..." overrides (tuning).
// (up to 64 activation rows: with more, every further group of rows would stage and unpack the weights again from
// eight waves' separate slices, and qgemm_kernel's shared staging is quicker)
WavePlan wave_plan(vx_backend *be, int fmt, const Segs &segs, int N, int K, int M) {
    WavePlan none = {0, 1};
    // 33 .. 64 rows: four activation tiles a step, whose sums and operand ring leave room for 3 weight tiles a
    // workgroup; tall matrices then take several rounds of workgroups (measured at 64 rows against qgemm_kernel:
    // 0.79 of its time for Q4_0, 0.87 for Q8_0, 0.75 for Q4_K over the four projections of a 7B / 8B layer)
    const bool rows64 = M > 32 && M <= 64 && fmt != VX_BF16;
    if (M > 32 && fmt != VX_BF16 && !rows64) return none;  // (BF16 has no other matrix-core kernel: it takes the groups of 32 rows)
    static const char *off = getenv("VEXEL_HIP_WAVE_OFF");
    if (off && atoi(off)) return none;
    if (fmt != VX_Q4_0 && fmt != VX_Q8_0 && fmt != VX_Q4_K && fmt != VX_BF16) return none;
    if (K % 256 != 0 || N % 16 != 0 || N < 64) return none;
    const int cus = gemm_cus(be), tiles = N / 16, n_chunks = K / 256;
    auto fits = [&](int r) {
        if (N < 16 * r) return false;
        for (int i = 0; i < 2; i++)
            if (segs.n_end[i] < N && segs.n_end[i] % (16 * r) != 0) return false;
        return true;
    };
    static const char *env = getenv("VEXEL_HIP_WPLAN");
    if (env) {
        char key[64];
        snprintf(key, sizeof key, "%dx%d:", N, K);
        const char *p = strstr(env, key);
        if (p) {
            int r = 0, ks = 1;
            if (sscanf(p + strlen(key), "%d,%d", &r, &ks) == 2 && fits(r)) return WavePlan{r, std::max(1, std::min(ks, n_chunks))};
        }
    }
    // more than 6 tiles a workgroup would spill registers: taller matrices (output heads) stay on qgemm_kernel
    const int max_r = rows64 ? 3 : (fmt == VX_Q8_0 ? 4 : (fmt == VX_BF16 ? 2 : 6));  // (wider staging leaves room for fewer tiles)
    const bool rounds = fmt == VX_BF16 || rows64;
    if (tiles > max_r * cus && !rounds) return none;
    static const int rs[] = {1, 2, 3, 4, 6};
    WavePlan best = none;
    float best_cost = 0.f;
    for (int r : rs) {
        if (!fits(r) || r > max_r) continue;
        const int rg = ceil_div(tiles, r);
        for (int ks = 1; ks <= std::min(n_chunks, 8); ks++) {
            if (rg * ks > cus && !(rounds && ks == 1 && r == max_r)) continue;  // (a tall BF16 matrix: several rounds of workgroups)
            const int wg_chunks = ceil_div(n_chunks, ks), wave_chunks = ceil_div(wg_chunks, 8);
            // In cycles, fitted to the 7B shapes at 32 rows: a wave's tile steps share a SIMD with one other
            // wave's (about 220 cycles a tile step for the pair); a compute unit pulls the 32 KB of activation
            // tiles of a chunk at about 32 bytes a cycle; slicing K costs the partial sums' trip through memory, the
            // consumer's pass over every slice, and the epilogues that only a whole sum can run.
            const float compute = (float)wave_chunks * 8.f * (float)r * 220.f;
            const float operand = (float)wg_chunks * 1024.f;
            const float part = ks > 1 ? (float)ks * (float)N * 0.06f + 5000.f : 0.f;
            const float cost = std::max(compute, operand) + part;
            if (best.r == 0 || cost < best_cost) {
                best = WavePlan{r, ks};
                best_cost = cost;
            }
        }
    }
    return best;
}

constexpr int WAVE_MT4_MAX_R = 3;  // weight tiles per workgroup up to which 64 activation rows' sums fit the registers

template <class W, int R>
int launch_gemm_wave(vx_backend *be, const Segs &segs, int N, float *out, const float *residual, bool to_partials, int M,
                     int K, int ks, int *ks_out, const QkvEpi &epi) {
    constexpr int NW = 8;
    const int mpad = mpad_for(M);
    const PrepView pv = prep_view(be, mpad, K);
    // activation rows per workgroup: 16, 32 or (33 .. 64 rows, where the tiles fit the registers) 64; beyond, groups of 32
    constexpr bool MT4 = R <= (W::PITCH >= 256 ? 1 : WAVE_MT4_MAX_R);
    const bool four = MT4 && mpad == 64;
    const int rg = ceil_div(N, 16 * R), mgroups = mpad <= 16 || four ? 1 : mpad / 32;
    float *partial = nullptr;
    if (ks > 1 || to_partials) {
        int rc = ensure_ws(be, &be->part_ws, &be->part_ws_bytes, (size_t)ks * M * N * sizeof(float), "split-K partial sums");
        if (rc) return rc;
        partial = (float *)be->part_ws;
    }
    dim3 grid(rg, ks, mgroups);
    const bool vec = ((uintptr_t)out % 16) == 0 && ((uintptr_t)residual % 16) == 0;
    const int n_chunks = K / 256, slices = ((n_chunks / ks) << 16) | (n_chunks % ks);  // the kernel takes the division done
    if (mpad <= 16)
        qgemm_wave_kernel<W, R, 1, NW><<<grid, 64 * NW, 0, be->stream>>>(segs, pv, out, residual, partial, M, mpad, N, K, slices, vec ? 1 : 0, epi);
    else if (!four)
        qgemm_wave_kernel<W, R, 2, NW><<<grid, 64 * NW, 0, be->stream>>>(segs, pv, out, residual, partial, M, mpad, N, K, slices, vec ? 1 : 0, epi);
    else if constexpr (MT4)
        qgemm_wave_kernel<W, R, 4, NW><<<grid, 64 * NW, 0, be->stream>>>(segs, pv, out, residual, partial, M, mpad, N, K, slices, vec ? 1 : 0, epi);
    VX_CHECK_LAUNCH();
    if (ks_out) *ks_out = ks;
    if (partial && !to_partials) {
        const size_t total = (size_t)M * N;
        qgemm_reduce_kernel<<<(unsigned)((total + 255) / 256), 256, 0, be->stream>>>(partial, pv.inv_scale, out, residual, M, N, ks);
        VX_CHECK_LAUNCH();
    }
    return VX_OK;
}

template <class W>
int launch_gemm_wave_r(vx_backend *be, const WavePlan &pl, const Segs &segs, int N, float *out, const float *residual,
                       bool to_partials, int M, int K, int *ks_out, const QkvEpi &epi) {
    if (pl.r == 1) return launch_gemm_wave<W, 1>(be, segs, N, out, residual, to_partials, M, K, pl.ks, ks_out, epi);
    if (pl.r == 2) return launch_gemm_wave<W, 2>(be, segs, N, out, residual, to_partials, M, K, pl.ks, ks_out, epi);
    if constexpr (W::PITCH < 256) {  // (the narrow formats: more tiles fit the registers and the LDS)
        switch (pl.r) {
        case 3: return launch_gemm_wave<W, 3>(be, segs, N, out, residual, to_partials, M, K, pl.ks, ks_out, epi);
        case 4: return launch_gemm_wave<W, 4>(be, segs, N, out, residual, to_partials, M, K, pl.ks, ks_out, epi);
        case 6: return launch_gemm_wave<W, 6>(be, segs, N, out, residual, to_partials, M, K, pl.ks, ks_out, epi);
        }
    }
    set_error("wave GEMM: no kernel for %d tiles per workgroup", pl.r);
    return VX_ERR_INVALID;
}

// The many-rows kernel's cut for (N, K) at M rows: R tiles per wave (128 R weight rows per workgroup) and K slices;
// r = 0: not served. Wide cuts first; slices only when even 128-row workgroups leave compute units idle.
// VEXEL_HIP_RPLAN="NxK:R,KS;..." overrides, VEXEL_HIP_ROWS_MIN=<rows> moves the smallest batch it takes.
WavePlan rows_plan(vx_backend *be, int fmt, const Segs &segs, int N, int K, int M) {
    WavePlan none = {0, 1};
    static const int min_rows = getenv("VEXEL_HIP_ROWS_MIN") ? atoi(getenv("VEXEL_HIP_ROWS_MIN")) : 97;
    // Q8_0 only: measured against qgemm_kernel at 128 / 256 / 512 rows it takes 0.86 / 0.83 / 0.75 of the time there,
    // while Q4_0 comes out even (its unpack is cheaper to repeat) and Q4_K's decoder does not fit the registers
    if (M < min_rows || fmt != VX_Q8_0) return none;
    if (K % 256 != 0 || N % 16 != 0 || N < 16) return none;
    const int cus = gemm_cus(be), n_chunks = K / 256, mgroups = ceil_div(mpad_for(M), 64);
    auto fits = [&](int r) {
        if (N % (16 * r) != 0) return false;
        for (int i = 0; i < 2; i++)
            if (segs.n_end[i] < N && segs.n_end[i] % (16 * r) != 0) return false;
        return true;
    };
    static const char *env = getenv("VEXEL_HIP_RPLAN");
    if (env) {
        char key[64];
        snprintf(key, sizeof key, "%dx%d:", N, K);
        const char *p = strstr(env, key);
        if (p) {
            int r = 0, ks = 1;
            if (sscanf(p + strlen(key), "%d,%d", &r, &ks) == 2 && (r == 1 || r == 2) && fits(r))
                return WavePlan{r, std::max(1, std::min(ks, n_chunks))};
        }
    }
    for (int r : {2, 1}) {  // (four tiles a wave need more registers than there are)
        if (!fits(r)) continue;
        const int wgs = ceil_div(N, 128 * r) * mgroups;
        if (wgs * 2 >= cus || r == 1) return WavePlan{r, std::max(1, std::min(std::min(n_chunks, 8), cus / std::max(wgs, 1)))};
    }
    return none;
}

template <class W, int R>
int launch_gemm_rows(vx_backend *be, const Segs &segs, int N, float *out, const float *residual, bool to_partials, int M,
                     int K, int ks, int *ks_out) {
    const int mpad = mpad_for(M);
    const PrepView pv = prep_view(be, mpad, K);
    float *partial = nullptr;
    if (ks > 1 || to_partials) {
        int rc = ensure_ws(be, &be->part_ws, &be->part_ws_bytes, (size_t)ks * M * N * sizeof(float), "split-K partial sums");
        if (rc) return rc;
        partial = (float *)be->part_ws;
    }
    const int n_chunks = K / 256, slices = ((n_chunks / ks) << 16) | (n_chunks % ks);
    dim3 grid(ceil_div(N, 128 * R), ks, ceil_div(mpad, 64));
    qgemm_rows_kernel<W, R, 4><<<grid, 512, 0, be->stream>>>(segs, pv, out, residual, partial, M, mpad, N, K, slices);
    VX_CHECK_LAUNCH();
    if (ks_out) *ks_out = ks;
    if (partial && !to_partials) {
        const size_t total = (size_t)M * N;
        qgemm_reduce_kernel<<<(unsigned)((total + 255) / 256), 256, 0, be->stream>>>(partial, pv.inv_scale, out, residual, M, N, ks);
        VX_CHECK_LAUNCH();
    }
    return VX_OK;
}

template <class W>
int launch_gemm_rows_r(vx_backend *be, const WavePlan &pl, const Segs &segs, int N, float *out, const float *residual,
                       bool to_partials, int M, int K, int *ks_out) {
    if (pl.r == 1) return launch_gemm_rows<W, 1>(be, segs, N, out, residual, to_partials, M, K, pl.ks, ks_out);
    return launch_gemm_rows<W, 2>(be, segs, N, out, residual, to_partials, M, K, pl.ks, ks_out);
}

RowNorm cur_row_norm(const vx_backend *be);

int launch_gemm_fmt(vx_backend *be, int fmt, const Segs &segs, int N, float *out, const float *residual,
                    bool to_partials, int M, int K, int *ks_out, const QkvEpi *epi_in = nullptr) {
    // packed copies of the matrices (vx_qweight_pack) and a decode-sized batch: the streaming kernel
    const bool fin = epi_in && epi_in->q_out;
    if (stream_gemm_ok(be, fmt, segs.w, segs.n_end, 3, N, K, M, fin)) {
        int ks = 1;
        const int mpad = mpad_for(M);
        const PrepView spv = prep_view(be, mpad, K);
        int rc = stream_gemm(be, fmt, segs.w, segs.n_end, 3, N, K, M, mpad, spv, epi_in, &ks);
        if (rc != VX_ERR_UNSUPPORTED) {
            if (rc) return rc;
            be->last_matmul = "qstream_kernel";
            if (ks_out) *ks_out = ks;
            if (!fin && !to_partials) {
                const size_t total = (size_t)M * N;
                qgemm_reduce_kernel<<<(unsigned)((total + 255) / 256), 256, 0, be->stream>>>((const float *)be->part_ws, spv.inv_scale, out,
                                                                                              residual, M, N, ks);
                VX_CHECK_LAUNCH();
            }
            return VX_OK;
        }
    }
    if (tiles_gemm_ok(be, fmt, segs.w, segs.n_end, 3, N, K, M)) {  // packed copies and a batch beyond the streaming kernel's
        int ks = 1;
        const int mpad = mpad_for(M);
        const PrepView spv = prep_view(be, mpad, K);
        // (a pending 1/rms: this launch folds it into the plain row factors beside its own work, for whoever
        // consumes its K slices' sums)
        const bool fold = to_partials && be->prep_norm_k > 0;
        const RowNorm fin = cur_row_norm(be);
        int rc = tiles_gemm(be, fmt, segs.w, segs.n_end, 3, N, K, M, mpad, spv, out, residual, to_partials, &ks, fold ? &fin : nullptr);
        if (rc != VX_ERR_UNSUPPORTED) {
            if (rc) return rc;
            if (fold) be->prep_norm_k = 0;
            be->last_matmul = "qtiles_kernel";
            if (ks_out) *ks_out = ks;
            if (!to_partials && ks > 1) {
                const size_t total = (size_t)M * N;
                qgemm_reduce_kernel<<<(unsigned)((total + 255) / 256), 256, 0, be->stream>>>((const float *)be->part_ws, spv.inv_scale, out,
                                                                                              residual, M, N, ks);
                VX_CHECK_LAUNCH();
            }
            return VX_OK;
        }
    }
    const WavePlan rp = rows_plan(be, fmt, segs, N, K, M);
    if (rp.r > 0) {
        be->last_matmul = "qgemm_rows_kernel";
        return launch_gemm_rows_r<WQ8_0>(be, rp, segs, N, out, residual, to_partials, M, K, ks_out);
    }
    const QkvEpi epi = epi_in ? *epi_in : QkvEpi{};  // (with an epilogue the caller has checked that the wave plan applies)
    const WavePlan pl = wave_plan(be, fmt, segs, N, K, M);
    if (pl.r > 0) {
        be->last_matmul = "qgemm_wave_kernel";
        if (fmt == VX_Q4_0) return launch_gemm_wave_r<WQ4_0>(be, pl, segs, N, out, residual, to_partials, M, K, ks_out, epi);
        if (fmt == VX_Q8_0) return launch_gemm_wave_r<WQ8_0>(be, pl, segs, N, out, residual, to_partials, M, K, ks_out, epi);
        if (fmt == VX_BF16) return launch_gemm_wave_r<WBF16>(be, pl, segs, N, out, residual, to_partials, M, K, ks_out, epi);
        return launch_gemm_wave_r<WQ4_K>(be, pl, segs, N, out, residual, to_partials, M, K, ks_out, epi);
    }
    be->last_matmul = "qgemm_kernel";
    switch (fmt) {
    case VX_Q4_0: return launch_gemm<PQ4_0>(be, segs, N, out, residual, to_partials, M, K, ks_out);
    case VX_Q8_0: return launch_gemm<PQ8_0>(be, segs, N, out, residual, to_partials, M, K, ks_out);
    case VX_Q6_K: return launch_gemm<PQ6_K>(be, segs, N, out, residual, to_partials, M, K, ks_out);
    case VX_Q5_0: return launch_gemm<PQ5_0>(be, segs, N, out, residual, to_partials, M, K, ks_out);
    case VX_Q5_K: return launch_gemm<PQ5_K>(be, segs, N, out, residual, to_partials, M, K, ks_out);
    default: return launch_gemm<PQ4_K>(be, segs, N, out, residual, to_partials, M, K, ks_out);
    }
}

// Q6_K rows are 210 bytes per 256 elements and need not start on 16-byte boundaries; its kernel stages
// them from the boundary below, which needs the whole matrix to be a multiple of 16 bytes.
bool fast_ok(int fmt, const void *b, int n, int k) {
    const size_t rb = fmt_row_bytes(fmt, k);
    if (fmt < VX_Q4_0 || fmt > VX_Q5_K) return false;  // BF16: the row kernel
    if (k % 256 != 0 || ((uintptr_t)b % 16) != 0 || n < 1) return false;
    return fmt == VX_Q6_K ? ((size_t)n * rb) % 16 == 0 : rb % 16 == 0;
}

int check_fmt(int fmt, int k) {
    if (fmt < VX_Q4_0 || fmt > VX_BF16) {
        set_error("quantized matmul: unknown format %d", fmt);
        return VX_ERR_UNSUPPORTED;
    }
    const int blk = fmt == VX_BF16 ? 1 : (fmt == VX_Q4_0 || fmt == VX_Q8_0 || fmt == VX_Q5_0) ? 32 : 256;
    VX_REQUIRE(k > 0 && k % blk == 0, "quantized matmul: K=%d is not a multiple of the block size %d", k, blk);
    return VX_OK;
}

// Pending RMSNorm of the currently prepared activation (none: sspart = NULL).
RowNorm cur_row_norm(const vx_backend *be) {
    RowNorm rn = {nullptr, 0, 0.f, 0.f};
    if (be->prep_norm_k > 0) {
        rn.sspart = (const float *)be->prep_sync + (size_t)be->rowfac_slot * VX_PREP_SYNC_CHUNKS * VX_PREP_SYNC_ROWS;
        rn.n_chunks = be->prep_norm_k / 256;
        rn.inv_k = 1.0f / (float)be->prep_norm_k;
        rn.eps = be->prep_norm_eps;
    }
    return rn;
}
float *cur_ss_out(vx_backend *be) {
    return (float *)be->prep_sync + (size_t)be->rowfac_slot * VX_PREP_SYNC_CHUNKS * VX_PREP_SYNC_ROWS;
}
// Folds a pending 1/rms into the plain row factors, for consumers that read only those.
int finalize_row_norm(vx_backend *be) {
    if (be->prep_norm_k <= 0) return VX_OK;
    const PrepView pv = prep_view(be, mpad_for(be->prep_m), be->prep_k);
    finalize_row_norm_kernel<<<be->prep_m, 64, 0, be->stream>>>(pv.inv_scale, cur_row_norm(be));
    VX_CHECK_LAUNCH();
    be->prep_norm_k = 0;
    return VX_OK;
}

int run_prepared(vx_backend *be, int fmt, const void *b, float *out, const float *residual, int m, int n, int k) {
    Segs segs;
    segs.w[0] = segs.w[1] = segs.w[2] = (const uint8_t *)b;
    segs.n_end[0] = segs.n_end[1] = segs.n_end[2] = n;
    int rc = finalize_row_norm(be);  // the GEMM epilogue and the reduce kernel read plain row factors
    if (rc) return rc;
    // without an output: the projection launch as the fused decode blocks issue it, its K slices' sums left in the
    // workspace for the consumer that follows there
    return launch_gemm_fmt(be, fmt, segs, n, out, residual, out == nullptr, m, k, nullptr);
}

}  // namespace

extern "C" {

int vx_prepare_act(vx_backend *be, const float *a, int m, int k) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(a && ((uintptr_t)a % 16 == 0), "vx_prepare_act: null or unaligned activation");
    PrepView pv;
    rc = prep_begin(be, m, k, &pv);
    if (rc) return rc;
    const int mpad = mpad_for(m);
    // beyond 256 rows a wave per row and 256-column chunk (each chunk with its own power-of-two factor): many small
    // workgroups instead of one of 1024 threads per row; up to there the row kernel, whose bits the decode paths share
    if (m > 256)
        chunk_plain_kernel<<<dim3(k / 256, mpad), 64, 0, be->stream>>>(a, m, k, pv, mpad);
    else
        prepare_kernel<PREP_PLAIN, false><<<mpad, PREP_THREADS, 0, be->stream>>>(a, nullptr, nullptr, m, k, 0.f, pv, mpad);
    VX_CHECK_LAUNCH();
    return VX_OK;
}

int vx_rmsnorm_prepare(vx_backend *be, const float *x, const float *weight, float *out, int rows, int cols, float eps) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(x && weight && ((uintptr_t)x % 16 == 0) && ((uintptr_t)weight % 16 == 0) && ((uintptr_t)out % 16 == 0),
               "vx_rmsnorm_prepare: null or unaligned pointer");
    PrepView pv;
    rc = prep_begin(be, rows, cols, &pv);
    if (rc) return rc;
    const int mpad = mpad_for(rows);
    prepare_kernel<PREP_RMSNORM, false><<<mpad, PREP_THREADS, 0, be->stream>>>(x, weight, out, rows, cols, eps, pv, mpad);
    VX_CHECK_LAUNCH();
    return VX_OK;
}

int vx_silu_mul_prepare(vx_backend *be, const float *gate, const float *up, float *out, int rows, int cols) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(gate && up && ((uintptr_t)gate % 16 == 0) && ((uintptr_t)up % 16 == 0) && ((uintptr_t)out % 16 == 0),
               "vx_silu_mul_prepare: null or unaligned pointer");
    PrepView pv;
    rc = prep_begin(be, rows, cols, &pv);
    if (rc) return rc;
    const int mpad = mpad_for(rows);
    if ((size_t)cols * 4 <= 48 * 1024)
        prepare_kernel<PREP_SILU_MUL, true><<<mpad, PREP_THREADS, (size_t)cols * 4, be->stream>>>(gate, up, out, rows, cols, 0.f,
                                                                                          pv, mpad);
    else
        prepare_kernel<PREP_SILU_MUL, false><<<mpad, PREP_THREADS, 0, be->stream>>>(gate, up, out, rows, cols, 0.f, pv, mpad);
    VX_CHECK_LAUNCH();
    return VX_OK;
}

int vx_gelu_mul_prepare(vx_backend *be, const float *gate, const float *up, float *out, int rows, int cols) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(gate && up && ((uintptr_t)gate % 16 == 0) && ((uintptr_t)up % 16 == 0) && ((uintptr_t)out % 16 == 0),
               "vx_gelu_mul_prepare: null or unaligned pointer");
    PrepView pv;
    rc = prep_begin(be, rows, cols, &pv);
    if (rc) return rc;
    const int mpad = mpad_for(rows);
    if ((size_t)cols * 4 <= 48 * 1024)
        prepare_kernel<PREP_GELU_MUL, true><<<mpad, PREP_THREADS, (size_t)cols * 4, be->stream>>>(gate, up, out, rows, cols, 0.f,
                                                                                          pv, mpad);
    else
        prepare_kernel<PREP_GELU_MUL, false><<<mpad, PREP_THREADS, 0, be->stream>>>(gate, up, out, rows, cols, 0.f, pv, mpad);
    VX_CHECK_LAUNCH();
    return VX_OK;
}

int vx_gelu_prepare(vx_backend *be, const float *x, float *out, int rows, int cols) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(x && ((uintptr_t)x % 16 == 0) && ((uintptr_t)out % 16 == 0), "vx_gelu_prepare: null or unaligned pointer");
    PrepView pv;
    rc = prep_begin(be, rows, cols, &pv);
    if (rc) return rc;
    const int mpad = mpad_for(rows);
    if ((size_t)cols * 4 <= 48 * 1024)
        prepare_kernel<PREP_GELU, true><<<mpad, PREP_THREADS, (size_t)cols * 4, be->stream>>>(x, nullptr, out, rows, cols, 0.f, pv, mpad);
    else
        prepare_kernel<PREP_GELU, false><<<mpad, PREP_THREADS, 0, be->stream>>>(x, nullptr, out, rows, cols, 0.f, pv, mpad);
    VX_CHECK_LAUNCH();
    return VX_OK;
}

int vx_matmul_quant_prepared(vx_backend *be, int fmt, const void *b, float *out, const float *residual, int m, int n,
                             int k) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(b && n >= 1 && (out || !residual), "vx_matmul_quant_prepared: bad arguments");
    rc = check_fmt(fmt, k);
    if (rc) return rc;
    VX_REQUIRE(be->prep_m == m && be->prep_k == k, "vx_matmul_quant_prepared: the prepared activation is %dx%d, not %dx%d",
               be->prep_m, be->prep_k, m, k);
    VX_REQUIRE(fast_ok(fmt, b, n, k), "vx_matmul_quant_prepared: format %d / N=%d / K=%d / alignment has no MFMA path", fmt, n, k);
    return run_prepared(be, fmt, b, out, residual, m, n, k);
}

int vx_matmul_quant_has_fast_path(int fmt, const void *b, int n, int k) { return fast_ok(fmt, b, n, k) ? 1 : 0; }

const char *vx_last_matmul_kernel(vx_backend *be) { return be ? be->last_matmul : ""; }

int vx_matmul_quant(vx_backend *be, int fmt, const float *a, const void *b, float *out, const float *residual, int m,
                    int n, int k) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(a && b && out, "vx_matmul_quant: null pointer");
    VX_REQUIRE(m >= 0 && n >= 0, "vx_matmul_quant: bad shape %dx%dx%d", m, n, k);
    rc = check_fmt(fmt, k);
    if (rc) return rc;
    if (m == 0 || n == 0) return VX_OK;
    static const bool no_matvec = getenv("VEXEL_HIP_NO_MATVEC") != nullptr;  // keeps M = 1 on the batched kernel
    if (m == 1 && !no_matvec) {  // a single row: the streaming matrix-vector kernel
        rc = run_matvec(be, fmt, a, b, out, residual, n, k);
        if (rc != VX_ERR_UNSUPPORTED) {
            be->last_matmul = "qmatvec_kernel";
            return rc;
        }
    }
    if (fmt == VX_BF16 && m >= 2 && k % 256 == 0 && ((uintptr_t)a % 16) == 0 && ((uintptr_t)b % 16) == 0) {
        // the matrix cores: bf16 -> f16 is exact for weights, the activations enter as hi + lo as everywhere
        Segs segs;
        segs.w[0] = segs.w[1] = segs.w[2] = (const uint8_t *)b;
        segs.n_end[0] = segs.n_end[1] = segs.n_end[2] = n;
        if (wave_plan(be, fmt, segs, n, k, m).r > 0) {
            rc = vx_prepare_act(be, a, m, k);
            if (rc) return rc;
            rc = finalize_row_norm(be);
            if (rc) return rc;
            return launch_gemm_fmt(be, fmt, segs, n, out, residual, false, m, k, nullptr);
        }
    }
    if (!fast_ok(fmt, b, n, k) || ((uintptr_t)a % 16) != 0) {
        const size_t rb = fmt_row_bytes(fmt, k);
        dim3 grid(n, ceil_div(m, FB_M));
        if (fmt > VX_Q6_K && k % 4 == 0 && ((uintptr_t)a % 16) == 0 && ((uintptr_t)b % 2) == 0) {
            const uint8_t *w = (const uint8_t *)b;
            if (fmt == VX_Q5_0) qrow4_kernel<VX_Q5_0><<<grid, 64, 0, be->stream>>>(w, a, out, residual, m, n, k, rb);
            else if (fmt == VX_Q5_K) qrow4_kernel<VX_Q5_K><<<grid, 64, 0, be->stream>>>(w, a, out, residual, m, n, k, rb);
            else qrow4_kernel<VX_BF16><<<grid, 64, 0, be->stream>>>(w, a, out, residual, m, n, k, rb);
            VX_CHECK_LAUNCH();
            be->last_matmul = "qrow4_kernel";
            return VX_OK;
        }
        qgemm_fallback_kernel<<<grid, 64, 0, be->stream>>>(fmt, (const uint8_t *)b, a, out, residual, m, n, k, rb);
        VX_CHECK_LAUNCH();
        be->last_matmul = "qgemm_fallback_kernel";
        return VX_OK;
    }
    rc = vx_prepare_act(be, a, m, k);
    if (rc) return rc;
    return run_prepared(be, fmt, b, out, residual, m, n, k);
}

static bool group_ok(const vx_qweight *const *ws, int nw) {
    for (int i = 0; i < nw; i++) {
        if (!ws[i] || !ws[i]->data) return false;
        if (ws[i]->fmt != ws[0]->fmt || ws[i]->k != ws[0]->k) return false;
        if (!fast_ok(ws[i]->fmt, ws[i]->data, ws[i]->n, ws[i]->k) || ws[i]->n % 16 != 0 || ws[i]->n <= 0) return false;
    }
    return true;
}

// Matrices that follow one another in memory (a loader that lays Q|K|V or gate|up out back to back) become one
// segment: the kernels then cut the rows where they like instead of at the matrices' boundaries.
static Segs make_segs(const vx_qweight *const *ws, int nw, int *ntot) {
    Segs sg;
    int acc = 0, ns = 0;
    const uint8_t *next = nullptr;  // where a matrix would have to start to continue the current segment
    for (int i = 0; i < nw; i++) {
        const vx_qweight *w = ws[i];
        const uint8_t *p = (const uint8_t *)w->data;
        acc += w->n;
        if (ns > 0 && p == next) {
            sg.n_end[ns - 1] = acc;
        } else {
            sg.w[ns] = p;
            sg.n_end[ns] = acc;
            ns++;
        }
        next = p + (size_t)w->n * fmt_row_bytes(w->fmt, w->k);
    }
    for (int i = ns; i < 3; i++) {  // unused slots repeat the last segment
        sg.w[i] = sg.w[ns - 1];
        sg.n_end[i] = acc;
    }
    *ntot = acc;
    return sg;
}

// The chunk-parallel prepares (a wave per row and 256-column chunk) cover decode batches, prompt chunks and trees of
// up to 512 rows; larger ones keep the one-workgroup-per-row kernels. VEXEL_HIP_PREP_ROW_KERNELS=1 (measurements):
// those from 65 rows on, as before the many-rows GEMM folded the pending 1/rms in.
bool chunk_prepare_ok(int rows, int k) {
    static const bool row_kernels = getenv("VEXEL_HIP_PREP_ROW_KERNELS") != nullptr;
    return mpad_for(rows) <= (row_kernels ? 64 : VX_PREP_SYNC_ROWS) && k / 256 <= VX_PREP_SYNC_CHUNKS;
}

extern "C++" {
namespace vx {
int prep_begin_chunked(vx_backend *be, int m, int k, PrepView *pv, int *mpad) {
    // (the attention kernel that merges its own splits into this form: decode batches of up to 64 rows)
    if (k < 256 || k % 256 != 0 || !chunk_prepare_ok(m, k) || mpad_for(m) > 64) return VX_ERR_UNSUPPORTED;
    *mpad = mpad_for(m);
    return prep_begin(be, m, k, pv);
}
}  // namespace vx
}
int vx_rope_table_prepare(vx_backend *be, const int32_t *positions, int rows, int head_dim, float theta) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(positions && rows >= 1 && head_dim >= 2 && head_dim % 2 == 0, "vx_rope_table_prepare: bad arguments");
    be->rope_tab_pos = nullptr;
    if (rows > VX_ROPE_TAB_ROWS || head_dim / 2 > VX_ROPE_TAB_PAIRS) return VX_OK;  // no table: the calls keep their own arithmetic
    rope_table_kernel<<<rows, head_dim / 2, 0, be->stream>>>(positions, (float2 *)be->rope_tab, head_dim, theta);
    VX_CHECK_LAUNCH();
    be->rope_tab_pos = positions;
    be->rope_tab_rows = rows;
    be->rope_tab_dim = head_dim;
    be->rope_tab_theta = theta;
    be->rope_tab_epoch = be->write_epoch;
    return VX_OK;
}

// Q and K of one format; V of the same, or of another with a matrix-core path (the Q4_K_M mixes keep attn_v in Q6_K):
// it then is a launch of its own between the shared prepare and the shared RoPE + store.
int vx_decode_attn_qkv_supported(const vx_qweight *wq, const vx_qweight *wk, const vx_qweight *wv, int head_dim) {
    const vx_qweight *ws[3] = {wq, wk, wv}, *wvs[1] = {wv};
    const bool ok = group_ok(ws, 3) || (group_ok(ws, 2) && group_ok(wvs, 1) && wv->k == wq->k);
    return ok && head_dim % 2 == 0 && head_dim <= 512 && (size_t)wq->k * 4 <= 64 * 1024;
}

int vx_decode_attn_qkv(vx_backend *be, const float *x, const float *norm_weight, float eps, int x_prepared,
                       const vx_qweight *wq, const vx_qweight *wk, const vx_qweight *wv, int rows,
                       const int32_t *positions, const int32_t *slot_mapping, void *kv_pool, int pool_is_f16,
                       int num_q_heads, int num_kv_heads, int head_dim, int block_size, float theta, float *q_out) {
    return vx_decode_attn_qkv_ex(be, x, norm_weight, eps, x_prepared, wq, wk, wv, nullptr, nullptr, nullptr, rows, positions,
                                 slot_mapping, kv_pool, pool_is_f16, num_q_heads, num_kv_heads, head_dim, block_size, theta, 0, 0,
                                 q_out);
}

int vx_decode_attn_qkv_ex(vx_backend *be, const float *x, const float *norm_weight, float eps, int x_prepared,
                          const vx_qweight *wq, const vx_qweight *wk, const vx_qweight *wv, const float *q_bias,
                          const float *k_bias, const float *v_bias, int rows, const int32_t *positions,
                          const int32_t *slot_mapping, void *kv_pool, int pool_is_f16, int num_q_heads, int num_kv_heads,
                          int head_dim, int block_size, float theta, int rope_dim, int rope_neox, float *q_out) {
    return vx_prefill_attn_qkv(be, x, norm_weight, eps, x_prepared, wq, wk, wv, q_bias, k_bias, v_bias, rows, positions,
                               slot_mapping, kv_pool, pool_is_f16, num_q_heads, num_kv_heads, head_dim, block_size, theta,
                               rope_dim, rope_neox, q_out, nullptr, nullptr);
}

int vx_prefill_attn_qkv(vx_backend *be, const float *x, const float *norm_weight, float eps, int x_prepared,
                        const vx_qweight *wq, const vx_qweight *wk, const vx_qweight *wv, const float *q_bias,
                        const float *k_bias, const float *v_bias, int rows, const int32_t *positions,
                        const int32_t *slot_mapping, void *kv_pool, int pool_is_f16, int num_q_heads, int num_kv_heads,
                        int head_dim, int block_size, float theta, int rope_dim, int rope_neox, float *q_out, float *k_out,
                        float *v_out) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE((k_out == nullptr) == (v_out == nullptr), "vx_prefill_attn_qkv: k_out and v_out go together");
    VX_REQUIRE(!k_out || (((uintptr_t)k_out % 8) == 0 && ((uintptr_t)v_out % 8) == 0), "vx_prefill_attn_qkv: unaligned output");
    const int eff_dim = rope_dim == 0 ? head_dim : rope_dim;
    VX_REQUIRE(eff_dim > 0 && eff_dim <= head_dim && eff_dim % 2 == 0, "vx_decode_attn_qkv: rope_dim %d invalid for head_dim %d",
               rope_dim, head_dim);
    // the interleaved whole-head form without biases keeps its own kernel
    const bool gen = q_bias || k_bias || v_bias || rope_neox || eff_dim != head_dim;
    const QkvExtra ex = {q_bias, k_bias, v_bias, eff_dim, rope_neox};
    if (!vx_decode_attn_qkv_supported(wq, wk, wv, head_dim)) {
        set_error("vx_decode_attn_qkv: weights have no fused MFMA path");
        return VX_ERR_UNSUPPORTED;
    }
    VX_REQUIRE(positions && slot_mapping && kv_pool && q_out && rows >= 1, "vx_decode_attn_qkv: bad arguments");
    VX_REQUIRE(wq->n == num_q_heads * head_dim && wk->n == num_kv_heads * head_dim && wv->n == wk->n && block_size >= 1,
               "vx_decode_attn_qkv: weight shapes do not match the head geometry");
    const int k = wq->k;
    static const bool no_matvec = getenv("VEXEL_HIP_NO_MATVEC") != nullptr;
    if (rows == 1 && !x_prepared && !no_matvec && pool_is_f16 && head_dim % 2 == 0 && !k_out) {
        // A single row: Q|K|V by one matrix-vector launch with the RMSNorm folded in (the row enters as x * w,
        // the dot products are divided by rms(x)), then RoPE and the KV store from that launch's output.
        const void *mw[3] = {wq->data, wk->data, wv->data};
        const int mn[3] = {wq->n, wk->n, wv->n};
        const int ntot1 = wq->n + wk->n + wv->n;
        const bool mixed1 = wv->fmt != wq->fmt;
        if (x && norm_weight && mixed1 && matvec_ok(wq->fmt, mw, mn, 2, k) && matvec_ok(wv->fmt, mw + 2, mn + 2, 1, k)) {
            // V in another format: its own launch, the outputs side by side
            rc = ensure_ws(be, &be->part_ws, &be->part_ws_bytes, (size_t)ntot1 * sizeof(float), "split-K partial sums");
            if (rc) return rc;
            MatvecSource src;
            src.x = x;
            src.norm_w = norm_weight;
            src.eps = eps;
            rc = run_matvec_fused(be, wq->fmt, mw, mn, 2, k, src, (float *)be->part_ws, nullptr, 0);
            if (rc) return rc;
            rc = run_matvec_fused(be, wv->fmt, mw + 2, mn + 2, 1, k, src, (float *)be->part_ws + wq->n + wk->n, nullptr, 0);
            if (rc) return rc;
            const int half1 = head_dim / 2;
            const int lanes1 = 256 / half1 > 0 ? 256 / half1 : 1;
            const int max_heads1 = num_q_heads > num_kv_heads ? num_q_heads : num_kv_heads;
            const RowNorm none = {nullptr, 0, 0.f, 0.f};
            const VSrc same = {nullptr, 0, 0};
            if (gen)
                rope_store_general_kernel<true, true><<<dim3(1, ceil_div(max_heads1, lanes1)), lanes1 * half1, 0, be->stream>>>(
                    (const float *)be->part_ws, 1, 1, be->ones, none, q_out, positions, slot_mapping, kv_pool, num_q_heads,
                    num_kv_heads, head_dim, block_size, theta, ex, same);
            else
                rope_store_partials_kernel<true><<<dim3(1, ceil_div(max_heads1, lanes1)), lanes1 * half1, 0, be->stream>>>(
                    (const float *)be->part_ws, 1, 1, be->ones, none, q_out, positions, slot_mapping, kv_pool, num_q_heads,
                    num_kv_heads, head_dim, block_size, theta, same);
            VX_CHECK_LAUNCH();
            return VX_OK;
        }
        if (x && norm_weight && !mixed1 && matvec_ok(wq->fmt, mw, mn, 3, k)) {
            rc = ensure_ws(be, &be->part_ws, &be->part_ws_bytes, (size_t)ntot1 * sizeof(float), "split-K partial sums");
            if (rc) return rc;
            MatvecSource src;
            src.x = x;
            src.norm_w = norm_weight;
            src.eps = eps;
            // With this step's table of angles the launch finishes the row itself: RoPE, Q out, K and V into the pool.
            static const bool no_epi = getenv("VEXEL_HIP_NO_QKV_EPILOGUE") != nullptr;
            const bool table1 = be->rope_tab_pos == positions && be->rope_tab_rows >= 1 && be->rope_tab_dim == head_dim &&
                                be->rope_tab_theta == theta && be->rope_tab_epoch == be->write_epoch;
            if (!gen && !no_epi && table1) {
                src.rope.q_out = q_out;
                src.rope.pool = kv_pool;
                src.rope.slot = slot_mapping;
                src.rope.cs_tab = (const float2 *)be->rope_tab;
                src.rope.qd = wq->n;
                src.rope.kvd = wk->n;
                src.rope.head_dim = head_dim;
                src.rope.block_size = block_size;
                rc = run_matvec_fused(be, wq->fmt, mw, mn, 3, k, src, (float *)be->part_ws, nullptr, 0);
                if (rc == VX_OK) return VX_OK;
                if (rc != VX_ERR_UNSUPPORTED) return rc;
                src.rope = MatvecRope();
            }
            rc = run_matvec_fused(be, wq->fmt, mw, mn, 3, k, src, (float *)be->part_ws, nullptr, 0);
            if (rc) return rc;
            const int half1 = head_dim / 2;
            const int lanes1 = 256 / half1 > 0 ? 256 / half1 : 1;
            const int max_heads1 = num_q_heads > num_kv_heads ? num_q_heads : num_kv_heads;
            const RowNorm none = {nullptr, 0, 0.f, 0.f};
            if (gen)
                rope_store_general_kernel<true, true><<<dim3(1, ceil_div(max_heads1, lanes1)), lanes1 * half1, 0, be->stream>>>(
                    (const float *)be->part_ws, 1, 1, be->ones, none, q_out, positions, slot_mapping, kv_pool, num_q_heads,
                    num_kv_heads, head_dim, block_size, theta, ex, VSrc{nullptr, 0, 0});
            else
                rope_store_partials_kernel<true><<<dim3(1, ceil_div(max_heads1, lanes1)), lanes1 * half1, 0, be->stream>>>(
                    (const float *)be->part_ws, 1, 1, be->ones, none, q_out, positions, slot_mapping, kv_pool, num_q_heads,
                    num_kv_heads, head_dim, block_size, theta, VSrc{nullptr, 0, 0});
            VX_CHECK_LAUNCH();
            return VX_OK;
        }
    }
    if (x_prepared) {
        VX_REQUIRE(be->prep_m == rows && be->prep_k == k, "vx_decode_attn_qkv: no prepared %dx%d activation (have %dx%d)",
                   rows, k, be->prep_m, be->prep_k);
    } else {
        rc = vx_rmsnorm_prepare(be, x, norm_weight, nullptr, rows, k, eps);
        if (rc) return rc;
    }
    const vx_qweight *ws[3] = {wq, wk, wv};
    const bool mixed = wv->fmt != wq->fmt;
    int ntot, ks;
    const Segs segs = make_segs(ws, mixed ? 2 : 3, &ntot);
    VSrc vs = {nullptr, 0, 0};
    // Q and K of one format and V of another, all three with packed copies: one launch leaves the K slices' sums of
    // the three side by side.
    const bool one_mixed = mixed && wk->fmt == wq->fmt && mpad_for(rows) <= 32 &&
                           stream_gemm_mixed_ok(be, wq->fmt, (const uint8_t *)wq->data, (const uint8_t *)wk->data, wq->n, wk->n,
                                                wv->fmt, (const uint8_t *)wv->data, wv->n, k, rows);
    if (mixed && !one_mixed) {
        // V first, into the second partial-sum area (the two change places around its launch), then Q|K as usual
        const vx_qweight *wvs[1] = {wv};
        int nv, ksv;
        const Segs sv = make_segs(wvs, 1, &nv);
        std::swap(be->part_ws, be->part_ws2);
        std::swap(be->part_ws_bytes, be->part_ws2_bytes);
        rc = launch_gemm_fmt(be, wv->fmt, sv, nv, nullptr, nullptr, true, rows, k, &ksv);
        std::swap(be->part_ws, be->part_ws2);
        std::swap(be->part_ws_bytes, be->part_ws2_bytes);
        if (rc) return rc;
        vs = VSrc{(const float *)be->part_ws2, ksv, nv};
    }
    // One K slice, one activation group, the plain RoPE form and a table of this step's angles: the GEMM's workgroups
    // finish their own rows (no partial sums, no second launch).
    if (!mixed && !k_out) {
        const WavePlan pl = wave_plan(be, wq->fmt, segs, ntot, k, rows);
        const bool table = be->rope_tab_pos == positions && be->rope_tab_rows >= rows && be->rope_tab_dim == head_dim &&
                           be->rope_tab_theta == theta && be->rope_tab_epoch == be->write_epoch;
        static const bool no_epi = getenv("VEXEL_HIP_NO_QKV_EPILOGUE") != nullptr;
        const bool one_launch = (pl.r > 0 && pl.ks == 1) || stream_gemm_ok(be, wq->fmt, segs.w, segs.n_end, 3, ntot, k, rows, true);
        if (!no_epi && !gen && table && one_launch && mpad_for(rows) <= 32 && (head_dim & (head_dim - 1)) == 0 &&
            head_dim >= 4 && ((uintptr_t)kv_pool % 16) == 0 && ((uintptr_t)q_out % 16) == 0) {
            QkvEpi epi;
            epi.q_out = q_out;
            epi.pool = kv_pool;
            epi.slots = slot_mapping;
            epi.cs_tab = (const float2 *)be->rope_tab;
            epi.rn = cur_row_norm(be);
            epi.qd = wq->n;
            epi.kvd = wk->n;
            epi.head_dim = head_dim;
            epi.block_size = block_size;
            epi.pool_f16 = pool_is_f16;
            return launch_gemm_fmt(be, wq->fmt, segs, ntot, nullptr, nullptr, false, rows, k, nullptr, &epi);
        }
    }
    const PrepView pv = prep_view(be, mpad_for(rows), k);
    if (one_mixed)
        rc = stream_gemm_mixed(be, wq->fmt, (const uint8_t *)wq->data, (const uint8_t *)wk->data, wq->n, wk->n, wv->fmt,
                               (const uint8_t *)wv->data, wv->n, k, rows, mpad_for(rows), pv, &ks);
    else
        rc = launch_gemm_fmt(be, wq->fmt, segs, ntot, nullptr, nullptr, true, rows, k, &ks);
    if (rc) return rc;
    if (one_mixed) be->last_matmul = "qstream_mixed_kernel";
    const int half = head_dim / 2;
    const int lanes = 256 / half > 0 ? 256 / half : 1;
    if ((lanes * half) % 64 != 0) {  // the row factor is a whole-wave computation
        rc = finalize_row_norm(be);
        if (rc) return rc;
    }
    const RowNorm rn = cur_row_norm(be);
    const int max_heads = num_q_heads > num_kv_heads ? num_q_heads : num_kv_heads;
    // the step's table of angles, where it stands for these positions (vx_rope_table_prepare)
    const bool have_table = be->rope_tab_pos == positions && be->rope_tab_rows >= rows && be->rope_tab_dim == head_dim &&
                            be->rope_tab_theta == theta && be->rope_tab_epoch == be->write_epoch;
    const float2 *cs_tab = have_table ? (const float2 *)be->rope_tab : nullptr;
    dim3 grid(rows, ceil_div(max_heads, lanes));
    if (gen && pool_is_f16)
        rope_store_general_kernel<true, true><<<grid, lanes * half, 0, be->stream>>>(
            (const float *)be->part_ws, ks, rows, pv.inv_scale, rn, q_out, positions, slot_mapping, kv_pool, num_q_heads,
            num_kv_heads, head_dim, block_size, theta, ex, vs, k_out, v_out);
    else if (gen)
        rope_store_general_kernel<false, true><<<grid, lanes * half, 0, be->stream>>>(
            (const float *)be->part_ws, ks, rows, pv.inv_scale, rn, q_out, positions, slot_mapping, kv_pool, num_q_heads,
            num_kv_heads, head_dim, block_size, theta, ex, vs, k_out, v_out);
    else if (pool_is_f16)
        rope_store_partials_kernel<true><<<grid, lanes * half, 0, be->stream>>>(
            (const float *)be->part_ws, ks, rows, pv.inv_scale, rn, q_out, positions, slot_mapping, kv_pool, num_q_heads,
            num_kv_heads, head_dim, block_size, theta, vs, cs_tab, k_out, v_out);
    else
        rope_store_partials_kernel<false><<<grid, lanes * half, 0, be->stream>>>(
            (const float *)be->part_ws, ks, rows, pv.inv_scale, rn, q_out, positions, slot_mapping, kv_pool, num_q_heads,
            num_kv_heads, head_dim, block_size, theta, vs, cs_tab, k_out, v_out);
    VX_CHECK_LAUNCH();
    return VX_OK;
}

int vx_decode_ffn_supported(const vx_qweight *wo, const vx_qweight *w1, const vx_qweight *w3, const vx_qweight *w2) {
    const vx_qweight *a[1] = {wo}, *b[2] = {w1, w3}, *c[1] = {w2};
    if (!group_ok(a, 1) || !group_ok(b, 2) || !group_ok(c, 1)) return 0;
    if (w1->n != w3->n || w2->k != w1->n || w2->n != wo->n || w1->k != wo->n) return 0;
    return (size_t)wo->n * 4 <= 64 * 1024 && (size_t)w1->n * 4 <= 64 * 1024 && wo->n % 256 == 0 && w1->n % 256 == 0;
}

int vx_decode_ffn(vx_backend *be, const float *attn, float *x, const vx_qweight *wo, const float *ffn_norm_weight,
                  float eps, const vx_qweight *w1, const vx_qweight *w3, const vx_qweight *w2, int rows,
                  const float *next_norm_weight) {
    int rc = enter(be);
    if (rc) return rc;
    if (!vx_decode_ffn_supported(wo, w1, w3, w2)) {
        set_error("vx_decode_ffn: weights have no fused MFMA path");
        return VX_ERR_UNSUPPORTED;
    }
    VX_REQUIRE(x && ffn_norm_weight && rows >= 1, "vx_decode_ffn: bad arguments");
    if (!attn) {
        VX_REQUIRE(be->split.batch == rows && be->split.num_q_heads * be->split.head_dim == wo->k,
                   "vx_decode_ffn: attn = NULL but no matching split-form attention result is pending "
                   "(call vx_sdpa_paged_decode_ragged with out = NULL right before)");
        VX_REQUIRE(be->split.head_dim % 4 == 0 && (size_t)wo->k * 4 <= 64 * 1024, "vx_decode_ffn: head geometry");
    }
    VX_REQUIRE(((uintptr_t)x % 16 == 0) && ((uintptr_t)ffn_norm_weight % 16 == 0) && ((uintptr_t)next_norm_weight % 16 == 0),
               "vx_decode_ffn: unaligned pointer");
    const int hidden = wo->n, ffn = w1->n, mpad = mpad_for(rows);
    static const bool no_matvec = getenv("VEXEL_HIP_NO_MATVEC") != nullptr;
    if (rows == 1 && !no_matvec) {
        // A single row: three matrix-vector launches. Wo takes the attention output (merged from the split
        // partials on the fly when attn is NULL) and adds the residual; gate|up take x * ffn_norm / rms(x) and
        // leave SiLU(gate) * up; down adds the residual.
        const void *m1[1] = {wo->data}, *m2[2] = {w1->data, w3->data}, *m3[1] = {w2->data};
        const int n1[1] = {wo->n}, n2[2] = {w1->n, w3->n}, n3[1] = {w2->n};
        const bool merge_ok = attn || (be->split.head_dim % 32 == 0 && be->split.head_dim >= 32);
        if (merge_ok && matvec_ok(wo->fmt, m1, n1, 1, wo->k) && matvec_ok(w1->fmt, m2, n2, 2, hidden) &&
            matvec_ok(w2->fmt, m3, n3, 1, ffn)) {
            rc = ensure_ws(be, &be->part_ws, &be->part_ws_bytes, (size_t)ffn * sizeof(float), "split-K partial sums");
            if (rc) return rc;
            float *h = (float *)be->part_ws;
            MatvecSource s1, s2, s3;
            if (attn) {
                VX_REQUIRE((uintptr_t)attn % 16 == 0, "vx_decode_ffn: unaligned pointer");
                s1.x = attn;
            } else if (be->split.plain) {
                s1.x = be->split.plain;
                be->split.batch = 0;
            } else {
                s1.attn_partial = (const float *)be->attn_ws;
                s1.kv_len = be->split.kv_lens;
                s1.head_dim = be->split.head_dim;
                s1.max_splits = be->split.max_splits;
                s1.tokens_per_split = be->split.tokens_per_split;
                be->split.batch = 0;
            }
            rc = run_matvec_fused(be, wo->fmt, m1, n1, 1, wo->k, s1, x, x, 0);
            if (rc) return rc;
            s2.x = x;
            s2.norm_w = ffn_norm_weight;
            s2.eps = eps;
            rc = run_matvec_fused(be, w1->fmt, m2, n2, 2, hidden, s2, h, nullptr, 1);
            if (rc) return rc;
            s3.x = h;
            rc = run_matvec_fused(be, w2->fmt, m3, n3, 1, ffn, s3, x, x, 0);
            if (rc) return rc;
            be->prep_m = 0;
            be->prep_k = 0;
            if (next_norm_weight) return vx_rmsnorm_prepare(be, x, next_norm_weight, nullptr, 1, hidden, eps);
            return VX_OK;
        }
    }
    int ks, ntot;
    // (the attention kernel may already have left the merged result in the prepared form: only where the workspace
    // still is where that kernel wrote it)
    const void *ws_before = be->gemm_ws;
    const size_t ws_bytes_before = be->gemm_ws_bytes;
    rc = prep_reserve(be, rows, ffn > wo->k ? (ffn > hidden ? ffn : hidden) : (wo->k > hidden ? wo->k : hidden));
    if (rc) return rc;
    const bool merged = !attn && be->split.merged && be->gemm_ws == ws_before && be->gemm_ws_bytes == ws_bytes_before &&
                        be->prep_m == rows && be->prep_k == wo->k;
    be->split.merged = 0;
    // attention output -> Wo -> partials
    if (attn) {
        rc = vx_prepare_act(be, attn, rows, wo->k);
        if (rc) return rc;
    } else if (merged) {
        be->split.batch = 0;
    } else {
        PrepView pa;
        rc = prep_begin(be, rows, wo->k, &pa);
        if (rc) return rc;
        if (chunk_prepare_ok(rows, wo->k))
            chunk_merge_kernel<<<dim3(wo->k / 256, mpad), 64, 0, be->stream>>>(
                (const float *)be->attn_ws, be->split.kv_lens, rows, wo->k, be->split.head_dim, be->split.max_splits,
                be->split.tokens_per_split, pa, mpad);
        else
            merge_prepare_kernel<<<mpad, PREP_THREADS, (size_t)wo->k * 4, be->stream>>>(
                (const float *)be->attn_ws, be->split.kv_lens, rows, wo->k, be->split.head_dim, be->split.max_splits,
                be->split.tokens_per_split, pa, mpad);
        VX_CHECK_LAUNCH();
        be->split.batch = 0;
    }
    const vx_qweight *a[1] = {wo};
    Segs segs = make_segs(a, 1, &ntot);
    rc = launch_gemm_fmt(be, wo->fmt, segs, ntot, nullptr, nullptr, true, rows, wo->k, &ks);
    if (rc) return rc;
    // x += Wo(attn); prepared <- RMSNorm(x) * ffn_norm
    PrepView pv;
    const float *inv_in = prep_view(be, mpad, wo->k).inv_scale;  // row factors of the activation that produced the partials
    RowNorm rn_in = cur_row_norm(be);                            // (none pending here: the attention output)
    rc = prep_begin(be, rows, hidden, &pv);
    if (rc) return rc;
    const bool chunked = chunk_prepare_ok(rows, hidden) && chunk_prepare_ok(rows, ffn);
    if (chunked) {
        chunk_add_norm_kernel<<<dim3(hidden / 256, mpad), 64, 0, be->stream>>>(
            x, (const float *)be->part_ws, ks, rows, hidden, ffn_norm_weight, eps, pv, mpad, inv_in, rn_in, cur_ss_out(be));
        be->prep_norm_k = hidden;
        be->prep_norm_eps = eps;
    } else
        fused_prepare_kernel<FUSE_ADD_RMSNORM><<<mpad, FP_THREADS, (size_t)hidden * 4, be->stream>>>(
            x, (const float *)be->part_ws, ks, rows, hidden, ffn_norm_weight, eps, pv, mpad, inv_in);
    VX_CHECK_LAUNCH();
    // gate | up -> partials
    const vx_qweight *b[2] = {w1, w3};
    segs = make_segs(b, 2, &ntot);
    rc = launch_gemm_fmt(be, w1->fmt, segs, ntot, nullptr, nullptr, true, rows, hidden, &ks);
    if (rc) return rc;
    // prepared <- SiLU(gate) * up
    inv_in = pv.inv_scale;
    rn_in = cur_row_norm(be);
    rc = prep_begin(be, rows, ffn, &pv);
    if (rc) return rc;
    // (a wave per row and 256-column chunk also for big prompt chunks: SiLU * up needs nothing that spans the row, and
    // beyond 256 rows the many small workgroups overlap their exponentials with the loads better than one workgroup
    // per row does - 8B shape, 512 rows: 1 % of the chunk's time; at 256 rows the two forms take the same time)
    if (chunked || (rows > 256 && ffn % 256 == 0))
        chunk_silu_kernel<<<dim3(ffn / 256, mpad), 64, 0, be->stream>>>((const float *)be->part_ws, ks, rows, ffn, pv, mpad,
                                                                        inv_in, rn_in);
    else
        fused_prepare_kernel<FUSE_SILU_MUL><<<mpad, FP_THREADS, (size_t)ffn * 4, be->stream>>>(
            nullptr, (const float *)be->part_ws, ks, rows, ffn, nullptr, 0.f, pv, mpad, inv_in);
    VX_CHECK_LAUNCH();
    // down -> partials
    const vx_qweight *c[1] = {w2};
    segs = make_segs(c, 1, &ntot);
    rc = launch_gemm_fmt(be, w2->fmt, segs, ntot, nullptr, nullptr, true, rows, ffn, &ks);
    if (rc) return rc;
    if (next_norm_weight) {
        inv_in = pv.inv_scale;
        rn_in = cur_row_norm(be);
        rc = prep_begin(be, rows, hidden, &pv);
        if (rc) return rc;
        if (chunked) {
            chunk_add_norm_kernel<<<dim3(hidden / 256, mpad), 64, 0, be->stream>>>(
                x, (const float *)be->part_ws, ks, rows, hidden, next_norm_weight, eps, pv, mpad, inv_in, rn_in,
                cur_ss_out(be));
            be->prep_norm_k = hidden;
            be->prep_norm_eps = eps;
        } else
            fused_prepare_kernel<FUSE_ADD_RMSNORM><<<mpad, FP_THREADS, (size_t)hidden * 4, be->stream>>>(
                x, (const float *)be->part_ws, ks, rows, hidden, next_norm_weight, eps, pv, mpad, inv_in);
        VX_CHECK_LAUNCH();
    } else {
        const size_t total4 = (size_t)rows * hidden / 4;
        add_partials_kernel<<<(unsigned)((total4 + 255) / 256), 256, 0, be->stream>>>(x, (const float *)be->part_ws, ks,
                                                                                     rows, hidden, pv.inv_scale);
        VX_CHECK_LAUNCH();
        be->prep_m = 0;  // the slot no longer matches any activation the caller knows about
        be->prep_k = 0;
    }
    return VX_OK;
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

int vx_matmul_q5_k(vx_backend *be, const float *a, const void *b, float *out, int m, int n, int k) {
    return vx_matmul_quant(be, VX_Q5_K, a, b, out, nullptr, m, n, k);
}
int vx_matmul_q5_0(vx_backend *be, const float *a, const void *b, float *out, int m, int n, int k) {
    return vx_matmul_quant(be, VX_Q5_0, a, b, out, nullptr, m, n, k);
}
int vx_matmul_bf16(vx_backend *be, const float *a, const void *b, float *out, int m, int n, int k) {
    return vx_matmul_quant(be, VX_BF16, a, b, out, nullptr, m, n, k);
}

}  // extern "C"
