// Quantized matrix-vector product for a single activation row (M = 1, the reference's decode call:
// inference/runtime/block.go:512-517 -> QuantizedMatMul with m = 1):   out[n] = sum_k a[k] * W[n][k]  (+ residual[n])
// W holds raw GGUF blocks (inference/pkg/gguf/dequant.go). HBM bound: every weight byte is read once with 16-byte
// loads, the arithmetic is plain float32 on the vector ALU (no matrix cores at M = 1).
//
// Shape of the work. grid = ceil(N / RG) workgroups of 256 threads; a workgroup owns RG consecutive weight rows.
//   * K is cut in four segments of whole "units" (a 32-element block for Q4_0 / Q8_0, a 256-element super-block for
//     Q4_K / Q6_K); wave w takes segment w of every row of the group.
//   * A wave's 64 lanes are 2 row lanes x 32 block lanes: lane l works on 32-element blocks (l % 32) + 32 t,
//     t < T <= 4, of rows (l / 32), (l / 32) + 2, ... The 32 activations of each of its blocks (and their sums) sit in
//     registers for the whole kernel, read once from global memory.
//   * Staging: the wave copies its segment of the RG rows to LDS with aligned 16-byte loads, all issued before the
//     first is waited for. A segment may start at any even byte of a row (Q4_0: 18-byte blocks, Q6_K: 210-byte
//     super-blocks, row lengths that are not multiples of 16): the copy starts at the 16-byte boundary below it and
//     the decoders add the offset. The matrix is 16-byte aligned and a multiple of 16 bytes long, so no aligned
//     piece leaves it.
//   * A lane turns the 32 codes of a block into floats with byte-to-float conversions and accumulates
//     sum a*code; the codes' offset (8, 128, 32) and the block scale are applied to the block sum:
//     d * (sum a*q - off * sum a). The 32 block lanes are added by DPP inside 16-lane rows plus one cross-row
//     exchange, the four waves through LDS, in a fixed order.
#include "common.h"

using namespace vx;

namespace {

constexpr int MV_THREADS = 256;
constexpr int MV_WAVES = 4;
constexpr int MV_MAX_T = 4;           // 32-element blocks per lane and row: K <= 4 * 4 * 32 * 32 = 16384
constexpr int MV_WAVE_LDS = 8 * 1024; // staging bytes per wave
constexpr int MV_MAX_RG = 8;

__device__ __forceinline__ float h2f(uint16_t h) {
    _Float16 v;
    __builtin_memcpy(&v, &h, 2);
    return (float)v;
}

// 4 bytes at byte offset `off` (any alignment) of a 4-byte aligned LDS array
__device__ __forceinline__ uint32_t lds_u32(const uint8_t *base, int off) {
    const uint32_t *w = (const uint32_t *)base;
    const int i = off >> 2;
    return __builtin_amdgcn_alignbyte(w[i + 1], w[i], (uint32_t)(off & 3));
}
__device__ __forceinline__ uint32_t lds_u16(const uint8_t *base, int off) { return *(const uint16_t *)(base + off); }

// sum_b x[b] * byte_b(w), b = 0..3
__device__ __forceinline__ float dot4(float acc, uint32_t w, const float *x) {
    acc = fmaf(x[0], (float)(uint8_t)w, acc);  // v_cvt_f32_ubyte0..3: one instruction per code
    acc = fmaf(x[1], (float)(uint8_t)(w >> 8), acc);
    acc = fmaf(x[2], (float)(uint8_t)(w >> 16), acc);
    acc = fmaf(x[3], (float)(uint8_t)(w >> 24), acc);
    return acc;
}

// Sum over the 32 block lanes of a half wave; every lane of the half gets the total.
__device__ __forceinline__ float half_wave_sum(float t) {
    t += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, t), 0xb1, 0xf, 0xf, false));   // quad_perm [1,0,3,2]
    t += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, t), 0x4e, 0xf, 0xf, false));   // quad_perm [2,3,0,1]
    t += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, t), 0x141, 0xf, 0xf, false));  // row_half_mirror
    t += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, t), 0x140, 0xf, 0xf, false));  // row_mirror
    t += __shfl_xor(t, 16, 64);
    return t;
}

// ---- per-format decoders: contribution of 32-element block `jl` of the staged segment `seg` (LDS byte offset of the
// segment's first byte inside `base`), given the block's activations x[32] and their sums over elements 0-15 / 16-31.
struct VQ4_0 {  // dequant.go:16-56: [f16 d][16 bytes], element i = low nibble of byte i, i+16 = high nibble, (q-8)*d
    static constexpr int UNIT_BLOCKS = 1, UNIT_BYTES = 18;
    static __device__ __forceinline__ float block(const uint8_t *base, int seg, int jl, const float *x, float s0, float s1) {
        const int o = seg + jl * 18;
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t w = lds_u32(base, o + 2 + 4 * i);
            acc = dot4(acc, w & 0x0F0F0F0Fu, x + 4 * i);
            acc = dot4(acc, (w >> 4) & 0x0F0F0F0Fu, x + 16 + 4 * i);
        }
        return h2f((uint16_t)lds_u16(base, o)) * (acc - 8.f * (s0 + s1));
    }
};

struct VQ8_0 {  // dequant.go:62-90: [f16 d][32 x int8], d*q
    static constexpr int UNIT_BLOCKS = 1, UNIT_BYTES = 34;
    static __device__ __forceinline__ float block(const uint8_t *base, int seg, int jl, const float *x, float s0, float s1) {
        const int o = seg + jl * 34;
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) acc = dot4(acc, lds_u32(base, o + 2 + 4 * i) ^ 0x80808080u, x + 4 * i);  // q + 128
        return h2f((uint16_t)lds_u16(base, o)) * (acc - 128.f * (s0 + s1));
    }
};

struct VQ4_K {  // dequant.go:342-409: 144-byte super-block, 8 sub-blocks of 32: d*sc*q - dmin*m
    static constexpr int UNIT_BLOCKS = 8, UNIT_BYTES = 144;
    static __device__ __forceinline__ float block(const uint8_t *base, int seg, int jl, const float *x, float s0, float s1) {
        const int j = jl & 7;
        const int sb = seg + (jl >> 3) * 144;  // 16-byte aligned: rows and segments are whole super-blocks
        const uint32_t *S = (const uint32_t *)(base + sb);
        const uint32_t *qp = S + 4 + 8 * (j >> 1);
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) acc = dot4(acc, (qp[i] >> (4 * (j & 1))) & 0x0F0F0F0Fu, x + 4 * i);
        const uint8_t *q = base + sb + 4;
        uint32_t sc, mn;  // getScaleMinK4, dequant.go:400-409
        if (j < 4) {
            sc = q[j] & 63;
            mn = q[j + 4] & 63;
        } else {
            sc = (q[j + 4] & 0x0F) | ((q[j - 4] >> 6) << 4);
            mn = (q[j + 4] >> 4) | ((q[j] >> 6) << 4);
        }
        const uint32_t hd = S[0];
        return h2f((uint16_t)(hd & 0xFFFF)) * (float)sc * acc - h2f((uint16_t)(hd >> 16)) * (float)mn * (s0 + s1);
    }
};

struct VQ6_K {  // dequant.go:272-331: 210-byte super-block [ql 128][qh 64][int8 sc 16][f16 d]
    static constexpr int UNIT_BLOCKS = 8, UNIT_BYTES = 210;
    static __device__ __forceinline__ float block(const uint8_t *base, int seg, int jl, const float *x, float s0, float s1) {
        const int j = jl & 7, n = j >> 2, qt = j & 3;  // half n, quarter qt: elements 128n + 32qt + (0..31)
        const int S = seg + (jl >> 3) * 210;
        const int ql = S + 64 * n + 32 * (qt & 1), qh = S + 128 + 32 * n;
        float a0 = 0.f, a1 = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const uint32_t lo = (lds_u32(base, ql + 4 * i) >> (4 * (qt >> 1))) & 0x0F0F0F0Fu;
            const uint32_t hi = (lds_u32(base, qh + 4 * i) >> (2 * qt)) & 0x03030303u;
            const uint32_t q = lo | (hi << 4);  // 6-bit code, value q - 32
            if (i < 4) a0 = dot4(a0, q, x + 4 * i);
            else a1 = dot4(a1, q, x + 4 * i);
        }
        const uint32_t sc = lds_u16(base, S + 192 + 8 * n + 2 * qt);  // scales of elements 0-15 and 16-31
        const float sa = (float)(int8_t)(sc & 0xFF), sb = (float)(int8_t)(sc >> 8);
        const float d = h2f((uint16_t)lds_u16(base, S + 208));
        return d * (sa * (a0 - 32.f * s0) + sb * (a1 - 32.f * s1));
    }
};

template <class F, int T>
__global__ void __launch_bounds__(MV_THREADS) qmatvec_kernel(const uint8_t *__restrict__ W, const float *__restrict__ a,
                                                             float *__restrict__ out, const float *__restrict__ residual,
                                                             int N, int K, size_t row_bytes, int lp, int units_per_wave) {
    __shared__ __attribute__((aligned(16))) uint8_t stage[MV_WAVES][MV_WAVE_LDS];
    __shared__ float part[MV_WAVES][MV_MAX_RG];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int bl = lane & 31, rp = lane >> 5;
    const int n_units = K / (32 * F::UNIT_BLOCKS);
    const int u0 = min(wave * units_per_wave, n_units), u1 = min(u0 + units_per_wave, n_units);
    const int seg_blocks = (u1 - u0) * F::UNIT_BLOCKS;
    const int passes = 1 << lp, rg = MV_MAX_RG >> lp;  // 64-piece passes per staged row; rows per group
    const int row0 = blockIdx.x * rg;

    // the lane's activations (one global read each for the whole kernel)
    float x[T][32], s0[T], s1[T];
#pragma unroll
    for (int t = 0; t < T; t++) {
        const int jl = bl + 32 * t;
        // every load is unconditional (a lane without a block re-reads the vector's start): loads under a branch
        // would be waited for one by one
        const float *ap = a + (jl < seg_blocks ? (size_t)(u0 * F::UNIT_BLOCKS + jl) * 32 : 0);
        s0[t] = s1[t] = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const float4 v = *(const float4 *)(ap + 4 * i);
            x[t][4 * i] = v.x; x[t][4 * i + 1] = v.y; x[t][4 * i + 2] = v.z; x[t][4 * i + 3] = v.w;
        }
#pragma unroll
        for (int i = 0; i < 16; i++) {
            s0[t] += x[t][i];
            s1[t] += x[t][16 + i];
        }
    }

    // stage the wave's segment of the group's rows: 16-byte pieces from the aligned address at or below the segment
    const size_t seg_off = (size_t)u0 * F::UNIT_BYTES;
    const int seg_bytes = (u1 - u0) * F::UNIT_BYTES;
    uint8_t *my = &stage[wave][0];
    // Row r of the group: pieces from (row start + seg_off) & ~15; its first segment byte lands at byte sh_r of its
    // LDS row. Rows have different sh_r when row_bytes is not a multiple of 16.
    const int rstride = (seg_bytes + 15 + 16 + 15) & ~15;  // room for the leading offset and the trailing over-read
    const int ppr = rstride / 16;                            // pieces per row (<= 64 * passes)
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    constexpr int NP = MV_MAX_RG;  // load slots per lane: slot i = (row i >> lp, pass i & (passes - 1))
    u32x4 pc[NP];
#pragma unroll
    for (int i = 0; i < NP; i++) {
        const int r = i >> lp, c = min(((i & (passes - 1)) << 6) + lane, ppr - 1);
        const int row = min(row0 + r, N - 1);
        const size_t start = row_bytes * (size_t)row + seg_off;
        const size_t first = start & ~(size_t)15;
        // pieces past the segment's end (the slack of rstride) are clamped to its last piece: never outside the matrix
        const size_t last = (start + (size_t)max(seg_bytes, 1) - 1) & ~(size_t)15;
        const size_t addr = seg_bytes > 0 ? min(first + (size_t)c * 16, last) : 0;  // an empty segment reads the matrix start
        pc[i] = *(const u32x4 *)(W + addr);
    }
#pragma unroll
    for (int i = 0; i < NP; i++) {
        const int r = i >> lp, c = ((i & (passes - 1)) << 6) + lane;
        if (c < ppr) *(u32x4 *)(my + (size_t)r * rstride + (size_t)c * 16) = pc[i];
    }
    // the wave reads only what it wrote: its own LDS operations are ordered, no barrier needed here

    for (int r = rp; r < rg; r += 2) {
        const int row = min(row0 + r, N - 1);
        const int sh = (int)((row_bytes * (size_t)row + seg_off) & 15);
        float acc = 0.f;
#pragma unroll
        for (int t = 0; t < T; t++) {
            const int jl = bl + 32 * t;
            if (jl < seg_blocks) acc += F::block(my, r * rstride + sh, jl, x[t], s0[t], s1[t]);
        }
        acc = half_wave_sum(acc);
        if (bl == 0) part[wave][r] = acc;
    }
    __syncthreads();
    if (tid < rg && row0 + tid < N) {
        float v = (part[0][tid] + part[1][tid]) + (part[2][tid] + part[3][tid]);
        if (residual) v = __fadd_rn(residual[row0 + tid], v);
        out[row0 + tid] = v;
    }
}

template <class F>
int launch(vx_backend *be, const uint8_t *W, const float *a, float *out, const float *residual, int n, int k) {
    const int n_units = k / (32 * F::UNIT_BLOCKS);
    const int upw = ceil_div(n_units, MV_WAVES);
    const int seg_blocks = upw * F::UNIT_BLOCKS;
    const int T = ceil_div(seg_blocks, 32);
    if (T > MV_MAX_T) return VX_ERR_UNSUPPORTED;
    const int rstride = (upw * F::UNIT_BYTES + 15 + 16 + 15) & ~15;
    // a staged row takes 1, 2 or 4 passes of 64 pieces; the group has 8, 4 or 2 rows, so that a lane always has 8 loads
    int lp = 0;
    while ((64 << lp) < rstride / 16) lp++;
    if (lp > 2 || (MV_MAX_RG >> lp) * rstride > MV_WAVE_LDS) return VX_ERR_UNSUPPORTED;
    const int rg = MV_MAX_RG >> lp;
    const size_t rb = (size_t)n_units * F::UNIT_BYTES;
    const dim3 grid(ceil_div(n, rg));
#define VX_MV(TT)                                                                                                    \
    case TT:                                                                                                         \
        qmatvec_kernel<F, TT><<<grid, MV_THREADS, 0, be->stream>>>(W, a, out, residual, n, k, rb, lp, upw);             \
        break;
    switch (T) {
        VX_MV(1) VX_MV(2) VX_MV(3) VX_MV(4)
    }
#undef VX_MV
    VX_CHECK_LAUNCH();
    return VX_OK;
}

}  // namespace

namespace vx {

// out[n] = a . W[n] (+ residual[n]) for one activation row. VX_ERR_UNSUPPORTED (nothing launched) when the shape is
// outside the kernel's range: the caller then takes another path.
int run_matvec(vx_backend *be, int fmt, const float *a, const void *b, float *out, const float *residual, int n, int k) {
    if (((uintptr_t)b % 16) != 0 || ((uintptr_t)a % 16) != 0 || n < 1) return VX_ERR_UNSUPPORTED;
    const uint8_t *W = (const uint8_t *)b;
    switch (fmt) {
    case VX_Q4_0:
        if (k % 32 != 0 || ((size_t)n * (k / 32) * 18) % 16 != 0) return VX_ERR_UNSUPPORTED;
        return launch<VQ4_0>(be, W, a, out, residual, n, k);
    case VX_Q8_0:
        if (k % 32 != 0 || ((size_t)n * (k / 32) * 34) % 16 != 0) return VX_ERR_UNSUPPORTED;
        return launch<VQ8_0>(be, W, a, out, residual, n, k);
    case VX_Q4_K:
        if (k % 256 != 0) return VX_ERR_UNSUPPORTED;
        return launch<VQ4_K>(be, W, a, out, residual, n, k);
    case VX_Q6_K:
        if (k % 256 != 0 || ((size_t)n * (k / 256) * 210) % 16 != 0) return VX_ERR_UNSUPPORTED;
        return launch<VQ6_K>(be, W, a, out, residual, n, k);
    }
    return VX_ERR_UNSUPPORTED;
}

}  // namespace vx
