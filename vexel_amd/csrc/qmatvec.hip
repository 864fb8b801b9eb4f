// Quantized matrix-vector product for a single activation row (M = 1, the reference's decode call:
// inference/runtime/block.go:512-517 -> QuantizedMatMul with m = 1):   out[n] = sum_k a[k] * W[n][k]  (+ residual[n])
// W holds raw GGUF blocks (inference/pkg/gguf/dequant.go). HBM bound: every weight byte is read once with 16-byte
// loads, the arithmetic is plain float32 on the vector ALU (no matrix cores at M = 1).
//
// Shape of the work. Workgroups of 256 threads; a workgroup takes groups of RG consecutive weight rows, one group
// per trip of its loop, and loads the next group's weights while it computes the current one.
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
#include <algorithm>

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

// ---- per-format decoders. X holds what a lane keeps of one 32-element block of the activation row (set once by
// prep from the block's 32 floats); block() is the contribution of block `jl` of the staged segment `seg` (LDS
// byte offset of the segment's first byte inside `base`).
//
// The arithmetic is integer: 4-byte dot products (v_dot4) of the weight codes, which ARE bytes or nibbles, with
// the activations as fixed-point integers. A block's activations are scaled by the power of two that puts the
// largest magnitude in [2^(BITS-2), 2^(BITS-1)) and rounded to integers xi (an error of at most 2^-(BITS-1) of
// the block's largest activation per element). Plane p holds byte p of the two's-complement xi of the 32
// elements, four to a dword in element order: xi = b0 + 256 b1 + 65536 b2 with b0, b1 unsigned and b2 signed,
// so sum(code * xi) = S0 + 256 S1 + 65536 S2 with Sp = sum(code * bp), exact in int32 for the BITS each format
// picks. The block's scale and the inverse power of two are applied to the float of that integer.
template <int BITS>
struct XInt {
    uint32_t p[3][8];  // plane, dword j = elements 4j .. 4j+3
    int s0, s1;        // sum of xi over elements 0-15 / 16-31
    float inv;         // activation = xi * inv
    __device__ __forceinline__ void prep(const float *v) {
        float m = 0.f;
#pragma unroll
        for (int i = 0; i < 32; i++) m = fmaxf(m, fabsf(v[i]));
        // scale = 2^(BITS - 2 - exponent(m)); zero, denormal-range and non-finite maxima take 1 (such rows give
        // zeros or garbage either way: the float path would too)
        const int ex = (int)((__float_as_uint(m) >> 23) & 0xFF);
        const bool usable = ex > BITS && ex < 255;
        const float scale = usable ? __uint_as_float((uint32_t)(127 + BITS - 2 + 127 - ex) << 23) : 1.f;
        inv = usable ? __uint_as_float((uint32_t)(ex - (BITS - 2)) << 23) : 1.f;
        s0 = s1 = 0;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            uint32_t xi[4];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                // adding 1.5 * 2^23 rounds v * scale (|.| < 2^22) to an integer, to nearest even, in the low
                // mantissa bits: the float's bits are 0x4B400000 + xi
                const uint32_t bits = __float_as_uint(fmaf(v[4 * j + k], scale, 12582912.f));
                xi[k] = bits - 0x4B400000u;
                if (j < 4) s0 += (int)xi[k];
                else s1 += (int)xi[k];
            }
            // v_perm_b32(hi, lo, sel): selector bytes 0-3 pick from lo, 4-7 from hi
            const uint32_t a01 = __builtin_amdgcn_perm(xi[1], xi[0], 0x05010400u);  // x0.b0 x1.b0 x0.b1 x1.b1
            const uint32_t a23 = __builtin_amdgcn_perm(xi[3], xi[2], 0x05010400u);
            const uint32_t c01 = __builtin_amdgcn_perm(xi[1], xi[0], 0x0c0c0602u);  // x0.b2 x1.b2 0 0
            const uint32_t c23 = __builtin_amdgcn_perm(xi[3], xi[2], 0x0c0c0602u);
            p[0][j] = __builtin_amdgcn_perm(a23, a01, 0x05040100u);
            p[1][j] = __builtin_amdgcn_perm(a23, a01, 0x07060302u);
            p[2][j] = __builtin_amdgcn_perm(c23, c01, 0x05040100u);
        }
    }
    // acc[p] += sum over the 4 unsigned code bytes of c times byte p of elements 4j .. 4j+3 (codes below 128)
    __device__ __forceinline__ void dot(int (&acc)[3], uint32_t c, int j) const {
        acc[0] = (int)__builtin_amdgcn_udot4(c, p[0][j], (uint32_t)acc[0], false);
        acc[1] = (int)__builtin_amdgcn_udot4(c, p[1][j], (uint32_t)acc[1], false);
        acc[2] = __builtin_amdgcn_sdot4((int)c, (int)p[2][j], acc[2], false);
    }
    // sum of the bytes of plane pl over all 32 elements
    __device__ __forceinline__ int plane_sum(int pl) const {
        uint32_t t = 0;
#pragma unroll
        for (int j = 0; j < 8; j++) t = __builtin_amdgcn_udot4(0x01010101u, p[pl][j], t, false);
        return (int)t;
    }
};

// N consecutive dwords starting at byte offset `off` (any alignment) of a 4-byte aligned LDS array: N + 1
// aligned reads at constant offsets from one address, then one byte alignment each.
template <int N>
__device__ __forceinline__ void lds_dwords(const uint8_t *base, int off, uint32_t (&w)[N]) {
    const uint32_t *p = (const uint32_t *)base + (off >> 2);
    const uint32_t sh = (uint32_t)(off & 3);
    uint32_t raw[N + 1];
#pragma unroll
    for (int i = 0; i <= N; i++) raw[i] = p[i];
#pragma unroll
    for (int i = 0; i < N; i++) w[i] = __builtin_amdgcn_alignbyte(raw[i + 1], raw[i], sh);
}

struct VQ4_0 {  // dequant.go:16-56: [f16 d][16 bytes], element i = low nibble of byte i, i+16 = high nibble, (q-8)*d
    static constexpr int UNIT_BLOCKS = 1, UNIT_BYTES = 18;
    typedef XInt<23> X;  // |xi| < 2^22: |sum q xi| <= 15 * 2^22 * 32 < 2^31
    static __device__ __forceinline__ float block(const uint8_t *base, int seg, int jl, const X &x) {
        const int o = seg + jl * 18;
        uint32_t w[4];
        lds_dwords<4>(base, o + 2, w);
        int acc[3] = {0, 0, 0};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            x.dot(acc, w[i] & 0x0F0F0F0Fu, i);
            x.dot(acc, (w[i] >> 4) & 0x0F0F0F0Fu, 4 + i);
        }
        const int t = acc[0] + (acc[1] << 8) + (acc[2] << 16) - 8 * (x.s0 + x.s1);  // sum (q - 8) xi, exact
        return h2f((uint16_t)lds_u16(base, o)) * ((float)t * x.inv);
    }
};

struct VQ8_0 {  // dequant.go:62-90: [f16 d][32 x int8], d*q
    static constexpr int UNIT_BLOCKS = 1, UNIT_BYTES = 34;
    struct X : XInt<23> {
        int b0, b1;  // byte sums of planes 0 and 1
        __device__ __forceinline__ void prep(const float *v) {
            XInt<23>::prep(v);
            b0 = plane_sum(0);
            b1 = plane_sum(1);
        }
    };
    static __device__ __forceinline__ float block(const uint8_t *base, int seg, int jl, const X &x) {
        const int o = seg + jl * 34;
        uint32_t w[8];
        lds_dwords<8>(base, o + 2, w);
        // the unsigned planes take the codes as q + 128 (unsigned), corrected by 128 * the plane's byte sum;
        // the signed top plane takes them as they are
        uint32_t u0 = 0, u1 = 0;
        int s2 = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const uint32_t c = w[i] ^ 0x80808080u;
            u0 = __builtin_amdgcn_udot4(c, x.p[0][i], u0, false);
            u1 = __builtin_amdgcn_udot4(c, x.p[1][i], u1, false);
            s2 = __builtin_amdgcn_sdot4((int)w[i], (int)x.p[2][i], s2, false);
        }
        // |S2| can reach 2^18, so the top plane joins in float32 (|S0 + 256 S1| < 2^31 stays exact)
        const int low = ((int)u0 - 128 * x.b0) + (((int)u1 - 128 * x.b1) << 8);
        const float t = (float)s2 * 65536.f + (float)low;
        return h2f((uint16_t)lds_u16(base, o)) * (t * x.inv);
    }
};

struct VQ4_K {  // dequant.go:342-409: 144-byte super-block, 8 sub-blocks of 32: d*sc*q - dmin*m
    static constexpr int UNIT_BLOCKS = 8, UNIT_BYTES = 144;
    typedef XInt<23> X;
    static __device__ __forceinline__ float block(const uint8_t *base, int seg, int jl, const X &x) {
        const int j = jl & 7;
        const int sb = seg + (jl >> 3) * 144;  // 16-byte aligned: rows and segments are whole super-blocks
        const uint32_t *S = (const uint32_t *)(base + sb);
        const uint32_t *qp = S + 4 + 8 * (j >> 1);
        int acc[3] = {0, 0, 0};
#pragma unroll
        for (int i = 0; i < 8; i++) x.dot(acc, (qp[i] >> (4 * (j & 1))) & 0x0F0F0F0Fu, i);
        const int t = acc[0] + (acc[1] << 8) + (acc[2] << 16);
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
        return (h2f((uint16_t)(hd & 0xFFFF)) * (float)sc * (float)t - h2f((uint16_t)(hd >> 16)) * (float)mn * (float)(x.s0 + x.s1)) * x.inv;
    }
};

struct VQ6_K {  // dequant.go:272-331: 210-byte super-block [ql 128][qh 64][int8 sc 16][f16 d]
    static constexpr int UNIT_BLOCKS = 8, UNIT_BYTES = 210;
    typedef XInt<22> X;  // |xi| < 2^21; per 16 elements: |sum q6 xi| <= 63 * 2^21 * 16 < 2^31
    static __device__ __forceinline__ float block(const uint8_t *base, int seg, int jl, const X &x) {
        const int j = jl & 7, n = j >> 2, qt = j & 3;  // half n, quarter qt: elements 128n + 32qt + (0..31)
        const int S = seg + (jl >> 3) * 210;
        const int ql = S + 64 * n + 32 * (qt & 1), qh = S + 128 + 32 * n;
        uint32_t wl[8], wh[8];
        lds_dwords<8>(base, ql, wl);
        lds_dwords<8>(base, qh, wh);
        int a[3] = {0, 0, 0}, b[3] = {0, 0, 0};
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const uint32_t lo = (wl[i] >> (4 * (qt >> 1))) & 0x0F0F0F0Fu;
            const uint32_t hi = (wh[i] >> (2 * qt)) & 0x03030303u;
            const uint32_t q = lo | (hi << 4);  // 6-bit codes, value q - 32
            if (i < 4) x.dot(a, q, i);
            else x.dot(b, q, i);
        }
        const int ta = a[0] + (a[1] << 8) + (a[2] << 16) - 32 * x.s0;  // elements 0-15
        const int tb = b[0] + (b[1] << 8) + (b[2] << 16) - 32 * x.s1;
        const uint32_t sc = lds_u16(base, S + 192 + 8 * n + 2 * qt);  // scales of elements 0-15 and 16-31
        const float sa = (float)(int8_t)(sc & 0xFF), sb = (float)(int8_t)(sc >> 8);
        const float d = h2f((uint16_t)lds_u16(base, S + 208));
        return d * ((sa * (float)ta + sb * (float)tb) * x.inv);
    }
};

// the 4 low bits of b, one each into bit 4 of the 4 bytes of a dword (bit i -> byte i)
__device__ __forceinline__ uint32_t fifth_bits(uint32_t b) { return ((b * 0x00204081u) & 0x01010101u) << 4; }

struct VQ5_0 {  // dequant.go:100-145: [f16 d][u32 qh][16 bytes], element i = nibble as Q4_0 | bit i of qh << 4, (q-16)*d
    static constexpr int UNIT_BLOCKS = 1, UNIT_BYTES = 22;
    typedef XInt<22> X;  // |xi| < 2^21: |sum q xi| <= 31 * 2^21 * 32 < 2^31
    static __device__ __forceinline__ float block(const uint8_t *base, int seg, int jl, const X &x) {
        const int o = seg + jl * 22;
        uint32_t w[5];
        lds_dwords<5>(base, o + 2, w);
        const uint32_t qh = w[0];
        int acc[3] = {0, 0, 0};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            x.dot(acc, (w[1 + i] & 0x0F0F0F0Fu) | fifth_bits((qh >> (4 * i)) & 15u), i);
            x.dot(acc, ((w[1 + i] >> 4) & 0x0F0F0F0Fu) | fifth_bits((qh >> (16 + 4 * i)) & 15u), 4 + i);
        }
        const int t = acc[0] + (acc[1] << 8) + (acc[2] << 16) - 16 * (x.s0 + x.s1);  // sum (q - 16) xi, exact
        return h2f((uint16_t)lds_u16(base, o)) * ((float)t * x.inv);
    }
};

struct VQ5_K {  // dequant.go:423-500: 176-byte super-block [d][dmin][12 scale bytes][qh 32][qs 128]: d*sc*q - dmin*m
    static constexpr int UNIT_BLOCKS = 8, UNIT_BYTES = 176;
    typedef XInt<22> X;
    static __device__ __forceinline__ float block(const uint8_t *base, int seg, int jl, const X &x) {
        const int j = jl & 7;
        const int sb = seg + (jl >> 3) * 176;  // 16-byte aligned: rows and segments are whole super-blocks
        const uint32_t *S = (const uint32_t *)(base + sb);
        const uint32_t *qp = S + 12 + 8 * (j >> 1);
        int acc[3] = {0, 0, 0};
#pragma unroll
        for (int i = 0; i < 8; i++)  // bit j of qh byte l is the fifth bit of element l of sub-block j
            x.dot(acc, ((qp[i] >> (4 * (j & 1))) & 0x0F0F0F0Fu) | (((S[4 + i] >> j) & 0x01010101u) << 4), i);
        const int t = acc[0] + (acc[1] << 8) + (acc[2] << 16);
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
        return (h2f((uint16_t)(hd & 0xFFFF)) * (float)sc * (float)t - h2f((uint16_t)(hd >> 16)) * (float)mn * (float)(x.s0 + x.s1)) * x.inv;
    }
};

// What one launch works on. Up to three weight matrices of one format and K, their rows concatenated (Q|K|V,
// gate|up); where the activation row comes from; what happens to the dot products.
struct MvArgs {
    const uint8_t *w0, *w1, *w2;  // matrix i holds the concatenated rows [end_{i-1}, end_i)
    int end0, end1;
    int N, K;                     // concatenated rows; columns
    size_t row_bytes;
    int units_per_wave, n_groups;
    int mode;                     // MV_PLAIN, MV_RMSNORM, MV_MERGED_ATTENTION
    const float *x;               // the activation row (MV_PLAIN, MV_RMSNORM)
    const float *norm_w;          // MV_RMSNORM: the row is x * norm_w and the dot products are divided by rms(x)
    float eps;
    const float *attn_partial;    // MV_MERGED_ATTENTION: split-KV partials (m, l, acc[D]) of one query,
    const int32_t *kv_len;        //   [head][split][D + 2], merged on the fly (the row is the attention output)
    int head_dim, max_splits, tokens_per_split;
    int pair;                     // > 0: rows i and pair + i belong together, out[i] = silu(dot_i) * dot_{pair+i}
    float *out;
    const float *residual;        // added to the result (not with pair)
    MatvecRope rope;              // qmatvec2_kernel only: the rows are Q|K|V of one token, finished in the epilogue
};
enum { MV_PLAIN = 0, MV_RMSNORM = 1, MV_MERGED_ATTENTION = 2 };

__device__ __forceinline__ float mv_sigmoid(float v) { return 1.0f / (1.0f + (float)exp((double)(-v))); }  // cpu.go:384,397

template <class F, int T, int LP>
__global__ void __launch_bounds__(MV_THREADS) qmatvec_kernel(const MvArgs p) {
    constexpr int PASSES = 1 << LP, RG = MV_MAX_RG >> LP;  // 64-piece passes per staged row; rows per group
    __shared__ __attribute__((aligned(16))) uint8_t stage[MV_WAVES][MV_WAVE_LDS];
    __shared__ float part[2][MV_WAVES][MV_MAX_RG];
    __shared__ float s_ss[MV_WAVES];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int bl = lane & 31, rp = lane >> 5;
    const int N = p.N, K = p.K;
    const size_t row_bytes = p.row_bytes;
    const int n_units = K / (32 * F::UNIT_BLOCKS);
    const int u0 = min(wave * p.units_per_wave, n_units), u1 = min(u0 + p.units_per_wave, n_units);
    const int seg_blocks = (u1 - u0) * F::UNIT_BLOCKS;
    const int pair = p.pair;

    // Staging geometry of the wave's segment: 16-byte pieces from the aligned address at or below the segment.
    // Row r of a group: pieces from (row start + seg_off) & ~15; its first segment byte lands at byte sh_r of its
    // LDS row. Rows have different sh_r when row_bytes is not a multiple of 16.
    // A wave whose segment is empty (fewer units than waves) stages the row's last unit instead and adds
    // nothing (seg_blocks = 0): its loads stay inside the matrix without a special case.
    const size_t seg_off = (size_t)min(u0, n_units - 1) * F::UNIT_BYTES;
    const int seg_bytes = max(u1 - u0, 1) * F::UNIT_BYTES;
    uint8_t *my = &stage[wave][0];
    const int rstride = (seg_bytes + 15 + 16 + 15) & ~15;  // room for the leading offset and the trailing over-read
    const int ppr = rstride / 16;                            // pieces per row (<= 64 * PASSES)
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    constexpr int NP = MV_MAX_RG;  // load slots per lane: slot i = (row i >> LP, pass i & (PASSES - 1))
    u32x4 pc[NP];
    // Row r of group grp in the concatenated row space. With pair the group's first half are rows of the first
    // matrix and the second half the same rows of the second. Rows past the end repeat the last row.
    auto crow = [&](int grp, int r) __attribute__((always_inline)) {
        if (pair > 0) return (r / (RG / 2)) * pair + min(grp * (RG / 2) + r % (RG / 2), pair - 1);
        return min(grp * RG + r, N - 1);
    };
    // Byte offset of a concatenated row inside its matrix, and the matrix (selects over values read once from
    // the kernel arguments: indexing an argument array by row would turn into dependent loads).
    auto row_off = [&](int row) __attribute__((always_inline)) {
        const int local = row < p.end0 ? row : (row < p.end1 ? row - p.end0 : row - p.end1);
        return row_bytes * (size_t)local + seg_off;
    };
    auto row_base = [&](int row) __attribute__((always_inline)) { return row < p.end0 ? p.w0 : (row < p.end1 ? p.w1 : p.w2); };
    // Every load is unconditional: loads under a branch would be waited for one by one. A row's address math is
    // scalar (one row per slot); a lane only clamps its piece index to the row's last piece, so that no load
    // leaves the matrix. A group past the end loads the last row eight times (cache hits, results unused).
    auto issue = [&](int grp) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < NP; i++) {
            const int row = crow(grp, i >> LP);
            const size_t start = row_off(row);
            const uint8_t *first = row_base(row) + (start & ~(size_t)15);
            const uint32_t last_piece = (uint32_t)(((start & 15) + (size_t)seg_bytes - 1) >> 4);
            const uint32_t c = min((uint32_t)(((i & (PASSES - 1)) << 6) + lane), last_piece);
            pc[i] = __builtin_nontemporal_load((const u32x4 *)(first + c * 16u));
        }
    };
    int grp = blockIdx.x;
    issue(grp);  // the first group's weights are on their way while the activations are read
    __builtin_amdgcn_sched_barrier(0);  // keeps the activation loads behind the weight loads

    // the lane's activations (read once for the whole kernel)
    typename F::X x[T];
    float ss = 0.f;  // MV_RMSNORM: sum of squares of the lane's elements
#pragma unroll
    for (int t = 0; t < T; t++) {
        const int jl = bl + 32 * t;
        const bool have = jl < seg_blocks;
        const size_t e0 = have ? (size_t)(u0 * F::UNIT_BLOCKS + jl) * 32 : 0;  // a lane without a block re-reads the row's start
        float v[32];
        if (p.mode == MV_MERGED_ATTENTION) {
            // paged_merge_kernel's arithmetic for the 32 elements of this block (one head)
            const int D = p.head_dim, qh = (int)(e0 / D), d0 = (int)(e0 % D);
            const int ns = (p.kv_len[0] + p.tokens_per_split - 1) / p.tokens_per_split;
            const float *pb = p.attn_partial + (size_t)qh * p.max_splits * (D + 2);
            float M = -INFINITY, L = 0.f;
            for (int sp = 0; sp < ns; sp++) M = fmaxf(M, pb[(size_t)sp * (D + 2)]);
#pragma unroll
            for (int i = 0; i < 32; i++) v[i] = 0.f;
            for (int sp = 0; sp < ns; sp++) {
                const float *ps = pb + (size_t)sp * (D + 2);
                const float f = exp2f(ps[0] - M);
                L += ps[1] * f;
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const float4 q = *(const float4 *)(ps + 2 + d0 + 4 * i);  // 8-byte aligned only: D + 2 floats per split
                    v[4 * i] += q.x * f; v[4 * i + 1] += q.y * f; v[4 * i + 2] += q.z * f; v[4 * i + 3] += q.w * f;
                }
            }
#pragma unroll
            for (int i = 0; i < 32; i++) v[i] = L > 0.f ? v[i] / L : 0.f;
        } else {
            const float *ap = p.x + e0;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const float4 q = *(const float4 *)(ap + 4 * i);
                v[4 * i] = q.x; v[4 * i + 1] = q.y; v[4 * i + 2] = q.z; v[4 * i + 3] = q.w;
            }
            if (p.mode == MV_RMSNORM) {
                const float *wp = p.norm_w + e0;
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const float4 q = *(const float4 *)(wp + 4 * i);
                    const float wv[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        if (have && rp == 0) ss = fmaf(v[4 * i + e], v[4 * i + e], ss);  // every element counted once
                        v[4 * i + e] *= wv[e];
                    }
                }
            }
        }
        x[t].prep(v);
    }
    float row_fac = 1.f;
    if (p.mode == MV_RMSNORM) {  // 1/rms of the whole row: lanes, then waves, in a fixed order (cpu.go:200-220)
        ss = half_wave_sum(ss);   // the second half-wave holds zeros
        if (lane == 0) s_ss[wave] = ss;
        __syncthreads();
        const float tot = (s_ss[0] + s_ss[1]) + (s_ss[2] + s_ss[3]);
        row_fac = 1.0f / (float)sqrt((double)(tot / (float)K + p.eps));
    }

    // A workgroup walks over row groups grp, grp + gridDim.x, ...: while it works on one group out of LDS, the
    // next group's weights are in flight into registers. All its threads make the same number of trips.
    for (int it = 0; grp < p.n_groups; grp += gridDim.x, it++) {
#pragma unroll
        for (int i = 0; i < NP; i++) {
            const int r = i >> LP, c = ((i & (PASSES - 1)) << 6) + lane;
            if (c < ppr) *(u32x4 *)(my + r * rstride + c * 16) = pc[i];
        }
        // the wave reads only what it wrote: its own LDS operations are ordered, no barrier needed here
        issue(grp + (int)gridDim.x);

        float acc[RG / 2];
#pragma unroll
        for (int rr = 0; rr < RG / 2; rr++) {  // the lane's rows rp, rp + 2, ...: independent, so their LDS reads overlap
            const int r = rp + 2 * rr;
            const int sh = (int)(row_off(crow(grp, r)) & 15);
            acc[rr] = 0.f;
#pragma unroll
            for (int t = 0; t < T; t++) {
                const int jl = bl + 32 * t;
                if (jl < seg_blocks) acc[rr] += F::block(my, r * rstride + sh, jl, x[t]);
            }
        }
#pragma unroll
        for (int rr = 0; rr < RG / 2; rr++) {
            const float v = half_wave_sum(acc[rr]);
            if (bl == 0) part[it & 1][wave][rp + 2 * rr] = v;
        }
        __syncthreads();  // the other parity of part[] is written next trip, after its readers passed this barrier
        const float(*pp)[MV_MAX_RG] = part[it & 1];
        if (pair > 0) {
            const int i = grp * (RG / 2) + tid;
            if (tid < RG / 2 && i < pair) {
                const int j = tid + RG / 2;
                const float g = ((pp[0][tid] + pp[1][tid]) + (pp[2][tid] + pp[3][tid])) * row_fac;
                const float u = ((pp[0][j] + pp[1][j]) + (pp[2][j] + pp[3][j])) * row_fac;
                p.out[i] = __fmul_rn(__fmul_rn(g, mv_sigmoid(g)), u);  // cpu.go:390-400
            }
        } else if (tid < RG && grp * RG + tid < N) {
            float v = ((pp[0][tid] + pp[1][tid]) + (pp[2][tid] + pp[3][tid])) * row_fac;
            if (p.residual) v = __fadd_rn(p.residual[grp * RG + tid], v);
            p.out[grp * RG + tid] = v;
        }
    }
}

int device_cus(vx_backend *be);

// ---- Q4_0, second form: whole rows per wave, the activation's integer planes in LDS.
// The kernel above spends most of its instructions around its loads (per-trip address arithmetic, a workgroup
// barrier per 8 rows, every workgroup preparing its lanes' activations again per K segment). Here a workgroup
// prepares the row's planes once, into LDS; after that its waves do not meet again. A wave takes passes of NR
// consecutive rows (with `pair`: NR/2 rows of each matrix): their bytes are one contiguous run, read as aligned
// 16-byte pieces, lane l piece l + 64 i - the pattern memory serves fastest - into registers, the next pass in
// flight while the current one is worked on; the pieces go to the wave's own LDS rows, from where lane l takes
// block t*64 + l of every row of the pass (18-byte stride, any alignment) against the planes of that block, read
// once per step for all NR rows. One butterfly over the wave per row at the end of the pass. The arithmetic of a
// block is VQ4_0::block's.
constexpr int MV2_XSTRIDE = 28;  // dwords per block in LDS: planes [3][8], sum of xi, inv; padded to whole 16-byte pieces

// x: the block's 28 dwords; w: its 16 code bytes; d: its scale
__device__ __forceinline__ float mv2_q4_0_dot(const uint32_t (&w)[4], uint32_t d, const uint32_t (&x)[MV2_XSTRIDE]) {
    int a0 = 0, a1 = 0, a2 = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t lo = w[i] & 0x0F0F0F0Fu, hi = (w[i] >> 4) & 0x0F0F0F0Fu;
        a0 = (int)__builtin_amdgcn_udot4(lo, x[i], (uint32_t)a0, false);
        a1 = (int)__builtin_amdgcn_udot4(lo, x[8 + i], (uint32_t)a1, false);
        a2 = __builtin_amdgcn_sdot4((int)lo, (int)x[16 + i], a2, false);
        a0 = (int)__builtin_amdgcn_udot4(hi, x[4 + i], (uint32_t)a0, false);
        a1 = (int)__builtin_amdgcn_udot4(hi, x[12 + i], (uint32_t)a1, false);
        a2 = __builtin_amdgcn_sdot4((int)hi, (int)x[20 + i], a2, false);
    }
    const int t = a0 + (a1 << 8) + (a2 << 16) - 8 * (int)x[24];  // sum (q - 8) xi, exact
    return h2f((uint16_t)d) * ((float)t * __uint_as_float(x[25]));
}

__device__ __forceinline__ float wave_sum64(float t) {
    t = half_wave_sum(t);
    return t + __shfl_xor(t, 32, 64);
}

// NR rows per pass, NPL 16-byte pieces per lane and pass (64 * NPL >= NR * row_bytes / 16). Every matrix (with
// `pair`: each of the two) holds a multiple of NR (NR/2) rows and whole 16-byte rows: the host checks.
// TT: steps of 64 blocks per row when known at compile time (the loop is then unrolled and its LDS reads overlap), 0: any.
template <int NR, int NPL, int TT = 0>
__global__ void __launch_bounds__(MV_THREADS) qmatvec2_kernel(const MvArgs p, int n_passes) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    extern __shared__ __attribute__((aligned(16))) uint32_t smem[];  // planes [nblocks + 1][MV2_XSTRIDE] (the last block zeros), then the waves' rows
    __shared__ float s_ss[MV_WAVES];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int K = p.K, nblocks = K / 32, pair = p.pair;
    const int T = TT > 0 ? TT : (nblocks + 63) / 64;
    const int rb = (int)p.row_bytes;
    const int total = NR * (rb / 16);         // pieces of a pass
    const int half_pieces = total / 2;        // pair: pieces of each matrix' share
    uint8_t *my = (uint8_t *)(smem + (size_t)(nblocks + 1) * MV2_XSTRIDE) + (size_t)wave * (NR * rb + 16);

    // Pass q: rows [q * NR, q * NR + NR) of the concatenated rows; with pair, rows [q * NR/2, ...) of both matrices.
    auto issue = [&](int q, u32x4 (&pc)[NPL]) __attribute__((always_inline)) {
        const uint8_t *b0, *b1;
        if (pair > 0) {
            b0 = p.w0 + (size_t)q * (NR / 2) * rb;
            b1 = p.w1 + (size_t)q * (NR / 2) * rb - (size_t)half_pieces * 16;
        } else {
            const int row = q * NR;
            const uint8_t *base = row < p.end0 ? p.w0 : (row < p.end1 ? p.w1 : p.w2);
            const int local = row < p.end0 ? row : (row < p.end1 ? row - p.end0 : row - p.end1);
            b0 = b1 = base + (size_t)local * rb;
        }
#pragma unroll
        for (int i = 0; i < NPL; i++) {
            const int c = min(lane + 64 * i, total - 1);
            const uint8_t *b = (pair > 0 && c >= half_pieces) ? b1 : b0;
            pc[i] = __builtin_nontemporal_load((const u32x4 *)(b + (size_t)c * 16));
        }
    };
    const int n_waves = gridDim.x * MV_WAVES;
    int q = blockIdx.x * MV_WAVES + wave;

    // The activation's first loads go ahead of the weights': behind them they would wait for all of those.
    float4 xv[8], nv[8];
    if (tid < nblocks) {
#pragma unroll
        for (int i = 0; i < 8; i++) xv[i] = *(const float4 *)(p.x + (size_t)tid * 32 + 4 * i);
        if (p.mode == MV_RMSNORM) {
#pragma unroll
            for (int i = 0; i < 8; i++) nv[i] = *(const float4 *)(p.norm_w + (size_t)tid * 32 + 4 * i);
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    u32x4 pc[NPL];
    if (q < n_passes) issue(q, pc);
    __builtin_amdgcn_sched_barrier(0);

    // activation -> integer planes in LDS (XInt<23>), one block per thread and trip
    float ss = 0.f;
    for (int j = tid; j < nblocks; j += MV_THREADS) {
        if (j != tid) {
#pragma unroll
            for (int i = 0; i < 8; i++) xv[i] = *(const float4 *)(p.x + (size_t)j * 32 + 4 * i);
            if (p.mode == MV_RMSNORM) {
#pragma unroll
                for (int i = 0; i < 8; i++) nv[i] = *(const float4 *)(p.norm_w + (size_t)j * 32 + 4 * i);
            }
        }
        float v[32];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            v[4 * i] = xv[i].x; v[4 * i + 1] = xv[i].y; v[4 * i + 2] = xv[i].z; v[4 * i + 3] = xv[i].w;
        }
        if (p.mode == MV_RMSNORM) {
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const float wv[4] = {nv[i].x, nv[i].y, nv[i].z, nv[i].w};
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    ss = fmaf(v[4 * i + e], v[4 * i + e], ss);
                    v[4 * i + e] *= wv[e];
                }
            }
        }
        XInt<23> x;
        x.prep(v);
        uint32_t *dst = smem + (size_t)j * MV2_XSTRIDE;
#pragma unroll
        for (int pl = 0; pl < 3; pl++) {
            *(u32x4 *)(dst + pl * 8) = u32x4{x.p[pl][0], x.p[pl][1], x.p[pl][2], x.p[pl][3]};
            *(u32x4 *)(dst + pl * 8 + 4) = u32x4{x.p[pl][4], x.p[pl][5], x.p[pl][6], x.p[pl][7]};
        }
        *(u32x4 *)(dst + 24) = u32x4{(uint32_t)(x.s0 + x.s1), __float_as_uint(x.inv), 0u, 0u};
    }
    if (tid < MV2_XSTRIDE) smem[(size_t)nblocks * MV2_XSTRIDE + tid] = 0u;
    float row_fac = 1.f;
    if (p.mode == MV_RMSNORM) {  // 1/rms of the row: lanes by a fixed butterfly, then the waves in order (cpu.go:200-220)
        for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
        if (lane == 0) s_ss[wave] = ss;
    }
    __syncthreads();
    if (p.mode == MV_RMSNORM) {
        const float tot = (s_ss[0] + s_ss[1]) + (s_ss[2] + s_ss[3]);
        row_fac = 1.0f / (float)sqrt((double)(tot / (float)K + p.eps));
    }

    // one pass: its pieces to the wave's LDS rows, the next pass on its way into the same registers, then the rows'
    // dot products
    auto pass = [&](int q, u32x4 (&pc)[NPL]) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < NPL; i++) {
            const int c = lane + 64 * i;
            if (c < total) *(u32x4 *)(my + (size_t)c * 16) = pc[i];
        }
        // (the wave reads only what it wrote itself: its LDS operations are ordered, no barrier)
        if (q + n_waves < n_passes) issue(q + n_waves, pc);
        float acc[NR];
#pragma unroll
        for (int r = 0; r < NR; r++) acc[r] = 0.f;
        constexpr int UNROLL_T = TT > 0 ? TT : 1;  // (a trip count known only at run time: as written)
#pragma unroll UNROLL_T
        for (int t = 0; t < (TT > 0 ? TT : T); t++) {
            const int j = t * 64 + lane;
            const int jx = j < nblocks ? j : nblocks;   // past the row's end: the zero planes
            const int jw = min(j, nblocks - 1);
            uint32_t x[MV2_XSTRIDE];
#pragma unroll
            for (int i = 0; i < MV2_XSTRIDE / 4; i++) {
                const u32x4 f = *(const u32x4 *)(smem + (size_t)jx * MV2_XSTRIDE + 4 * i);
                x[4 * i] = f[0]; x[4 * i + 1] = f[1]; x[4 * i + 2] = f[2]; x[4 * i + 3] = f[3];
            }
#pragma unroll
            for (int r = 0; r < NR; r++) {
                const int o = r * rb + jw * 18;
                uint32_t w[4];
                lds_dwords<4>(my, o + 2, w);
                acc[r] += mv2_q4_0_dot(w, lds_u16(my, o), x);
            }
        }
#pragma unroll
        for (int r = 0; r < NR; r++) acc[r] = wave_sum64(acc[r]) * row_fac;
        if (pair > 0) {
            float g = acc[0], u = acc[NR / 2];
#pragma unroll
            for (int r = 1; r < NR / 2; r++) {
                g = lane == r ? acc[r] : g;
                u = lane == r ? acc[NR / 2 + r] : u;
            }
            if (lane < NR / 2) p.out[q * (NR / 2) + lane] = __fmul_rn(__fmul_rn(g, mv_sigmoid(g)), u);  // cpu.go:390-400
        } else {
            float v = acc[0];
#pragma unroll
            for (int r = 1; r < NR; r++) v = lane == r ? acc[r] : v;
            if (p.rope.q_out) {
                // rows 2j and 2j + 1 of a head are a RoPE pair (backend/cpu/cpu.go:226-303) and sit in lanes 2i, 2i + 1
                const float other = __shfl_xor(v, 1, 64);
                if (lane < NR) {
                    const int row = q * NR + lane, qd = p.rope.qd, kvd = p.rope.kvd;
                    const bool is_q = row < qd, is_v = row >= qd + kvd;
                    const int o = is_q ? row : (is_v ? row - qd - kvd : row - qd);
                    float res = v;
                    if (!is_v) {
                        const float2 cs = p.rope.cs_tab[(o & (p.rope.head_dim - 1)) >> 1];
                        const float a = (lane & 1) ? other : v, b = (lane & 1) ? v : other;
                        res = (lane & 1) ? __fadd_rn(__fmul_rn(a, cs.y), __fmul_rn(b, cs.x))
                                         : __fsub_rn(__fmul_rn(a, cs.x), __fmul_rn(b, cs.y));
                    }
                    if (is_q) {
                        p.rope.q_out[o] = res;
                    } else {
                        const int slot = p.rope.slot[0], blk = slot / p.rope.block_size, off = slot - blk * p.rope.block_size;
                        const size_t part = (size_t)p.rope.block_size * kvd;
                        ((_Float16 *)p.rope.pool)[(size_t)blk * 2 * part + (size_t)off * kvd + (is_v ? part : 0) + o] = (_Float16)res;
                    }
                }
            } else if (lane < NR) {
                const int row = q * NR + lane;
                if (p.residual) v = __fadd_rn(p.residual[row], v);
                p.out[row] = v;
            }
        }
    };
    for (; q < n_passes; q += n_waves) pass(q, pc);
}

template <int NR, int NPL, int TT = 0>
void launch_second(vx_backend *be, MvArgs &a, size_t lds) {
    static int per_cu = 0;
    if (per_cu == 0) {
        (void)hipFuncSetAttribute((const void *)qmatvec2_kernel<NR, NPL, TT>, hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, qmatvec2_kernel<NR, NPL, TT>, MV_THREADS, lds) != hipSuccess || per_cu < 1)
            per_cu = 1;
    }
    const int n_passes = a.pair > 0 ? a.pair / (NR / 2) : a.N / NR;
    // as many workgroups as fit at once, or fewer when that makes every wave's number of passes equal
    const int wgs = ceil_div(n_passes, MV_WAVES);
    const int trips = ceil_div(wgs, per_cu * device_cus(be));
    qmatvec2_kernel<NR, NPL, TT><<<ceil_div(wgs, trips), MV_THREADS, lds, be->stream>>>(a, n_passes);
}

// Launches the second form when it serves the call: Q4_0, an activation row from memory, rows of whole 16-byte
// pieces, every matrix a whole number of passes.
bool launch_second_form(vx_backend *be, int fmt, MvArgs &a) {
    static const bool off = getenv("VEXEL_HIP_MATVEC_FIRST_FORM") != nullptr;
    if (off || fmt != VX_Q4_0 || a.mode == MV_MERGED_ATTENTION) return false;
    const int nblocks = a.K / 32;
    const size_t rb = (size_t)nblocks * 18;
    if (rb % 16 != 0) return false;
    int nr, npl;
    if (4 * rb / 16 <= 64 * 9) nr = 4, npl = 9;         // K <= 4096
    else if (2 * rb / 16 <= 64 * 9) nr = 2, npl = 9;    // K <= 8192
    else if (2 * rb / 16 <= 64 * 13) nr = 2, npl = 13;  // K <= 11776
    else return false;
    if (a.rope.q_out && (a.pair > 0 || a.residual || nr % 2 != 0 || a.rope.qd % nr != 0 || a.rope.kvd % nr != 0 ||
                         (a.rope.head_dim & (a.rope.head_dim - 1)) != 0 || a.N != a.rope.qd + 2 * a.rope.kvd))
        return false;
    const int unit = a.pair > 0 ? nr / 2 : nr;
    if (a.pair > 0) {
        if (a.pair % unit != 0) return false;
    } else if (a.end0 % unit != 0 || a.end1 % unit != 0 || a.N % unit != 0)
        return false;
    const size_t lds = (size_t)(nblocks + 1) * MV2_XSTRIDE * 4 + MV_WAVES * (nr * rb + 16);
    if (lds > 120 * 1024) return false;
    a.row_bytes = rb;
    const int steps = (nblocks + 63) / 64;
    if (nr == 4 && steps == 2) launch_second<4, 9, 2>(be, a, lds);       // K = 4096
    else if (nr == 4) launch_second<4, 9>(be, a, lds);
    else if (npl == 9) launch_second<2, 9>(be, a, lds);
    else if (steps == 6) launch_second<2, 13, 6>(be, a, lds);           // K = 11008
    else launch_second<2, 13>(be, a, lds);
    return true;
}

// ---- BF16, one activation row: out[n] = sum_k a[k] * W[n][k] in float32 (the bf16 pattern is the high half of the
// float32 it stands for, pkg/gguf/dequant.go:215-228). The activation row sits in LDS as floats; a wave takes two rows
// at a time, every lane 16 bytes (eight weights) of each per trip, up to eight trips' loads in flight, and adds its
// lanes by one butterfly per row. HBM bound: 2 bytes per weight.
__global__ void __launch_bounds__(MV_THREADS) bf16_matvec_kernel(const uint8_t *__restrict__ W, const float *__restrict__ a,
                                                                float *__restrict__ out, const float *__restrict__ residual,
                                                                int N, int K) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    extern __shared__ __attribute__((aligned(16))) float xs[];  // [K]
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    for (int i = tid * 4; i < K; i += MV_THREADS * 4) *(float4 *)(xs + i) = *(const float4 *)(a + i);
    __syncthreads();
    const int n_waves = gridDim.x * MV_WAVES, pieces = K / 8;  // 16-byte pieces of a row
    constexpr int U = 8;
    for (int pr = blockIdx.x * MV_WAVES + wave; 2 * pr < N; pr += n_waves) {
        const int r0 = 2 * pr, r1 = min(r0 + 1, N - 1);
        const uint8_t *w0 = W + (size_t)r0 * K * 2, *w1 = W + (size_t)r1 * K * 2;
        float acc0 = 0.f, acc1 = 0.f;
        for (int p0 = 0; p0 < pieces; p0 += 64 * U) {
            u32x4 q0[U], q1[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int pc = min(p0 + 64 * u + lane, pieces - 1);  // (past the row's end: the last piece again, not added)
                q0[u] = __builtin_nontemporal_load((const u32x4 *)(w0 + (size_t)pc * 16));
                q1[u] = __builtin_nontemporal_load((const u32x4 *)(w1 + (size_t)pc * 16));
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int pc = p0 + 64 * u + lane;
                if (pc < pieces) {
                    const float4 xa = *(const float4 *)(xs + pc * 8), xb = *(const float4 *)(xs + pc * 8 + 4);
                    const float x[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        acc0 = fmaf(x[2 * e], __uint_as_float(q0[u][e] << 16), acc0);
                        acc0 = fmaf(x[2 * e + 1], __uint_as_float(q0[u][e] & 0xFFFF0000u), acc0);
                        acc1 = fmaf(x[2 * e], __uint_as_float(q1[u][e] << 16), acc1);
                        acc1 = fmaf(x[2 * e + 1], __uint_as_float(q1[u][e] & 0xFFFF0000u), acc1);
                    }
                }
            }
        }
        acc0 = wave_sum64(acc0);
        acc1 = wave_sum64(acc1);
        if (lane == 0) {
            out[r0] = residual ? __fadd_rn(residual[r0], acc0) : acc0;
            if (r0 + 1 < N) out[r0 + 1] = residual ? __fadd_rn(residual[r0 + 1], acc1) : acc1;
        }
    }
}

int device_cus(vx_backend *be) {
    static int cus = 0;
    if (cus == 0) {
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, be->device) != hipSuccess || cus <= 0) cus = 256;
    }
    return cus;
}

// Launches qmatvec_kernel<F, T, LP> on as many workgroups as are resident at once (registers and LDS, asked once
// per instantiation), each walking over several row groups.
template <class F, int T, int LP>
void launch_tl(vx_backend *be, MvArgs &a) {
    static int per_cu = 0;
    if (per_cu == 0) {
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, qmatvec_kernel<F, T, LP>, MV_THREADS, 0) != hipSuccess || per_cu < 1)
            per_cu = 1;
    }
    constexpr int RG = MV_MAX_RG >> LP;
    a.n_groups = a.pair > 0 ? ceil_div(a.pair, RG / 2) : ceil_div(a.N, RG);
    // as many workgroups as fit at once, or fewer when that makes every workgroup's number of trips equal
    const int resident = per_cu * device_cus(be);
    const int trips = ceil_div(a.n_groups, resident);
    const dim3 grid(ceil_div(a.n_groups, trips));
    qmatvec_kernel<F, T, LP><<<grid, MV_THREADS, 0, be->stream>>>(a);
}

template <class F>
int launch(vx_backend *be, MvArgs &a) {
    const int n_units = a.K / (32 * F::UNIT_BLOCKS);
    const int upw = ceil_div(n_units, MV_WAVES);
    const int seg_blocks = upw * F::UNIT_BLOCKS;
    const int T = ceil_div(seg_blocks, 32);
    if (T > MV_MAX_T) return VX_ERR_UNSUPPORTED;
    const int rstride = (upw * F::UNIT_BYTES + 15 + 16 + 15) & ~15;
    // a staged row takes 1, 2 or 4 passes of 64 pieces; the group has 8, 4 or 2 rows, so that a lane always has 8 loads
    int lp = 0;
    while ((64 << lp) < rstride / 16) lp++;
    if (lp > 2 || (MV_MAX_RG >> lp) * rstride > MV_WAVE_LDS) return VX_ERR_UNSUPPORTED;
    a.row_bytes = (size_t)n_units * F::UNIT_BYTES;
    a.units_per_wave = upw;
#define VX_MV(TT, LL)                   \
    case TT * 4 + LL:                   \
        launch_tl<F, TT, LL>(be, a);    \
        break;
    switch (T * 4 + lp) {
        VX_MV(1, 0) VX_MV(1, 1) VX_MV(2, 0) VX_MV(2, 1) VX_MV(2, 2) VX_MV(3, 1) VX_MV(3, 2) VX_MV(4, 1) VX_MV(4, 2)
    default: return VX_ERR_UNSUPPORTED;
    }
#undef VX_MV
    VX_CHECK_LAUNCH();
    return VX_OK;
}

// Bytes of one weight row, 0 when the format or K has no matrix-vector kernel.
size_t mv_row_bytes(int fmt, int k) {
    switch (fmt) {
    case VX_Q4_0: return k % 32 == 0 ? (size_t)(k / 32) * 18 : 0;
    case VX_Q8_0: return k % 32 == 0 ? (size_t)(k / 32) * 34 : 0;
    case VX_Q4_K: return k % 256 == 0 ? (size_t)(k / 256) * 144 : 0;
    case VX_Q6_K: return k % 256 == 0 ? (size_t)(k / 256) * 210 : 0;
    case VX_Q5_0: return k % 32 == 0 ? (size_t)(k / 32) * 22 : 0;
    case VX_Q5_K: return k % 256 == 0 ? (size_t)(k / 256) * 176 : 0;
    }
    return 0;
}

// Whether qmatvec_kernel has an instantiation for rows of this format and length.
template <class F>
bool shape_ok(int k) {
    const int n_units = k / (32 * F::UNIT_BLOCKS);
    const int upw = ceil_div(n_units, MV_WAVES);
    const int T = ceil_div(upw * F::UNIT_BLOCKS, 32);
    if (n_units < 1 || T > MV_MAX_T) return false;
    const int rstride = (upw * F::UNIT_BYTES + 15 + 16 + 15) & ~15;
    int lp = 0;
    while ((64 << lp) < rstride / 16) lp++;
    if (lp > 2 || (MV_MAX_RG >> lp) * rstride > MV_WAVE_LDS) return false;
    switch (T * 4 + lp) {
    case 4: case 5: case 8: case 9: case 10: case 13: case 14: case 17: case 18: return true;
    }
    return false;
}

int launch_fmt(vx_backend *be, int fmt, MvArgs &a) {
    if (launch_second_form(be, fmt, a)) {
        VX_CHECK_LAUNCH();
        return VX_OK;
    }
    if (a.rope.q_out) return VX_ERR_UNSUPPORTED;  // only that kernel finishes Q|K|V rows itself
    switch (fmt) {
    case VX_Q4_0: return launch<VQ4_0>(be, a);
    case VX_Q8_0: return launch<VQ8_0>(be, a);
    case VX_Q4_K: return launch<VQ4_K>(be, a);
    case VX_Q6_K: return launch<VQ6_K>(be, a);
    case VX_Q5_0: return launch<VQ5_0>(be, a);
    case VX_Q5_K: return launch<VQ5_K>(be, a);
    }
    return VX_ERR_UNSUPPORTED;
}

}  // namespace

namespace vx {

bool matvec_ok(int fmt, const void *const *ws, const int *ns, int nw, int k) {
    const size_t rb = mv_row_bytes(fmt, k);
    if (rb == 0 || nw < 1 || nw > 3) return false;
    for (int i = 0; i < nw; i++)
        if (ns[i] < 1 || ((uintptr_t)ws[i] % 16) != 0 || ((size_t)ns[i] * rb) % 16 != 0) return false;
    switch (fmt) {
    case VX_Q4_0: return shape_ok<VQ4_0>(k);
    case VX_Q8_0: return shape_ok<VQ8_0>(k);
    case VX_Q4_K: return shape_ok<VQ4_K>(k);
    case VX_Q6_K: return shape_ok<VQ6_K>(k);
    case VX_Q5_0: return shape_ok<VQ5_0>(k);
    case VX_Q5_K: return shape_ok<VQ5_K>(k);
    }
    return false;
}

// out[n] = a . W[n] (+ residual[n]) for one activation row. VX_ERR_UNSUPPORTED (nothing launched) when the shape is
// outside the kernel's range: the caller then takes another path.
int run_matvec(vx_backend *be, int fmt, const float *a, const void *b, float *out, const float *residual, int n, int k) {
    if (fmt == VX_BF16) {
        if (k % 8 != 0 || (size_t)k * 4 > 96 * 1024 || ((uintptr_t)b % 16) != 0 || ((uintptr_t)a % 16) != 0) return VX_ERR_UNSUPPORTED;
        static int per_cu = 0;
        if (per_cu == 0) {
            (void)hipFuncSetAttribute((const void *)bf16_matvec_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);
            per_cu = 1;
        }
        const int wgs = std::min(ceil_div(ceil_div(n, 2), MV_WAVES), 4 * device_cus(be));
        bf16_matvec_kernel<<<wgs, MV_THREADS, (size_t)k * 4, be->stream>>>((const uint8_t *)b, a, out, residual, n, k);
        VX_CHECK_LAUNCH();
        return VX_OK;
    }
    MatvecSource src;
    src.x = a;
    const void *ws[1] = {b};
    const int ns[1] = {n};
    return run_matvec_fused(be, fmt, ws, ns, 1, k, src, out, residual, 0);
}

// The general form: nw <= 3 matrices of one format and K, rows concatenated; the activation row from `src`;
// pair != 0: two matrices of equal height, out[i] = silu(row i of the first) * (row i of the second).
int run_matvec_fused(vx_backend *be, int fmt, const void *const *ws, const int *ns, int nw, int k, const MatvecSource &src,
                     float *out, const float *residual, int pair) {
    const size_t rb = mv_row_bytes(fmt, k);
    if (rb == 0 || nw < 1 || nw > 3) return VX_ERR_UNSUPPORTED;
    MvArgs a = {};
    const uint8_t *w[3] = {nullptr, nullptr, nullptr};
    int end[3] = {0, 0, 0}, tot = 0;
    for (int i = 0; i < 3; i++) {
        const int j = i < nw ? i : nw - 1;
        if (i < nw) {
            // aligned 16-byte pieces must stay inside each matrix: aligned base, a whole number of pieces
            if (ns[i] < 1 || ((uintptr_t)ws[i] % 16) != 0 || ((size_t)ns[i] * rb) % 16 != 0) return VX_ERR_UNSUPPORTED;
            tot += ns[i];
        }
        w[i] = (const uint8_t *)ws[j];
        end[i] = tot;
    }
    if (pair && (nw != 2 || ns[0] != ns[1] || residual)) return VX_ERR_UNSUPPORTED;
    a.w0 = w[0]; a.w1 = w[1]; a.w2 = w[2];
    a.end0 = end[0]; a.end1 = end[1];
    a.N = tot; a.K = k;
    a.pair = pair ? ns[0] : 0;
    a.out = out; a.residual = residual;
    a.rope = src.rope;
    if (a.rope.q_out && src.attn_partial) return VX_ERR_UNSUPPORTED;
    if (src.attn_partial) {
        if (!src.kv_len || src.head_dim < 32 || src.head_dim % 32 != 0 || k % src.head_dim != 0) return VX_ERR_UNSUPPORTED;
        a.mode = MV_MERGED_ATTENTION;
        a.attn_partial = src.attn_partial; a.kv_len = src.kv_len;
        a.head_dim = src.head_dim; a.max_splits = src.max_splits; a.tokens_per_split = src.tokens_per_split;
    } else {
        if (!src.x || ((uintptr_t)src.x % 16) != 0 || ((uintptr_t)src.norm_w % 16) != 0) return VX_ERR_UNSUPPORTED;
        a.mode = src.norm_w ? MV_RMSNORM : MV_PLAIN;
        a.x = src.x; a.norm_w = src.norm_w; a.eps = src.eps;
    }
    return launch_fmt(be, fmt, a);
}

}  // namespace vx
