// The prepared activation of the quantized GEMMs: where its parts sit in the workspace and how one wave writes
// one 256-column chunk of one row. Shared by the kernels that prepare activations (qgemm.hip) and the decode
// attention kernel, whose last workgroup of a chunk merges the split partial sums straight into this form.
#pragma once
#include "common.h"

namespace vx {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));

// Workspace layout (be->gemm_ws): inv_scale[Mpad], then tiles [K/32][Mpad/16][2][64] half8,
// then bsum[K/32][Mpad] (block sums of the scaled row, for Q4_K's min term), then cscale[K/256][Mpad].
struct PrepView {
    half8 *tiles;
    float *inv_scale;  // [Mpad] row factor: multiplies the finished dot products of the row
    float *cscale;     // [K/256][Mpad] factor of each 256-column chunk's partial dot product
    float *bsum;
};

__host__ __device__ inline size_t prep_tiles_bytes(int mpad, int k) { return (size_t)(k / 32) * (mpad / 16) * 2 * 64 * 16; }

__device__ __forceinline__ float wave_max(float v) {
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

// Scales the wave's 256 values by a power of two chosen from their maximum, splits them hi + lo and writes the
// MFMA-ready tiles, the block sums and the chunk factor of (row r, chunk c).
__device__ __forceinline__ void write_chunk(const PrepView &pv, int r, int c, const float (&y)[4], int Mpad) {
    const int lane = threadIdx.x & 63;
    const float amax = wave_max(fmaxf(fmaxf(fabsf(y[0]), fabsf(y[1])), fmaxf(fabsf(y[2]), fabsf(y[3]))));
    float s = 1.f, inv = 1.f;
    if (amax > 0.f && amax < INFINITY) {
        int ex;
        (void)frexpf(amax, &ex);
        s = ldexpf(1.f, 13 - ex);
        inv = ldexpf(1.f, ex - 13);
    }
    if (lane == 0) pv.cscale[(size_t)c * Mpad + r] = inv;
    // lane l = 8*step + 4*half + g holds block elements 16*half + 4g .. +3; slot order of lane group g is
    // {4g, 4g+2, 16+4g, 16+4g+2, 4g+1, 4g+3, 16+4g+1, 16+4g+3}: the low-half lane fetches the high half's values
    const float a[4] = {y[0] * s, y[1] * s, y[2] * s, y[3] * s};
    float b[4];
#pragma unroll
    for (int i = 0; i < 4; i++) b[i] = __shfl_down(a[i], 4, 64);
    float bs = a[0] + a[1] + a[2] + a[3];
    bs += __shfl_xor(bs, 1, 64);
    bs += __shfl_xor(bs, 2, 64);
    bs += __shfl_xor(bs, 4, 64);
    const int step = c * 8 + (lane >> 3), half = (lane >> 2) & 1, g = lane & 3;
    if (half == 0) {
        const float v[8] = {a[0], a[2], b[0], b[2], a[1], a[3], b[1], b[3]};
        half8 h, l;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            h[i] = (_Float16)v[i];
            l[i] = (_Float16)(v[i] - (float)h[i]);
        }
        const int mtiles = Mpad / 16, mt = r >> 4, ln = r & 15;
        half8 *t = pv.tiles + ((size_t)(step * mtiles + mt) * 2) * 64 + g * 16 + ln;
        t[0] = h;
        t[64] = l;
        if (g == 0) pv.bsum[(size_t)step * Mpad + r] = bs;
    }
}

// Columns k .. k+3 of row r's attention output from its split partial sums (per row and head: max_splits records
// of [running maximum, sum of weights, D weighted value sums], the first ns of them written), as
// paged_merge_kernel computes it for up to eight splits (splits added in index order; beyond eight, in groups of eight
// under a running maximum).
// DEVICE_SCOPE: the records were written by other workgroups of the running launch with device-scope stores; every
// value is read by a device-scope load, which is served from where those stores went and not from this compute
// unit's or this die's cache.
template <bool DEVICE_SCOPE = false>
__device__ __forceinline__ void split_merge4(const float *__restrict__ part, int ns, int num_heads, int D, int max_splits,
                                             int r, int k, float (&y)[4]) {
    auto ld = [](const float *p) {
        return DEVICE_SCOPE ? __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : *p;
    };
    const int P = D + 2, h = k / D, d = k % D;
    const float *pb = part + ((size_t)r * num_heads + h) * max_splits * P;
    // Eight splits at a time, all their loads in flight together (a device-scope load is a trip to memory): the
    // running maximum moves up between the groups and what was added so far is rescaled, the first group from zero.
    float Mx = -INFINITY, L = 0.f, A[4] = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < ns; s0 += 8) {
        float v[8][6];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const float *ps = pb + (size_t)min(s0 + j, ns - 1) * P;
            v[j][0] = ld(ps);
            v[j][1] = ld(ps + 1);
#pragma unroll
            for (int e = 0; e < 4; e++) v[j][2 + e] = ld(ps + 2 + d + e);
        }
        float Mn = Mx;
#pragma unroll
        for (int j = 0; j < 8; j++) Mn = fmaxf(Mn, s0 + j < ns ? v[j][0] : -INFINITY);
        const float keep = (Mx == -INFINITY) ? 0.f : exp2f(Mx - Mn);
        Mx = Mn;
        L *= keep;
#pragma unroll
        for (int e = 0; e < 4; e++) A[e] *= keep;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            if (s0 + j >= ns) break;
            const float f = exp2f(v[j][0] - Mx);
            L += v[j][1] * f;
#pragma unroll
            for (int e = 0; e < 4; e++) A[e] += v[j][2 + e] * f;
        }
    }
#pragma unroll
    for (int e = 0; e < 4; e++) y[e] = (L > 0.f) ? A[e] / L : 0.f;
}

// Makes the prepared-activation workspace hold an [m,k] activation whose rows carry the factor 1 and returns its
// view, when the chunk-wise kernels serve the shape (qgemm.hip); VX_ERR_UNSUPPORTED when they do not.
int prep_begin_chunked(vx_backend *be, int m, int k, PrepView *pv, int *mpad);

}  // namespace vx
