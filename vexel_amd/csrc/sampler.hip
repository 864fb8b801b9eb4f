// Token sampling on the device: Sampler.Sample (inference/pkg/sampler/sampler.go:48-204) row by row, with the
// uniform draw of each row given by the caller. The reference works in float32 and adds in index order (softmax
// sum, the sums after top-k and top-p, the final cumulative walk) or in descending-probability order (the nucleus
// walk); those sums are kept sequential here, so the chosen token is the reference's bit for bit:
//   * one workgroup per row; everything that is order-free (scaling, maximum, exp, division, the top-k threshold by
//     bitwise selection, the sort for the nucleus) runs on all 1024 threads;
//   * a sequential sum is walked by wave 0: its lanes stage 256 consecutive values at a time in LDS and the running
//     sum takes them from there in order, one dependent addition per element;
//   * an entry that a cut sets to 0 adds nothing to any later sum, so after top-k (and again after top-p) the
//     survivors are compacted, in index order, into a short list, and the later walks and the sort run over it;
//   * the nucleus order is a bitonic sort of 64-bit keys (probability bits inverted, then the list position:
//     descending probability, ties by ascending index) in the row's scratch.
#include <float.h>

#include "common.h"

using namespace vx;

namespace {

constexpr int ST = 1024;

// The two sequential walks over values 0..cnt-1, by all 64 lanes of one wave; load(i) gives value i and is only
// called with i < cnt. The lanes fetch 256 consecutive values at a time into a wave-private LDS stage (the next 256
// while the current ones are added); every lane then reads them back in order (same address in all lanes: a
// broadcast) and adds, so the chain is one dependent float32 addition per element.
typedef float f4v __attribute__((ext_vector_type(4)));
struct WalkStage {
    float v[2][256];
};

template <class L>
__device__ __forceinline__ void stage_put(WalkStage &st, int half, int i0, int cnt, L load) {
    const int lane = threadIdx.x & 63;
    float4 o;
    o.x = (i0 + 0 < cnt) ? load(i0 + 0) : 0.f;
    o.y = (i0 + 1 < cnt) ? load(i0 + 1) : 0.f;
    o.z = (i0 + 2 < cnt) ? load(i0 + 2) : 0.f;
    o.w = (i0 + 3 < cnt) ? load(i0 + 3) : 0.f;
    *(float4 *)&st.v[half][lane * 4] = o;
}

// Sum in index order, float32, one rounding per addition (values past the end count as +0, which changes nothing).
template <class L>
__device__ __forceinline__ float sum_in_order(int cnt, L load, WalkStage &st) {
    const int lane = threadIdx.x & 63;
    float s = 0.f;
    stage_put(st, 0, lane * 4, cnt, load);
    int half = 0;
    for (int base = 0; base < cnt; base += 256, half ^= 1) {
        __builtin_amdgcn_wave_barrier();
        if (base + 256 < cnt) stage_put(st, half ^ 1, base + 256 + lane * 4, cnt, load);
        __builtin_amdgcn_wave_barrier();
#pragma unroll 16
        for (int i = 0; i < 256; i += 4) {
            const f4v v = *(const f4v *)&st.v[half][i];
            s = __fadd_rn(__fadd_rn(__fadd_rn(__fadd_rn(s, v.x), v.y), v.z), v.w);
        }
    }
    return s;
}

// First position whose cumulative sum (same order, same rounding) exceeds `bound`, or -1.
template <class L>
__device__ __forceinline__ int first_past(int cnt, float bound, L load, WalkStage &st) {
    const int lane = threadIdx.x & 63;
    float s = 0.f;
    int found = -1;
    stage_put(st, 0, lane * 4, cnt, load);
    int half = 0;
    for (int base = 0; base < cnt && found < 0; base += 256, half ^= 1) {
        __builtin_amdgcn_wave_barrier();
        if (base + 256 < cnt) stage_put(st, half ^ 1, base + 256 + lane * 4, cnt, load);
        __builtin_amdgcn_wave_barrier();
#pragma unroll 16
        for (int i = 0; i < 256; i += 4) {
            const f4v v = *(const f4v *)&st.v[half][i];
            s = __fadd_rn(s, v.x);
            found = (found < 0 && s > bound) ? base + i : found;
            s = __fadd_rn(s, v.y);
            found = (found < 0 && s > bound) ? base + i + 1 : found;
            s = __fadd_rn(s, v.z);
            found = (found < 0 && s > bound) ? base + i + 2 : found;
            s = __fadd_rn(s, v.w);
            found = (found < 0 && s > bound) ? base + i + 3 : found;
        }
    }
    return (found >= 0 && found < cnt) ? found : -1;
}

// Sum of one int per thread over the workgroup, to every thread. scratch: ST / 64 ints.
__device__ __forceinline__ int block_sum(int v, int *scratch) {
    const int tid = threadIdx.x;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    __syncthreads();  // scratch may still be read from an earlier call
    if ((tid & 63) == 0) scratch[tid >> 6] = v;
    __syncthreads();
    int t = 0;
#pragma unroll
    for (int w = 0; w < ST / 64; w++) t += scratch[w];
    return t;
}

// Exclusive prefix sum of one int per thread over the workgroup; *total gets the sum. scratch: ST / 64 + 1 ints.
__device__ __forceinline__ int block_exclusive_scan(int v, int *scratch, int *total) {
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    int inc = v;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const int o = __shfl_up(inc, off, 64);
        if (lane >= off) inc += o;
    }
    __syncthreads();  // scratch may still be read from an earlier call
    if (lane == 63) scratch[wave] = inc;
    __syncthreads();
    if (tid == 0) {
        int run = 0;
        for (int w = 0; w < ST / 64; w++) {
            const int t = scratch[w];
            scratch[w] = run;
            run += t;
        }
        scratch[ST / 64] = run;
    }
    __syncthreads();
    *total = scratch[ST / 64];
    return scratch[wave] + inc - v;
}

// Keeps, in order, the entries of a list for which keep(j) holds: thread t owns a contiguous stretch of positions.
// src_idx == nullptr: the list is the whole row and position = token id. Returns the new length (to every thread).
template <class K>
__device__ __forceinline__ int compact(int cnt, const float *src_val, const int32_t *src_idx, float *dst_val, int32_t *dst_idx,
                                       int *scratch, K keep) {
    const int per = (cnt + ST - 1) / ST, j0 = min(cnt, (int)threadIdx.x * per), j1 = min(cnt, j0 + per);
    int mine = 0;
    for (int j = j0; j < j1; j++) mine += keep(j) ? 1 : 0;
    int total;
    int at = block_exclusive_scan(mine, scratch, &total);
    for (int j = j0; j < j1; j++)
        if (keep(j)) {
            dst_val[at] = src_val[j];
            dst_idx[at] = src_idx ? src_idx[j] : j;
            at++;
        }
    __syncthreads();
    return total;
}

__global__ void __launch_bounds__(ST) sample_rows_kernel(const float *__restrict__ logits, int n, int n_pad,
                                                         const float *__restrict__ temperature, const int32_t *__restrict__ top_k,
                                                         const float *__restrict__ top_p, const float *__restrict__ uniform,
                                                         float *__restrict__ f_ws, int32_t *__restrict__ i_ws,
                                                         unsigned long long *__restrict__ keys_ws, int32_t *__restrict__ out) {
    const int row = blockIdx.x, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const float *x = logits + (size_t)row * n;
    float *p = f_ws + (size_t)row * 3 * n, *va = p + n, *vb = va + n;   // probabilities; two compacted value lists
    int32_t *ia = i_ws + (size_t)row * 3 * n, *ib = ia + n, *flags = ib + n;
    unsigned long long *keys = keys_ws + (size_t)row * n_pad;
    __shared__ float s_f[ST / 64];
    __shared__ int s_i[ST / 64 + 1];
    __shared__ float s_val;
    __shared__ int s_int;
    __shared__ __attribute__((aligned(16))) WalkStage s_stage;
    const float T = temperature[row];

    // ---- maximum (and, for temperature 0, its first index: Argmax, sampler.go:80-91)
    float bv = -FLT_MAX;
    int bi = 0;
    for (int j = tid; j < n; j += ST) {
        const float v = (T == 0.f) ? x[j] : __fdiv_rn(x[j], T);
        if (v > bv) {
            bv = v;
            bi = j;
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, 64);
        const int oi = __shfl_xor(bi, off, 64);
        if (ov > bv || (ov == bv && oi < bi)) {
            bv = ov;
            bi = oi;
        }
    }
    if (lane == 0) {
        s_f[wave] = bv;
        s_i[wave] = bi;
    }
    __syncthreads();
    if (tid == 0) {
        for (int i = 1; i < ST / 64; i++)
            if (s_f[i] > bv || (s_f[i] == bv && s_i[i] < bi)) {
                bv = s_f[i];
                bi = s_i[i];
            }
        s_val = bv;
        s_int = (bv > -FLT_MAX) ? bi : 0;
    }
    __syncthreads();
    if (T == 0.f) {
        if (tid == 0) out[row] = s_int;
        return;
    }
    const float mx = s_val;
    __syncthreads();

    // ---- softmax (sampler.go:94-117): exp in float64, the sum in index order, one division per element
    for (int j = tid; j < n; j += ST) p[j] = (float)exp((double)__fsub_rn(__fdiv_rn(x[j], T), mx));
    __syncthreads();
    if (wave == 0) {
        const float s = sum_in_order(n, [&](int i) { return p[i]; }, s_stage);
        if (lane == 0) s_val = s;
    }
    __syncthreads();
    {
        const float s = s_val;
        for (int j = tid; j < n; j += ST) p[j] = __fdiv_rn(p[j], s);
    }
    __syncthreads();

    // The surviving entries as a list (values, token ids) in index order; entries that were set to 0 add nothing
    // to any later sum, so leaving them out changes no result. Before any cut the list is the row itself.
    const float *val = p;
    const int32_t *idx = nullptr;
    int cnt = n;

    // ---- top-k (sampler.go:120-146): the k-th largest value by selection over the float bits
    const int k = top_k[row];
    if (k > 0 && k < n) {
        // bit by bit from the top: how many candidates (entries that match the bits decided so far) have this
        // bit set; if at least `want`, the k-th largest has it too, otherwise those larger ones are passed over
        unsigned int prefix = 0;
        int want = k;
        for (int b = 30; b >= 0; b--) {
            const unsigned int cand = prefix | (1u << b), care = ~((1u << b) - 1u);
            int c = 0;
            for (int j = tid; j < n; j += ST) c += ((__float_as_uint(p[j]) & care) == cand) ? 1 : 0;
            const int total = block_sum(c, s_i);
            if (total >= want)
                prefix = cand;
            else
                want -= total;
        }
        const float threshold = __uint_as_float(prefix);
        cnt = compact(n, p, nullptr, va, ia, s_i, [&](int j) { return !(p[j] < threshold); });
        if (wave == 0) {
            const float s = sum_in_order(cnt, [&](int i) { return va[i]; }, s_stage);
            if (lane == 0) s_val = s;
        }
        __syncthreads();
        const float s = s_val;
        if (s > 0.f)
            for (int j = tid; j < cnt; j += ST) va[j] = __fdiv_rn(va[j], s);
        __syncthreads();
        val = va;
        idx = ia;
    }

    // ---- top-p (sampler.go:149-189): descending order, ties by ascending index; walk until the sum passes p.
    // (The reference sorts the zeros too; they come last and add nothing, so the walk over the survivors ends
    // at the same place, and "never passed" keeps everything either way.)
    const float tp = top_p[row];
    if (tp > 0.f && tp < 1.0f) {
        int m = 2;
        while (m < cnt) m <<= 1;
        for (int j = tid; j < m; j += ST)
            keys[j] = j < cnt ? ((unsigned long long)(~__float_as_uint(val[j])) << 32) | (unsigned int)j : ~0ull;
        __syncthreads();
        for (int kk = 2; kk <= m; kk <<= 1) {
            for (int jj = kk >> 1; jj > 0; jj >>= 1) {
                for (int t = tid; t < m / 2; t += ST) {
                    const int i = 2 * t - (t & (jj - 1));  // the pair's lower position: bit jj clear
                    const int o = i + jj;
                    const unsigned long long a = keys[i], b = keys[o];
                    if ((a > b) == ((i & kk) == 0)) {
                        keys[i] = b;
                        keys[o] = a;
                    }
                }
                __syncthreads();
            }
        }
        if (wave == 0) {
            const int at = first_past(cnt, tp, [&](int i) { return __uint_as_float(~(unsigned int)(keys[i] >> 32)); }, s_stage);
            if (lane == 0) s_int = at < 0 ? cnt : at + 1;
        }
        __syncthreads();
        const int cutoff = s_int;
        for (int j = tid; j < cnt; j += ST) flags[(unsigned int)keys[j]] = j < cutoff ? 1 : 0;
        __syncthreads();
        const int kept = compact(cnt, val, idx, vb, ib, s_i, [&](int j) { return flags[j] != 0; });
        cnt = kept;
        if (wave == 0) {
            const float s = sum_in_order(cnt, [&](int i) { return vb[i]; }, s_stage);
            if (lane == 0) s_val = s;
        }
        __syncthreads();
        const float s = s_val;
        if (s > 0.f)
            for (int j = tid; j < cnt; j += ST) vb[j] = __fdiv_rn(vb[j], s);
        __syncthreads();
        val = vb;
        idx = ib;
    }

    // ---- the draw (sampler.go:192-204): first index whose cumulative sum exceeds r, else the last token
    if (wave == 0) {
        const int at = first_past(cnt, uniform[row], [&](int i) { return val[i]; }, s_stage);
        if (lane == 0) out[row] = at < 0 ? n - 1 : (idx ? idx[at] : at);
    }
}

}  // namespace

extern "C" {

int vx_sample_rows(vx_backend *be, const float *logits, int rows, int n, const float *temperature, const int32_t *top_k,
                   const float *top_p, const float *uniform, int32_t *out_idx) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(logits && temperature && top_k && top_p && uniform && out_idx, "vx_sample_rows: null pointer");
    VX_REQUIRE(rows >= 0 && n > 0 && n <= (1 << 24), "vx_sample_rows: bad shape %d x %d", rows, n);
    if (rows == 0) return VX_OK;
    int n_pad = 2;
    while (n_pad < n) n_pad <<= 1;
    // per row: three float lists and three int lists of n entries, n_pad 64-bit sort keys
    const size_t list_bytes = ((size_t)rows * 3 * n * 4 + 255) / 256 * 256;
    rc = ensure_ws(be, &be->sample_ws, &be->sample_ws_bytes, 2 * list_bytes + (size_t)rows * n_pad * 8, "sampling");
    if (rc) return rc;
    char *ws = (char *)be->sample_ws;
    sample_rows_kernel<<<rows, ST, 0, be->stream>>>(logits, n, n_pad, temperature, top_k, top_p, uniform, (float *)ws,
                                                   (int32_t *)(ws + list_bytes),
                                                   (unsigned long long *)(ws + 2 * list_bytes), out_idx);
    VX_CHECK_LAUNCH();
    return VX_OK;
}

}  // extern "C"
