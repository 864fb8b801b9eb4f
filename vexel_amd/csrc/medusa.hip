// Medusa prediction heads (inference/medusa/heads.go:83-171): logits_h = SiLU(hidden . FC1_h) . FC2_h for every
// head h, and the k largest logits of a row. The weights are float32 [in, out] matrices, read once per call whatever
// the number of hidden rows (<= 8): the work is streaming FC2 (hidden x vocab floats per head) from HBM.
#include <float.h>

#include "common.h"

using namespace vx;

namespace {

constexpr int KN_THREADS = 256;  // 4 waves; a wave's lane owns 4 consecutive output columns
constexpr int KN_COLS = 256;     // columns per workgroup
constexpr int KN_MAX_ROWS = 8;

typedef float f4 __attribute__((ext_vector_type(4)));

// P[split][head][m][n] = sum over the split's k range of a[head or 0][m][k] * B[head][k][n].
// grid = (column tiles, splits, heads). Wave w of the workgroup takes the rows k0 + w, k0 + w + 4, ... of the
// split; the four waves' sums are added through LDS in wave order.
template <int M>
__global__ void __launch_bounds__(KN_THREADS) kn_partial_kernel(const float *__restrict__ a, size_t a_head_stride,
                                                                const float *__restrict__ B, float *__restrict__ P,
                                                                int rows, int K, int N, int k_per_split) {
    __shared__ f4 red[3][M][64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // scalar: the loads of `a` become scalar loads
    const int head = blockIdx.z, split = blockIdx.y;
    const int col = blockIdx.x * KN_COLS + lane * 4;
    const bool live = col < N;  // N is a multiple of 4: a live lane's 4 columns exist
    const int k0 = split * k_per_split, k1 = min(K, k0 + k_per_split);
    const float *ah = a + (size_t)head * a_head_stride;
    const float *Bh = B + (size_t)head * K * N + (live ? col : 0);
    f4 acc[M];
#pragma unroll
    for (int m = 0; m < M; m++) acc[m] = (f4){0.f, 0.f, 0.f, 0.f};
    int k = k0 + wave;
    for (; k + 12 < k1; k += 16) {  // four rows in flight
        f4 b[4];
#pragma unroll
        for (int u = 0; u < 4; u++) b[u] = *(const f4 *)(Bh + (size_t)(k + 4 * u) * N);
#pragma unroll
        for (int u = 0; u < 4; u++)
#pragma unroll
            for (int m = 0; m < M; m++) {
                const float av = ah[(size_t)min(m, rows - 1) * K + k + 4 * u];
                acc[m] += av * b[u];
            }
    }
    for (; k < k1; k += 4) {
        const f4 b = *(const f4 *)(Bh + (size_t)k * N);
#pragma unroll
        for (int m = 0; m < M; m++) acc[m] += ah[(size_t)min(m, rows - 1) * K + k] * b;
    }
    if (wave > 0) {
#pragma unroll
        for (int m = 0; m < M; m++) red[wave - 1][m][lane] = acc[m];
    }
    __syncthreads();
    if (wave == 0 && live) {
#pragma unroll
        for (int m = 0; m < M; m++) {
            f4 t = acc[m];
            t += red[0][m][lane];
            t += red[1][m][lane];
            t += red[2][m][lane];
            if (m < rows) *(f4 *)(P + (((size_t)split * gridDim.z + head) * rows + m) * N + col) = t;
        }
    }
}

// out[head][m][n] = act(sum over splits, in split order, of P[split][head][m][n]); total = heads * rows * N
template <bool SILU>
__global__ void kn_reduce_kernel(const float *__restrict__ P, float *__restrict__ out, int splits, size_t total) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    float t = 0.f;
    int s = 0;
    for (; s + 4 <= splits; s += 4) {  // four loads in flight, added in split order
        const float p0 = P[(size_t)s * total + i], p1 = P[(size_t)(s + 1) * total + i];
        const float p2 = P[(size_t)(s + 2) * total + i], p3 = P[(size_t)(s + 3) * total + i];
        t += p0;
        t += p1;
        t += p2;
        t += p3;
    }
    for (; s < splits; s++) t += P[(size_t)s * total + i];
    if (SILU) t = t / (1.0f + (float)exp((double)(-t)));  // heads.go:20-22
    out[i] = t;
}

// The k largest values of a row and their indices, largest first, ties to the lower index (heads.go:146-171,
// tree.go:242-271). One workgroup per row; round r takes the largest element that comes after round r-1's in that
// order. Values that are not above -FLT_MAX (and NaN) are never taken: the index is then -1 and the value -FLT_MAX.
__global__ void __launch_bounds__(1024) topk_rows_kernel(const float *__restrict__ x, int n, int k, int32_t *__restrict__ idx,
                                                         float *__restrict__ val) {
    __shared__ float sv[16];
    __shared__ int si[16];
    __shared__ float pick_v;
    __shared__ int pick_i;
    const float *xr = x + (size_t)blockIdx.x * n;
    float pv = INFINITY;
    int pi = -1;
    for (int r = 0; r < k; r++) {
        float bv = -FLT_MAX;
        int bi = -1;
        for (int j = threadIdx.x; j < n; j += blockDim.x) {
            const float v = xr[j];
            const bool after = v < pv || (v == pv && j > pi);
            if (after && v > bv) {  // ascending j: a tie keeps the lower index
                bv = v;
                bi = j;
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const float ov = __shfl_xor(bv, off, 64);
            const int oi = __shfl_xor(bi, off, 64);
            if (oi >= 0 && (bi < 0 || ov > bv || (ov == bv && oi < bi))) {
                bv = ov;
                bi = oi;
            }
        }
        const int w = threadIdx.x >> 6, l = threadIdx.x & 63;
        if (l == 0) {
            sv[w] = bv;
            si[w] = bi;
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            for (int i = 1; i < (int)(blockDim.x >> 6); i++)
                if (si[i] >= 0 && (bi < 0 || sv[i] > bv || (sv[i] == bv && si[i] < bi))) {
                    bv = sv[i];
                    bi = si[i];
                }
            idx[(size_t)blockIdx.x * k + r] = bi;
            if (val) val[(size_t)blockIdx.x * k + r] = bi >= 0 ? bv : -FLT_MAX;
            pick_v = bv;
            pick_i = bi;
        }
        __syncthreads();
        // nothing left: the remaining rounds find nothing either (pv = -FLT_MAX excludes every candidate)
        pv = pick_i >= 0 ? pick_v : -FLT_MAX;
        pi = pick_i >= 0 ? pick_i : n;
    }
}

int choose_splits(int col_tiles, int heads, int K) {
    // enough workgroups to fill the chip several times over, at least 64 rows of k per split
    int splits = 1;
    while (col_tiles * heads * splits < 2048 && K / (splits * 2) >= 64) splits *= 2;
    return splits;
}

template <int M>
void launch_partial(vx_backend *be, const float *a, size_t a_head_stride, const float *B, float *P, int rows, int heads, int K,
                    int N, int splits) {
    const int kps = ceil_div(ceil_div(K, splits), 4) * 4;
    dim3 grid(ceil_div(N, KN_COLS), splits, heads);
    kn_partial_kernel<M><<<grid, KN_THREADS, 0, be->stream>>>(a, a_head_stride, B, P, rows, K, N, kps);
}

// out[head][rows][N] = act(a . B[head]) with a = a[rows][K] (a_head_stride 0) or a[head][rows][K]
int kn_matmul(vx_backend *be, const float *a, size_t a_head_stride, const float *B, float *out, int rows, int heads, int K,
              int N, bool silu) {
    const int splits = choose_splits(ceil_div(N, KN_COLS), heads, K);
    const size_t total = (size_t)heads * rows * N;
    int rc = ensure_ws(be, &be->part_ws, &be->part_ws_bytes, (size_t)splits * total * sizeof(float), "Medusa partial sums");
    if (rc) return rc;
    float *P = (float *)be->part_ws;
    if (rows == 1) launch_partial<1>(be, a, a_head_stride, B, P, rows, heads, K, N, splits);
    else if (rows == 2) launch_partial<2>(be, a, a_head_stride, B, P, rows, heads, K, N, splits);
    else if (rows <= 4) launch_partial<4>(be, a, a_head_stride, B, P, rows, heads, K, N, splits);
    else launch_partial<8>(be, a, a_head_stride, B, P, rows, heads, K, N, splits);
    VX_CHECK_LAUNCH();
    const int blocks = (int)((total + 255) / 256);
    if (silu) kn_reduce_kernel<true><<<blocks, 256, 0, be->stream>>>(P, out, splits, total);
    else kn_reduce_kernel<false><<<blocks, 256, 0, be->stream>>>(P, out, splits, total);
    VX_CHECK_LAUNCH();
    return VX_OK;
}

}  // namespace

extern "C" {

int vx_medusa_forward(vx_backend *be, const float *hidden, const float *fc1, const float *fc2, float *intermediate,
                      float *logits, int rows, int num_heads, int hidden_size, int vocab_size) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(hidden && fc1 && fc2 && intermediate && logits, "vx_medusa_forward: null pointer");
    VX_REQUIRE(rows >= 0 && rows <= KN_MAX_ROWS, "vx_medusa_forward: %d rows (at most %d)", rows, KN_MAX_ROWS);
    VX_REQUIRE(num_heads >= 1 && hidden_size >= 1 && vocab_size >= 1, "vx_medusa_forward: bad shape");
    VX_REQUIRE(hidden_size % 4 == 0 && vocab_size % 4 == 0, "vx_medusa_forward: hidden %d and vocab %d must be multiples of 4",
               hidden_size, vocab_size);
    VX_REQUIRE(((uintptr_t)fc1 % 16) == 0 && ((uintptr_t)fc2 % 16) == 0, "vx_medusa_forward: weights must be 16-byte aligned");
    VX_REQUIRE((size_t)num_heads * rows * vocab_size <= (size_t)INT32_MAX, "vx_medusa_forward: output too large");
    if (rows == 0) return VX_OK;
    // intermediate[head][rows][hidden] = SiLU(hidden . FC1[head])                     heads.go:96-104
    rc = kn_matmul(be, hidden, 0, fc1, intermediate, rows, num_heads, hidden_size, hidden_size, true);
    if (rc) return rc;
    // logits[head][rows][vocab] = intermediate[head] . FC2[head]                     heads.go:106-114
    return kn_matmul(be, intermediate, (size_t)rows * hidden_size, fc2, logits, rows, num_heads, hidden_size, vocab_size,
                     false);
}

int vx_topk_rows(vx_backend *be, const float *x, int rows, int n, int k, int32_t *out_idx, float *out_val) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(x && out_idx && rows >= 0 && n >= 1 && k >= 0, "vx_topk_rows: bad arguments");
    VX_REQUIRE(k <= n, "vx_topk_rows: k %d exceeds the row length %d", k, n);
    VX_REQUIRE(k <= 256, "vx_topk_rows: k %d above 256 (the selection makes one pass over the row per pick)", k);
    if (rows == 0 || k == 0) return VX_OK;
    topk_rows_kernel<<<rows, 1024, 0, be->stream>>>(x, n, k, out_idx, out_val);
    VX_CHECK_LAUNCH();
    return VX_OK;
}

}  // extern "C"
