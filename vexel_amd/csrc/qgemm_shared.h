// Declarations shared by the quantized GEMM translation units (qgemm.hip, qstream.hip).
#pragma once
#include "prep_tiles.h"

namespace vx {

// The sums of squares of a row's chunks, from which whoever consumes the activation's products takes 1/rms.
struct RowNorm {
    const float *sspart;  // [VX_PREP_SYNC_CHUNKS][VX_PREP_SYNC_ROWS], NULL when the rows carry no pending RMSNorm
    int n_chunks;
    float inv_k, eps;
};

__device__ __forceinline__ float wave_sum(float v) {
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// Factor of row r's finished dot products: the stored row factor times, for a pending RMSNorm, 1/rms from the
// chunks' sums of squares (added by a fixed butterfly over the wave, so every caller gets the same bits).
// Must be called by all 64 lanes of a wave.
__device__ __forceinline__ float row_factor(const float *__restrict__ inv_rows, const RowNorm &rn, int r) {
    float f = inv_rows[r];
    if (rn.sspart) {
        const int lane = threadIdx.x & 63;
        const float ss = wave_sum(lane < rn.n_chunks ? rn.sspart[lane * VX_PREP_SYNC_ROWS + r] : 0.f);
        const float rms = (float)sqrt((double)(ss * rn.inv_k + rn.eps));  // backend/cpu/cpu.go:214
        f = f / rms;
    }
    return f;
}

// What the Q|K|V launch needs to finish its rows itself (RoPE, the rotated Q to q_out, K and V into the paged
// pool: rope_store_partials_kernel's work) when one K slice holds the whole sum. q_out == NULL: not in use.
struct QkvEpi {
    float *q_out;
    void *pool;
    const int32_t *slots;
    const float2 *cs_tab;  // [row][head_dim / 2] (cos, sin) of the row's position
    RowNorm rn;
    int qd, kvd, head_dim, block_size, pool_f16;
};

// qstream.hip: the GEMMs over load-time packed copies of Q4_0 / Q8_0 / Q4_K / Q6_K matrices. w / n_end: up to nseg row
// segments of raw matrices (device addresses, cumulative row ends); served when every matrix in them has a packed
// copy (vx_qweight_pack), 2 <= M <= 64 and the shape fits. stream_gemm leaves the K slices' raw sums in
// be->part_ws as [slice][M][N] (*ks_out slices) or, given an epilogue, finishes the Q|K|V rows itself.
bool stream_gemm_ok(vx_backend *be, int fmt, const uint8_t *const *w, const int *n_end, int nseg, int N, int K, int M, bool epi);
int stream_gemm(vx_backend *be, int fmt, const uint8_t *const *w, const int *n_end, int nseg, int N, int K, int M, int mpad,
                const PrepView &pv, const QkvEpi *epi, int *ks_out);

// A Q|K|V group whose V matrix (format fb) differs from Q and K (format fa), each with a packed copy, in one launch:
// the K slices' raw sums of all three as [slice][M][nq + nk + nv] in be->part_ws.
bool stream_gemm_mixed_ok(vx_backend *be, int fa, const uint8_t *wq, const uint8_t *wk, int nq, int nk, int fb, const uint8_t *wv,
                          int nv, int K, int M);
int stream_gemm_mixed(vx_backend *be, int fa, const uint8_t *wq, const uint8_t *wk, int nq, int nk, int fb, const uint8_t *wv, int nv,
                      int K, int M, int mpad, const PrepView &pv, int *ks_out);

// More than 64 rows over the same packed copies. With one K slice and to_partials false the finished rows (row
// factors, residual) go to out; otherwise the slices' sums to be->part_ws, *ks_out of them.
bool tiles_gemm_ok(vx_backend *be, int fmt, const uint8_t *const *w, const int *n_end, int nseg, int N, int K, int M);
int tiles_gemm(vx_backend *be, int fmt, const uint8_t *const *w, const int *n_end, int nseg, int N, int K, int M, int mpad,
               const PrepView &pv, float *out, const float *residual, bool to_partials, int *ks_out,
               const RowNorm *fin_norm = nullptr);  // fin_norm (to_partials only): a pending 1/rms the launch folds into pv.inv_scale

}  // namespace vx
