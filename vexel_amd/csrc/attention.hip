// Attention kernels.
//
//  * attn_generic_kernel: any head_dim <= 256, F32 or F16 K/V, three addressing modes
//    (head-major contiguous, token-major causal prefill, paged through a block table),
//    optional per-query kv length and optional tree mask. One workgroup per (query, head),
//    online softmax over chunks of positions. Serves Backend.SDPA, SDPAPrefill and the
//    single-sequence PagedKVOps methods.
//  * paged_decode_f16_kernel (+ paged_merge_kernel where the caller wants plain rows): the
//    batched-decode hot path. Ragged batch, F16 pool, one query per sequence, split over the KV
//    length so a launch has thousands of workgroups whatever the mix of context lengths.
//    HBM-bound: every K/V byte is read once with 16-byte loads, a token's head vector is one
//    contiguous 2*head_dim-byte run shared by head_dim/8 lanes. When the result goes on to the
//    output projection the kernel merges its own splits (the last workgroup of a chunk does it).
//  * paged_decode_gqa_kernel: the same for grouped queries (2 to 16 queries per K/V row, heads of 64 or
//    128) and for the batched tree attention's entries, on the f16 matrix cores; same splits, same merge.
//  * paged_mq_kernel: many query rows of one sequence over its paged F16 context (later prompt
//    chunks, linear verification), the grouped-query kernel's products with a tile of query rows
//    per wave; no LDS.
//  * prefill_fa2_kernel: tiled causal prefill (dense float32 K/V) and paged multi-query attention
//    for other block sizes on the f16 matrix cores (operands as two f16 halves), K/V tiles in LDS.
//
// Arithmetic: float32 dot products and accumulation (the matrix-core kernels: f16 products of
// two-halves operands, float32 accumulation), softmax through exp2 of the max-subtracted score; the CPU reference (backend/cpu/cpu.go:568-632) normalises the
// weights before the V accumulation, here the accumulator is divided once at the end.
#include <float.h>

#include "common.h"
#include "prep_tiles.h"

using namespace vx;

namespace {

constexpr float kLog2e = 1.4426950408889634f;

enum { MODE_CONTIG = 0, MODE_PREFILL = 1, MODE_PAGED = 2 };

struct AttnParams {
    const float *q;
    float *out;
    const void *k;  // contiguous / prefill: K base; paged: pool base
    const void *v;  // contiguous / prefill: V base; paged: unused
    int mode;
    int f16;
    int num_q_heads, num_kv_heads, head_dim;
    float scale;
    float softcap;  // > 0: scaled scores pass through softcap * tanh(score / softcap) (cpu.go:735-737)
    // contiguous
    int kv_head_stride;
    int kv_len;  // fixed kv length (contiguous, single paged decode); ignored when kv_lens != nullptr
    // paged
    const int32_t *block_table;          // one table (single sequence / multiquery / tree)
    const int32_t *const *bt_ptrs;       // per-query tables (batched), or nullptr
    const int32_t *bt_matrix;            // padded [rows,max_blocks] matrix, or nullptr
    const int32_t *bt_rows;              // row of each query in bt_matrix, or nullptr (row = query)
    int max_blocks;
    int block_size;
    const int32_t *kv_lens;              // per-query kv length (device), or nullptr
    // tree mask
    const uint8_t *tree_mask;
    int tree_base;
    int query_len;
};

__device__ __forceinline__ float ld_elem(const void *base, size_t idx, int f16) {
    return f16 ? (float)((const _Float16 *)base)[idx] : ((const float *)base)[idx];
}

constexpr int GEN_THREADS = 256;
constexpr int GEN_CHUNK = 1024;

__global__ void __launch_bounds__(GEN_THREADS) attn_generic_kernel(AttnParams p) {
    __shared__ float s_scores[GEN_CHUNK];
    __shared__ float s_red[GEN_THREADS / 64];
    __shared__ float s_acc[GEN_THREADS];
    __shared__ float s_q[256];

    const int h = blockIdx.x, qi = blockIdx.y, tid = threadIdx.x;
    const int D = p.head_dim;
    const int kvh = h / (p.num_q_heads / p.num_kv_heads);
    const size_t qoff = ((size_t)qi * p.num_q_heads + h) * D;

    int kv_len;
    const int32_t *bt = nullptr;
    if (p.mode == MODE_PREFILL) {
        kv_len = qi + 1;
    } else if (p.tree_mask) {
        kv_len = p.tree_base + p.query_len;
    } else {
        kv_len = p.kv_lens ? p.kv_lens[qi] : p.kv_len;
    }
    if (p.mode == MODE_PAGED) {
        if (p.bt_ptrs)
            bt = p.bt_ptrs[qi];
        else if (p.bt_matrix)
            bt = p.bt_matrix + (size_t)(p.bt_rows ? p.bt_rows[qi] : qi) * p.max_blocks;
        else
            bt = p.block_table;
    }
    for (int d = tid; d < D; d += GEN_THREADS) s_q[d] = p.q[qoff + d];
    __syncthreads();

    const size_t hs = (size_t)p.num_kv_heads * D;
    const size_t part = (size_t)p.block_size * hs;
    auto krow = [&](int pos) -> size_t {
        if (p.mode == MODE_CONTIG) return (size_t)kvh * p.kv_head_stride + (size_t)pos * D;
        if (p.mode == MODE_PREFILL) return ((size_t)pos * p.num_kv_heads + kvh) * D;
        return (size_t)bt[pos / p.block_size] * 2 * part + (size_t)(pos % p.block_size) * hs + (size_t)kvh * D;
    };
    const void *vbase = (p.mode == MODE_PAGED) ? p.k : p.v;
    const size_t vadd = (p.mode == MODE_PAGED) ? part : 0;

    // accumulation layout: thread t owns dimension t % D for the position subset t / D
    const int ng = (GEN_THREADS / D) > 0 ? (GEN_THREADS / D) : 1;
    const int my_d = tid % D, my_g = tid / D;
    const bool acc_active = my_g < ng && tid < ng * D;
    float acc = 0.f, m_run = -INFINITY, l_run = 0.f;

    for (int c0 = 0; c0 < kv_len; c0 += GEN_CHUNK) {
        int cn = min(GEN_CHUNK, kv_len - c0);
        float lmax = -INFINITY;
        for (int i = tid; i < cn; i += GEN_THREADS) {
            int pos = c0 + i;
            float sc;
            bool masked = p.tree_mask && pos >= p.tree_base &&
                          !p.tree_mask[(size_t)qi * p.query_len + (pos - p.tree_base)];
            if (masked) {
                sc = -INFINITY;
            } else {
                size_t kb = krow(pos);
                float dot = 0.f;
                for (int d = 0; d < D; d++) dot = fmaf(s_q[d], ld_elem(p.k, kb + d, p.f16), dot);
                sc = dot * p.scale;
                if (p.softcap > 0.f) sc = p.softcap * (float)tanh((double)(sc / p.softcap));
            }
            s_scores[i] = sc;
            lmax = fmaxf(lmax, sc);
        }
        // block max
        for (int off = 32; off > 0; off >>= 1) lmax = fmaxf(lmax, __shfl_xor(lmax, off, 64));
        __syncthreads();
        if ((tid & 63) == 0) s_red[tid >> 6] = lmax;
        __syncthreads();
        float cmax = fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3]));
        float m_new = fmaxf(m_run, cmax);
        float alpha = (m_run == -INFINITY) ? 0.f : exp2f((m_run - m_new) * kLog2e);
        float lsum = 0.f;
        for (int i = tid; i < cn; i += GEN_THREADS) {
            float sc = s_scores[i];
            float e = (sc == -INFINITY) ? 0.f : exp2f((sc - m_new) * kLog2e);
            s_scores[i] = e;
            lsum += e;
        }
        for (int off = 32; off > 0; off >>= 1) lsum += __shfl_xor(lsum, off, 64);
        __syncthreads();
        if ((tid & 63) == 0) s_red[tid >> 6] = lsum;
        __syncthreads();
        float csum = s_red[0] + s_red[1] + s_red[2] + s_red[3];
        l_run = l_run * alpha + csum;
        m_run = m_new;
        acc *= alpha;
        if (acc_active) {
            for (int i = my_g; i < cn; i += ng) {
                float w = s_scores[i];
                if (w != 0.f) acc = fmaf(w, ld_elem(vbase, krow(c0 + i) + vadd + my_d, p.f16), acc);
            }
        }
        __syncthreads();
    }
    s_acc[tid] = acc_active ? acc : 0.f;
    __syncthreads();
    if (tid < D) {
        float t = 0.f;
        for (int g = 0; g < ng; g++) t += s_acc[g * D + tid];
        p.out[qoff + tid] = (l_run > 0.f) ? t / l_run : 0.f;
    }
}

// --------------------------------------------------------------------------------------------
// Hot path: ragged batched decode over an F16 paged pool with 16-token blocks.
//
// grid = (num_kv_heads, splits, batch); block = 256 threads (4 waves).
// A workgroup owns the tokens [split*TPW, min(kv_len,(split+1)*TPW)) of one (sequence, kv head)
// and all G = Hq/Hkv query heads that share that kv head. A wave takes 16-token pool blocks
// round-robin. Within a wave LPT = D/8 lanes hold one token's head vector (8 halves = 16 bytes
// each), so one load instruction covers TPI = 64/LPT tokens and a block needs NL = 16/TPI K loads
// and as many V loads. The block id is wave-uniform (scalar load); all 2*NL loads of the next
// block are in flight while the current block is reduced.
// Partials (m, l, acc[D]) per (sequence, q head, split) go to a scratch buffer; paged_merge_kernel
// combines the splits, or the kernel itself does (MergeOut).
constexpr int TPW = ATTN_TPW;  // tokens per workgroup (smaller, a kernel argument, for batches that would not fill the chip)
constexpr int HOT_BS = 16;

// x = h + l in two f16 halves. The float32 value, its rounded half and their difference each pass through a register
// of their own: left to itself the compiler folds the operations that produced x into mixed-precision
// multiply-adds that round once from the unrounded product, and the halves then add up to less than x's 24 bits
// (measured: attention outputs off by 3e-5 instead of 1e-6).
struct HalfPair { _Float16 h, l; };
__device__ __forceinline__ HalfPair split_hl(float x) {
    asm volatile("" : "+v"(x));
    HalfPair r;
    r.h = (_Float16)x;
    float hf = (float)r.h;
    asm volatile("" : "+v"(hf));
    float d = x - hf;
    asm volatile("" : "+v"(d));
    r.l = (_Float16)d;
    return r;
}
typedef float float4v __attribute__((ext_vector_type(4)));

// A read of K/V pool bytes that a launch reads once (the decode kernels: one workgroup per KV head and token range):
// the non-temporal form does not keep the line in the die's L2 and streams measurably faster (570 MB: 6.6 - 6.7 TB/s
// against 5.9 with plain loads). Not for bytes that several workgroups or two instructions share a line of (the
// multi-query kernel's rows, weight units of 32 bytes per lane, head vectors of 160 or 192 bytes, whose lines straddle
// the heads of neighbouring workgroups): those measured slower with it.
template <bool NT = true, class T> __device__ __forceinline__ T stream_load(const T *p) {
    if constexpr (NT) return __builtin_nontemporal_load(p);
    else return *p;
}

// Sum over the N adjacent lanes (N = 8, 16 or 32, aligned) that hold one token's head vector, by DPP inside a
// 16-lane row (no LDS traffic): quads, then the mirrored quad of the half, then the mirrored half; heads of 256
// span two rows, joined by one cross-row exchange.
template <int N>
__device__ __forceinline__ float token_sum(float t) {
    static_assert(N == 8 || N == 16 || N == 32, "a head vector spans 8, 16 or 32 lanes");
    t += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, t), 0xb1, 0xf, 0xf, false));   // quad_perm [1,0,3,2]
    t += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, t), 0x4e, 0xf, 0xf, false));   // quad_perm [2,3,0,1]
    t += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, t), 0x141, 0xf, 0xf, false));  // row_half_mirror
    if (N >= 16) t += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, t), 0x140, 0xf, 0xf, false));  // row_mirror
    if (N == 32) t += __shfl_xor(t, 16, 64);
    return t;
}

// Where the workgroup that finishes a sequence's 256-column chunk last leaves the chunk merged over its splits,
// as the prepared activation of the output projection (cnt == nullptr: nobody merges, the partial sums are the
// result). cnt[sequence * units + unit] counts the arrivals and is zero again when the launch ends.
// The unit of the in-kernel merge for workgroups of GD = G * D output columns: the fewest KV heads whose columns are
// a whole number of 256-column chunks (HPC of them, CH chunks).
constexpr int gcd_c(int a, int b) { return b == 0 ? a : gcd_c(b, a % b); }
template <int GD>
struct MergeUnit {
    static constexpr int HPC = 256 / gcd_c(GD, 256);
    static constexpr int CH = HPC * GD / 256;
};

struct MergeOut {
    PrepView pv;
    int32_t *cnt = nullptr;
    int mpad = 0;
    float *plain = nullptr;  // != nullptr: the merged rows as plain float32 [row][heads * D] instead (a single row's matrix-vector product reads that)
};

// The wave's 256 merged columns (chunk c of row `row`, four per lane): as a chunk of the prepared operand or as floats.
__device__ __forceinline__ void put_merged(const MergeOut &mg, int row, int c, const float (&y)[4], int K) {
    const int lane = threadIdx.x & 63;
    if (mg.plain) {
        *(float4 *)(mg.plain + (size_t)row * K + c * 256 + lane * 4) = make_float4(y[0], y[1], y[2], y[3]);
        return;
    }
    write_chunk(mg.pv, row, c, y, mg.mpad);
    if (c == 0 && lane == 0) mg.pv.inv_scale[row] = 1.f;
}

// What follows once each of the workgroup's 4 waves has left its (m, l, acc) of the G*RG queries in LDS: the waves'
// sums are combined, written as the split's partial sums and, with mg.cnt, merged over the splits by the workgroup
// that arrives last at its chunk of 256 output columns.
template <int D, int G, int RG>
__device__ __forceinline__ void finish_split(const float (&s_m)[4][G * RG], const float (&s_l)[4][G * RG],
                                             const float (&s_acc)[4][G * RG][D], float *__restrict__ partial, int seq,
                                             int kvh, int split, int kv_len, int num_q_heads, int num_kv_heads,
                                             int max_splits, const MergeOut &mg, int tps) {
    constexpr int GG = G * RG;
    constexpr int GD = G * D;                          // this workgroup's columns of the output
    constexpr bool MERGES = RG == 1;
    constexpr int CH = MergeUnit<GD>::CH;    // 256-column chunks of a merge unit
    constexpr int HPC = MergeUnit<GD>::HPC;  // kv heads of a merge unit
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    __syncthreads();
    for (int idx = tid; idx < GG * D; idx += 256) {
        const int g = idx / D, d = idx % D;
        float M = fmaxf(fmaxf(s_m[0][g], s_m[1][g]), fmaxf(s_m[2][g], s_m[3][g]));
        float L = 0.f, A = 0.f;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const float f = (s_m[w][g] == -INFINITY) ? 0.f : exp2f(s_m[w][g] - M);
            L += s_l[w][g] * f;
            A += s_acc[w][g][d] * f;
        }
        const int qh = kvh * G + g % G;
        float *po = partial + ((((size_t)seq * RG + g / G) * num_q_heads + qh) * max_splits + split) * (D + 2);
        // (device-scope stores: written through to where a workgroup on another die reads them, see below)
        __hip_atomic_store(po + 2 + d, A, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (d == 0) {
            __hip_atomic_store(po, M, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(po + 1, L, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    // The last workgroup to arrive at a (sequence, chunk of 256 output columns) merges the chunk's splits in
    // index order - the sums do not depend on who that is - and writes it as the next GEMM's operand.
    if constexpr (MERGES) {
        if (!mg.cnt) return;
        // Ordering without device-wide cache write-backs and invalidations (a release / acquire fence pair at
        // device scope costs this kernel several times its run time: every workgroup would flush and drop its
        // die's L2): the partial sums above are device-scope stores and are read back by device-scope loads, which
        // the dies' caches do not hold back or serve stale; each wave waits until its stores are acknowledged
        // before the workgroup's barrier, thread 0 counts the arrival after the barrier, and whoever counts the
        // last one reads only after that atomic has returned.
        // This is an argument about gfx950's memory system (device-scope accesses are served by the home die's
        // memory-side L2, and a store is acknowledged once it is visible there), not about the HIP memory model,
        // which would ask for the fences: other targets must not compile it. vx_backend_set_attn_merge(be, 0) /
        // VEXEL_HIP_NO_ATTN_MERGE select the separate merge launch, which needs none of this.
#if defined(__HIP_DEVICE_COMPILE__) && !defined(__gfx950__)
#error "the in-kernel merge of the attention splits is ordered for gfx950 only"
#endif
        __shared__ int s_last;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        const int ns = (kv_len + tps - 1) / tps;  // workgroups of one kv head that arrive for this sequence
        const int unit = kvh / HPC;
        if (tid == 0) {
            int32_t *cnt = mg.cnt + (size_t)seq * (num_kv_heads / HPC) + unit;
            const int last = __hip_atomic_fetch_add(cnt, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == ns * HPC - 1;
            if (last) __hip_atomic_store(cnt, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // (nobody else comes before the next launch)
            s_last = last;
        }
        __syncthreads();
        if (!s_last) return;
        for (int ch = wave; ch < CH; ch += 4) {
            const int c = unit * CH + ch;
            float y[4];
            split_merge4<true>(partial, ns, num_q_heads, D, max_splits, seq, c * 256 + lane * 4, y);
            put_merged(mg, seq, c, y, num_q_heads * D);
        }
    }
}

// RG > 1: an entry of the batch is RG consecutive query rows that share one sequence's context (the rows of a
// candidate tree): the workgroup serves the G*RG queries (row, head) of its kv head from one pass over the K/V.
// One item of the work: the tokens of split `split` of sequence `seq` for kv head `kvh` (all of the workgroup).
template <int D, int G, int RG>
__device__ __forceinline__ void paged_decode_f16_item(
    const float *__restrict__ q, const _Float16 *__restrict__ pool, const int32_t *__restrict__ bt_matrix, int max_blocks,
    float *__restrict__ partial, int num_q_heads, int num_kv_heads, float scale, int max_splits, const MergeOut &mg, int tps,
    const int kvh, const int split, const int seq, int kv_len, const int row) {
    constexpr int GG = G * RG;       // queries per K/V row
    constexpr int DL = D / 8;        // 8-element slices of a head vector
    // lanes per token: the next power of two; the lanes past DL (heads of 80 or 96) repeat the last slice's loads
    // with a zero query, so they add nothing and write nothing
    constexpr int LPT = DL <= 8 ? 8 : (DL <= 16 ? 16 : 32);
    static_assert(D % 8 == 0 && DL <= 32, "head vectors are whole 16-byte slices on at most 32 lanes");
    constexpr int TPI = 64 / LPT;    // tokens per load instruction
    constexpr int NL = HOT_BS / TPI; // load instructions per block and per K or V
    typedef _Float16 half8 __attribute__((ext_vector_type(8)));
    // The caller's max_kv_len sized the partial sums (max_splits per sequence and head). A length above it is
    // attended over its first max_splits * TPW tokens by every kernel of the path alike: defined, and inside the
    // buffers.
    kv_len = min(kv_len, max_splits * tps);  // (tps: tokens per split, a multiple of the block size)
    const int t_begin = split * tps;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    constexpr int GD = G * D;                          // this workgroup's columns of the output
    constexpr bool MERGES = RG == 1;
    constexpr int CH = MergeUnit<GD>::CH;    // 256-column chunks of a merge unit
    constexpr int HPC = MergeUnit<GD>::HPC;  // kv heads of a merge unit
    if (split >= max_splits || t_begin >= kv_len) {
        // a sequence without tokens has nobody to merge for it: zeros, as the merge of no splits gives
        if constexpr (MERGES) {
            if (mg.cnt && kv_len == 0 && split == 0 && kvh % HPC == 0) {
                const float zero[4] = {0.f, 0.f, 0.f, 0.f};
                for (int ch = wave; ch < CH; ch += 4) put_merged(mg, seq, kvh / HPC * CH + ch, zero, num_q_heads * D);
            }
        }
        return;
    }
    const int t_end = min(kv_len, t_begin + tps);
    const int32_t *bt = bt_matrix + (size_t)row * max_blocks + t_begin / HOT_BS;

    const int tl = lane / LPT;  // token slot within a load
    const int dl = DL == LPT ? lane % LPT : min(lane % LPT, DL - 1);  // 8-element slice of the head vector
    const bool live = DL == LPT ? true : lane % LPT < DL;
    const size_t hs = (size_t)num_kv_heads * D;
    const size_t part = (size_t)HOT_BS * hs;
    const size_t lane_off = (size_t)tl * hs + (size_t)kvh * D + dl * 8;

    // query slices, pre-multiplied by scale*log2(e) so scores are in the exp2 domain
    float qf[GG][8];
    const float qs = scale * kLog2e;
#pragma unroll
    for (int g = 0; g < GG; g++) {
        const float *qp = q + (((size_t)seq * RG + g / G) * num_q_heads + (size_t)kvh * G + g % G) * D + dl * 8;
#pragma unroll
        for (int e = 0; e < 8; e++) qf[g][e] = live ? qp[e] * qs : 0.f;
    }
    float acc[GG][8], m_run[GG], l_run[GG];
#pragma unroll
    for (int g = 0; g < GG; g++) {
        m_run[g] = -INFINITY;
        l_run[g] = 0.f;
#pragma unroll
        for (int e = 0; e < 8; e++) acc[g][e] = 0.f;
    }

    const int n_blocks = (t_end - t_begin + HOT_BS - 1) / HOT_BS;
    half8 kk[NL], vv[NL], kn[NL], vn[NL];
    auto issue = [&](int bi, half8 *kd, half8 *vd) {
        const int blk = __builtin_amdgcn_readfirstlane(bt[bi]);
        const _Float16 *base = pool + (size_t)blk * 2 * part + lane_off;
#pragma unroll
        for (int u = 0; u < NL; u++) {
            kd[u] = stream_load<D % 64 == 0>((const half8 *)(base + (size_t)u * TPI * hs));
            vd[u] = stream_load<D % 64 == 0>((const half8 *)(base + part + (size_t)u * TPI * hs));
        }
    };
    if (wave < n_blocks) issue(wave, kn, vn);
    for (int bi = wave; bi < n_blocks; bi += 4) {
#pragma unroll
        for (int u = 0; u < NL; u++) {
            kk[u] = kn[u];
            vv[u] = vn[u];
        }
        if (bi + 4 < n_blocks) issue(bi + 4, kn, vn);
        __builtin_amdgcn_sched_barrier(0);
        const int tok0 = t_begin + bi * HOT_BS + tl;
#pragma unroll
        for (int g = 0; g < GG; g++) {
            float s[NL];
            float gm = -INFINITY;
#pragma unroll
            for (int u = 0; u < NL; u++) {
                float t = 0.f;
#pragma unroll
                for (int e = 0; e < 8; e++) t = fmaf(qf[g][e], (float)kk[u][e], t);
                t = token_sum<LPT>(t);
                s[u] = (tok0 + u * TPI < t_end) ? t : -INFINITY;
                gm = fmaxf(gm, s[u]);
            }
            // max over the token slots of the wave (the block's first token is always valid)
#pragma unroll
            for (int off = LPT; off < 64; off <<= 1) gm = fmaxf(gm, __shfl_xor(gm, off, 64));
            const float m_new = fmaxf(m_run[g], gm);
            const float alpha = exp2f(m_run[g] - m_new);  // m_new is finite; exp2(-inf) = 0 on the first block
            m_run[g] = m_new;
            float lsum = 0.f;
#pragma unroll
            for (int e = 0; e < 8; e++) acc[g][e] *= alpha;
#pragma unroll
            for (int u = 0; u < NL; u++) {
                const bool ok = tok0 + u * TPI < t_end;
                const float pw = ok ? exp2f(s[u] - m_new) : 0.f;
                lsum += pw;
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const float vf = ok ? (float)vv[u][e] : 0.f;  // slots past the end may hold anything
                    acc[g][e] = fmaf(pw, vf, acc[g][e]);
                }
            }
            l_run[g] = l_run[g] * alpha + lsum;
        }
    }

    // combine token slots inside the wave (m is already wave-uniform per g)
#pragma unroll
    for (int g = 0; g < GG; g++) {
#pragma unroll
        for (int off = LPT; off < 64; off <<= 1) {
            l_run[g] += __shfl_xor(l_run[g], off, 64);
#pragma unroll
            for (int e = 0; e < 8; e++) acc[g][e] += __shfl_xor(acc[g][e], off, 64);
        }
    }

    // combine the 4 waves through LDS
    __shared__ float s_m[4][GG], s_l[4][GG];
    __shared__ float s_acc[4][GG][D];
    if (tl == 0 && live) {
#pragma unroll
        for (int g = 0; g < GG; g++) {
#pragma unroll
            for (int e = 0; e < 8; e++) s_acc[wave][g][dl * 8 + e] = acc[g][e];
            if (dl == 0) {
                s_m[wave][g] = m_run[g];
                s_l[wave][g] = l_run[g];
            }
        }
    }
    finish_split<D, G, RG>(s_m, s_l, s_acc, partial, seq, kvh, split, kv_len, num_q_heads, num_kv_heads, max_splits, mg, tps);
}

// grid = (kv heads, items or splits, 1 or sequences). With a work list a workgroup walks the items y, y + grid.y, ...;
// the grid's second dimension normally covers the most items the list can hold, so that every workgroup takes one
// item or none (the host cannot know how many the packing kernel listed; the empty workgroups are the grid's last and
// cost nothing measurable). A grid of just the workgroups the device holds at once, each walking several items
// (VEXEL_HIP_ATTN_WG_PER_CU=n), measured slower at 4, 5, 6 and 8 per compute unit (110.6 - 118.7 us against 105.5):
// the dispatcher hands the next item to whichever slot frees first, a fixed stride does not.
template <int D, int G, int RG = 1>
__global__ void __launch_bounds__(256) paged_decode_f16_kernel(
    const float *__restrict__ q, const _Float16 *__restrict__ pool, const int32_t *__restrict__ bt_matrix,
    const int32_t *__restrict__ bt_rows, int max_blocks, const int32_t *__restrict__ kv_lens,
    float *__restrict__ partial, int num_q_heads, int num_kv_heads, float scale, int max_splits,
    const int32_t *__restrict__ items, MergeOut mg, int tps) {
    const int kvh = blockIdx.x;
    if (items) {
        const int n = __builtin_amdgcn_readfirstlane(items[0]);
        for (int it = blockIdx.y; it < n; it += gridDim.y) {
            const int4 rec = ((const int4 *)(items + 4))[it];  // (sequence, split, kv length, table row)
            paged_decode_f16_item<D, G, RG>(q, pool, bt_matrix, max_blocks, partial, num_q_heads, num_kv_heads, scale, max_splits, mg,
                                            tps, kvh, rec.y, rec.x, rec.z, rec.w);
            __syncthreads();  // (the next item reuses the workgroup's LDS)
        }
    } else {
        const int seq = blockIdx.z;
        paged_decode_f16_item<D, G, RG>(q, pool, bt_matrix, max_blocks, partial, num_q_heads, num_kv_heads, scale, max_splits, mg, tps,
                                        kvh, blockIdx.y, seq, kv_lens[seq], bt_rows ? bt_rows[seq] : seq);
    }
}

// The same split of the work for grouped queries (G*RG = 2 .. 16 queries per K/V row) on the matrix cores: the vector
// form above repeats its multiply-adds, reductions and exponentials per query and is bound by them from G = 2 on.
// Per 16-token block a wave forms
//   S^T[token][query] = K Q^T   with v_mfma_f32_16x16x32_f16: A = K (exact f16), B = Q^T as hi + lo f16 halves of
//                               the row scaled by a power of two (so that the halves carry 22 bits of every element
//                               relative to the row's largest), D/32 steps x 2 halves;
//   O[query][d] += P V          with v_mfma_f32_16x16x16_f16: A = P as hi + lo halves of 2^10 p (p <= 1; the factor
//                               is carried as m - 10 in the partial sums), B = V (exact f16), D/16 tiles x 2 halves.
// The operand layouts are chosen so that nothing moves between lanes: as A operand, lane (c = lane % 16,
// g = lane / 16) holds row 4*(c % 4) + c / 4 of the block's K, so that the result's lane (query c, g) holds the
// scores of the tokens 4i + g, i = 0..3 - which is the A operand of the second product as it stands - and the
// V rows of exactly those tokens, D/16 columns from c * D/16 on, are what the same lane loads (for D = 128 the
// 16 bytes per lane of the vector form: whole rows per instruction); tile e of the output holds columns
// c * D/16 + e. K reaches its operand layout through the wave's own LDS rows. Rows of Q beyond G*RG are zero and
// their results are dropped.
template <int D, int G, int RG = 1>
__global__ void __launch_bounds__(256, 3) paged_decode_gqa_kernel(
    const float *__restrict__ q, const _Float16 *__restrict__ pool, const int32_t *__restrict__ bt_matrix,
    const int32_t *__restrict__ bt_rows, int max_blocks, const int32_t *__restrict__ kv_lens,
    float *__restrict__ partial, int num_q_heads, int num_kv_heads, float scale, int max_splits,
    const int32_t *__restrict__ items, MergeOut mg, int tps) {
    constexpr int GG = G * RG;
    static_assert(GG >= 1 && GG <= 16 && (D == 64 || D == 128), "up to 16 queries per K/V row, heads of 64 or 128");
    constexpr int NS = D / 32;  // steps of the first product (32 head elements each)
    constexpr int NT = D / 16;  // 16-column tiles of the output = halves per lane and token of V
    typedef _Float16 halfv __attribute__((ext_vector_type(NT)));
    typedef _Float16 half4 __attribute__((ext_vector_type(4)));
    const int kvh = blockIdx.x;
    int split = blockIdx.y, seq = blockIdx.z, kv_len, row;
    if (items) {
        if ((int)blockIdx.y >= items[0]) return;
        const int4 rec = ((const int4 *)(items + 4))[blockIdx.y];  // (sequence, split, kv length, table row)
        seq = rec.x;
        split = rec.y;
        kv_len = rec.z;
        row = rec.w;
    } else {
        kv_len = kv_lens[seq];
        row = bt_rows ? bt_rows[seq] : seq;
    }
    kv_len = min(kv_len, max_splits * tps);
    const int t_begin = split * tps;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    constexpr int GD = G * D;
    constexpr bool MERGES = RG == 1;
    constexpr int CH = MergeUnit<GD>::CH;    // 256-column chunks of a merge unit
    constexpr int HPC = MergeUnit<GD>::HPC;  // kv heads of a merge unit
    if (split >= max_splits || t_begin >= kv_len) {
        if constexpr (MERGES) {
            if (mg.cnt && kv_len == 0 && split == 0 && kvh % HPC == 0) {
                const float zero[4] = {0.f, 0.f, 0.f, 0.f};
                for (int ch = wave; ch < CH; ch += 4) put_merged(mg, seq, kvh / HPC * CH + ch, zero, num_q_heads * D);
            }
        }
        return;
    }
    const int t_end = min(kv_len, t_begin + tps);
    const int32_t *bt = bt_matrix + (size_t)row * max_blocks + t_begin / HOT_BS;
    const int c16 = lane & 15, g4 = lane >> 4;
    const size_t hs = (size_t)num_kv_heads * D;
    const size_t part = (size_t)HOT_BS * hs;

    const int n_blocks = (t_end - t_begin + HOT_BS - 1) / HOT_BS;
    // K is loaded as whole rows per instruction, the way V is (LPT lanes a row, TPI rows an instruction), and turned
    // into the A operand's layout - one row per 16 lanes, a quarter of it per lane group - through the wave's own
    // LDS rows: loading it in operand layout straight from the pool (16 bytes per lane at four places of every row)
    // measured 5 - 9 % slower.
    constexpr int LPT = D / 8, TPI = 64 / LPT;
    constexpr int KP = D + 8;  // halves per staged row
    __shared__ __attribute__((aligned(16))) _Float16 kst[4][HOT_BS * KP];
    const int tok_row = 4 * (c16 & 3) + (c16 >> 2);
    const size_t k_off = (size_t)(lane / LPT) * hs + (size_t)kvh * D + (lane % LPT) * 8;
    const size_t k_step = (size_t)TPI * hs;
    const size_t v_off = part + (size_t)g4 * hs + (size_t)kvh * D + c16 * NT;
    half8 kk[NS], kn[NS];
    halfv vv[4], vn[4];
    auto issue = [&](int bi, half8 *kd, halfv *vd) {
        const int blk = __builtin_amdgcn_readfirstlane(bt[bi]);
        const _Float16 *base = pool + (size_t)blk * 2 * part;
#pragma unroll
        for (int s = 0; s < NS; s++) kd[s] = stream_load((const half8 *)(base + k_off + k_step * s));
#pragma unroll
        for (int i = 0; i < 4; i++) vd[i] = stream_load((const halfv *)(base + v_off + (size_t)i * 4 * hs));  // token 4i + g4
    };
    // (the wave's first block is on its way while the query operand is built: the launch waits for K/V bytes)
    if (wave < n_blocks) issue(wave, kn, vn);
    __builtin_amdgcn_sched_barrier(0);
    // Q^T as the B operand: lane (query c16, head elements g4 * D/4 + 8s .. + 7 in step s), times scale * log2(e)
    // and the row's power of two, hi + lo
    half8 qh[NS], ql[NS];
    float q_inv;  // undoes the power of two on this lane's scores (query c16)
    {
        float x[NS][8];
        float amax = 0.f;
        const float qs = scale * kLog2e;
        const float *qp = q + (((size_t)seq * RG + c16 / G) * num_q_heads + (size_t)kvh * G + c16 % G) * D + g4 * (D / 4);
#pragma unroll
        for (int s = 0; s < NS; s++) {
            float4 a = make_float4(0.f, 0.f, 0.f, 0.f), b = a;
            if (c16 < GG) {
                a = *(const float4 *)(qp + 8 * s);
                b = *(const float4 *)(qp + 8 * s + 4);
            }
            const float t[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
            for (int e = 0; e < 8; e++) {
                x[s][e] = t[e] * qs;
                amax = fmaxf(amax, fabsf(x[s][e]));
            }
        }
        amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
        amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
        int ex = 11;
        if (amax > 0.f && amax < INFINITY) {
            (void)frexpf(amax, &ex);  // amax = mantissa in [0.5, 1) * 2^ex
            ex = max(ex, -60);
        }
        const float f = ldexpf(1.f, 11 - ex);  // the row's largest element lands in [1024, 2048)
        q_inv = ldexpf(1.f, ex - 11);
#pragma unroll
        for (int s = 0; s < NS; s++)
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const HalfPair t = split_hl(x[s][e] * f);
                qh[s][e] = t.h;
                ql[s][e] = t.l;
            }
    }
    float4v o[NT];
#pragma unroll
    for (int e = 0; e < NT; e++) o[e] = (float4v){0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;  // of query c16; l_run over this lane's tokens only until the end

    for (int bi = wave; bi < n_blocks; bi += 4) {
#pragma unroll
        for (int s = 0; s < NS; s++) *(half8 *)&kst[wave][(s * TPI + lane / LPT) * KP + (lane % LPT) * 8] = kn[s];
#pragma unroll
        for (int i = 0; i < 4; i++) vv[i] = vn[i];
        if (bi + 4 < n_blocks) issue(bi + 4, kn, vn);
        // (the wave's own rows: its LDS accesses stay in order, the compiler must keep them so)
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int s = 0; s < NS; s++) kk[s] = *(const half8 *)&kst[wave][tok_row * KP + g4 * (D / 4) + 8 * s];
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_sched_barrier(0);
        float4v sc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < NS; s++) {
            sc = __builtin_amdgcn_mfma_f32_16x16x32_f16(kk[s], qh[s], sc, 0, 0, 0);
            sc = __builtin_amdgcn_mfma_f32_16x16x32_f16(kk[s], ql[s], sc, 0, 0, 0);
        }
        const int tok0 = t_begin + bi * HOT_BS + g4;             // sc[i]: token tok0 + 4i
        const bool whole = t_begin + (bi + 1) * HOT_BS <= t_end;  // (the same for the whole wave)
        float sv[4], gm = -INFINITY;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            sv[i] = (whole || tok0 + 4 * i < t_end) ? sc[i] * q_inv : -INFINITY;
            gm = fmaxf(gm, sv[i]);
        }
        gm = fmaxf(gm, __shfl_xor(gm, 16, 64));
        gm = fmaxf(gm, __shfl_xor(gm, 32, 64));  // (finite: a block's first token is always valid)
        if (__builtin_amdgcn_ballot_w64(gm > m_run) != 0) {  // some query's maximum grows: rescale (a factor of 1 otherwise)
            const float m_new = fmaxf(m_run, gm);
            const float alpha = exp2f(m_run - m_new);  // exp2(-inf) = 0 on the first block
            m_run = m_new;
            l_run *= alpha;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float a = __shfl(alpha, 4 * g4 + i, 64);  // o[.][i] is query 4 g4 + i
#pragma unroll
                for (int e = 0; e < NT; e++) o[e][i] *= a;
            }
        }
        half4 ph, pl;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float pw = exp2f(sv[i] - m_run + 10.f);  // 2^10 p; 0 for a masked token
            l_run += pw;
            const HalfPair t = split_hl(pw);
            ph[i] = t.h;
            pl[i] = t.l;
        }
        if (!whole) {  // rows past the end may hold anything
#pragma unroll
            for (int i = 0; i < 4; i++)
                if (tok0 + 4 * i >= t_end)
#pragma unroll
                    for (int e = 0; e < NT; e++) vv[i][e] = (_Float16)0.f;
        }
#pragma unroll
        for (int e = 0; e < NT; e++) {
            const half4 vb = {vv[0][e], vv[1][e], vv[2][e], vv[3][e]};
            o[e] = __builtin_amdgcn_mfma_f32_16x16x16f16(ph, vb, o[e], 0, 0, 0);
            o[e] = __builtin_amdgcn_mfma_f32_16x16x16f16(pl, vb, o[e], 0, 0, 0);
        }
    }
    l_run += __shfl_xor(l_run, 16, 64);
    l_run += __shfl_xor(l_run, 32, 64);

    __shared__ float s_m[4][GG], s_l[4][GG];
    __shared__ float s_acc[4][GG][D];
    if (g4 == 0 && c16 < GG) {
        s_m[wave][c16] = m_run - 10.f;  // (the sums carry 2^10)
        s_l[wave][c16] = l_run;
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int qr = 4 * g4 + i;
        if (qr < GG) {
#pragma unroll
            for (int e = 0; e < NT; e++) s_acc[wave][qr][c16 * NT + e] = o[e][i];
        }
    }
    finish_split<D, G, RG>(s_m, s_l, s_acc, partial, seq, kvh, split, kv_len, num_q_heads, num_kv_heads, max_splits, mg, tps);
}

// Many query rows of one sequence over its paged F16 context, each row with its own number of visible keys (the
// later chunks of a prompt, linear verification): paged_decode_gqa_kernel's two matrix-core products and operand
// layouts, with QT tiles of 16 consecutive query rows of one head per wave instead of 16 (row, head) queries of one
// KV head and the per-row limits as the mask. A workgroup holds NSUB (head of the KV head's group, row tile) pairs
// next to each other - the same rows for the heads that share the K/V rows, or neighbouring row tiles - times KS
// shares of the blocks (block b belongs to share b % KS). The NSUB waves of a share bring each block into LDS
// together, whole rows per load instruction, and read their operands from there, so the K/V rows pass through the
// memory system once per workgroup; the shares' (m, l, O) meet in LDS at the end and share 0 writes the rows.
// grid = (ceil(G * row tiles / NSUB), num_kv_heads); block = 64 * NSUB * KS.
template <int D, int QT, int KS, int NSUB = 4>
__global__ void __launch_bounds__(64 * NSUB * KS) paged_mq_kernel(const float *__restrict__ q, const _Float16 *__restrict__ pool,
                                                         const int32_t *__restrict__ table, const int32_t *__restrict__ kv_lens,
                                                         float *__restrict__ out, int query_len, int max_keys, int num_q_heads,
                                                         int num_kv_heads, float scale) {
    constexpr int NS = D / 32, NT = D / 16;
    typedef _Float16 halfv __attribute__((ext_vector_type(NT)));
    typedef _Float16 half4 __attribute__((ext_vector_type(4)));
    const int kvh = blockIdx.y, G = num_q_heads / num_kv_heads;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int sub = wave % NSUB, ksub = wave / NSUB;  // which of the workgroup's NSUB (head, row group) pairs, which share of the blocks
    const int row_groups = (query_len + 16 * QT - 1) / (16 * QT);
    const bool idle = blockIdx.x * NSUB + sub >= G * row_groups;  // (a wave without work walks no block; it still meets the others)
    const int combo = min((int)blockIdx.x * NSUB + sub, G * row_groups - 1);
    const int head = kvh * G + combo % G, r0 = (combo / G) * 16 * QT;
    const int c16 = lane & 15, g4 = lane >> 4;
    const size_t hs = (size_t)num_kv_heads * D, part = (size_t)HOT_BS * hs, qs = (size_t)num_q_heads * D;

    half8 qh[QT][NS], ql[QT][NS];
    float q_inv[QT];
    int lim[QT];  // query row r0 + 16 t + c16 sees the keys 0 .. lim[t] - 1
    int len_max = 0, len_min = max_keys;
#pragma unroll
    for (int t = 0; t < QT; t++) {
        const int qi = r0 + 16 * t + c16;
        lim[t] = qi < query_len ? min(max(kv_lens[qi], 0), max_keys) : 0;
        len_max = max(len_max, lim[t]);
        if (qi < query_len) len_min = min(len_min, lim[t]);
        float x[NS][8];
        float amax = 0.f;
        const float f0 = scale * kLog2e;
        const float *qp = q + (size_t)min(qi, query_len - 1) * qs + (size_t)head * D + g4 * (D / 4);
#pragma unroll
        for (int s = 0; s < NS; s++) {
            const float4 a = *(const float4 *)(qp + 8 * s), b = *(const float4 *)(qp + 8 * s + 4);
            const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
            for (int e = 0; e < 8; e++) {
                x[s][e] = v[e] * f0;
                amax = fmaxf(amax, fabsf(x[s][e]));
            }
        }
        amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
        amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
        int ex = 11;
        if (amax > 0.f && amax < INFINITY) {
            (void)frexpf(amax, &ex);
            ex = max(ex, -60);
        }
        const float f = ldexpf(1.f, 11 - ex);
        q_inv[t] = ldexpf(1.f, ex - 11);
#pragma unroll
        for (int s = 0; s < NS; s++)
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const HalfPair hl = split_hl(x[s][e] * f);
                qh[t][s][e] = hl.h;
                ql[t][s][e] = hl.l;
            }
    }
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {  // over the wave's rows
        len_max = max(len_max, __shfl_xor(len_max, off, 64));
        len_min = min(len_min, __shfl_xor(len_min, off, 64));
    }
    float4v o[QT][NT];
    float m_run[QT], l_run[QT];
#pragma unroll
    for (int t = 0; t < QT; t++) {
        m_run[t] = -INFINITY;
        l_run[t] = 0.f;
#pragma unroll
        for (int e = 0; e < NT; e++) o[t][e] = (float4v){0.f, 0.f, 0.f, 0.f};
    }
    const int n_blocks = idle ? 0 : (len_max + HOT_BS - 1) / HOT_BS;
    const int tok_row = 4 * (c16 & 3) + (c16 >> 2);  // this lane's K row of a block as A operand
    half8 kk[NS];
    halfv vv[4];
    // one block against the wave's query tiles (kk, vv hold the block's operands)
    auto compute = [&](int bi) __attribute__((always_inline)) {
        const int tok0 = bi * HOT_BS + g4;                       // score i of a tile: token tok0 + 4i
        const bool open = (bi + 1) * HOT_BS <= len_min;          // every row of the wave sees the whole block
#pragma unroll
        for (int t = 0; t < QT; t++) {
            float4v sc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < NS; s++) {
                sc = __builtin_amdgcn_mfma_f32_16x16x32_f16(kk[s], qh[t][s], sc, 0, 0, 0);
                sc = __builtin_amdgcn_mfma_f32_16x16x32_f16(kk[s], ql[t][s], sc, 0, 0, 0);
            }
            float sv[4], gm = -INFINITY;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                sv[i] = (open || tok0 + 4 * i < lim[t]) ? sc[i] * q_inv[t] : -INFINITY;
                gm = fmaxf(gm, sv[i]);
            }
            gm = fmaxf(gm, __shfl_xor(gm, 16, 64));
            gm = fmaxf(gm, __shfl_xor(gm, 32, 64));
            if (__builtin_amdgcn_ballot_w64(gm > m_run[t]) != 0) {
                const float m_new = fmaxf(m_run[t], gm);
                const float alpha = exp2f(m_run[t] - m_new);  // (m_new is finite in every lane that gets here with gm > m_run; 1 elsewhere)
                const float a_own = gm > m_run[t] ? alpha : 1.f;
                m_run[t] = m_new;
                l_run[t] *= a_own;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float a = __shfl(a_own, 4 * g4 + i, 64);
#pragma unroll
                    for (int e = 0; e < NT; e++) o[t][e][i] *= a;
                }
            }
            const float m_use = m_run[t] == -INFINITY ? 0.f : m_run[t];  // (a row that has seen no key yet: every weight 0)
            half4 ph, pl;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float pw = exp2f(sv[i] - m_use + 10.f);
                l_run[t] += pw;
                const HalfPair hl = split_hl(pw);
                ph[i] = hl.h;
                pl[i] = hl.l;
            }
#pragma unroll
            for (int e = 0; e < NT; e++) {
                const half4 vb = {vv[0][e], vv[1][e], vv[2][e], vv[3][e]};
                o[t][e] = __builtin_amdgcn_mfma_f32_16x16x16f16(ph, vb, o[t][e], 0, 0, 0);
                o[t][e] = __builtin_amdgcn_mfma_f32_16x16x16f16(pl, vb, o[t][e], 0, 0, 0);
            }
        }
    };
    {
        // The NSUB waves that share a block (same KV head, same share of the blocks) bring it into LDS together, whole
        // rows per load instruction, once for all of them, and each reads its operands from there: one pass over
        // the K/V rows per workgroup instead of one per wave. Two buffers, one barrier per block; the loop runs to
        // the longest of the workgroup's row tiles for every wave.
        constexpr int KP = D + 8;                      // halves per staged row (rows 4 banks apart)
        constexpr int TG = NSUB * 64, PIECES = HOT_BS * D / 8, PPT = (PIECES + TG - 1) / TG;
        __shared__ __attribute__((aligned(16))) _Float16 stg[KS][2][2][HOT_BS * KP];
        __shared__ int s_wg[2];
        if (tid == 0) s_wg[0] = s_wg[1] = 0;
        __syncthreads();
        if (lane == 0 && !idle) {
            atomicMax(&s_wg[0], n_blocks);
            atomicMax(&s_wg[1], len_max);
        }
        __syncthreads();
        const int wg_blocks = s_wg[0], wg_len = s_wg[1];
        const int tg = sub * 64 + lane;
        half8 kreg[PPT], vreg[PPT];
        auto issue = [&](int bi) {
            const int blk = __builtin_amdgcn_readfirstlane(table[bi]);
            const _Float16 *base = pool + (size_t)blk * 2 * part + (size_t)kvh * D;
#pragma unroll
            for (int j = 0; j < PPT; j++) {
                const int pc = min(j * TG + tg, PIECES - 1), row = pc / (D / 8), c8 = pc % (D / 8);
                // (plain loads: the workgroups of other row tiles and heads read the same rows, from the die's L2)
                kreg[j] = *(const half8 *)(base + (size_t)row * hs + c8 * 8);
                vreg[j] = *(const half8 *)(base + part + (size_t)row * hs + c8 * 8);
            }
        };
        auto commit = [&](int bi, int buf) {
#pragma unroll
            for (int j = 0; j < PPT; j++) {
                const int pc = j * TG + tg, row = pc / (D / 8), c8 = pc % (D / 8);
                if (PIECES % TG != 0 && pc >= PIECES) continue;
                half8 v = vreg[j];
                if (bi * HOT_BS + row >= wg_len) v = (half8){0, 0, 0, 0, 0, 0, 0, 0};  // rows past the sequence's end may hold anything
                *(half8 *)&stg[ksub][buf][0][row * KP + c8 * 8] = kreg[j];
                *(half8 *)&stg[ksub][buf][1][row * KP + c8 * 8] = v;
            }
        };
        const int iters = (wg_blocks + KS - 1) / KS;
        if (ksub < wg_blocks) issue(ksub);
        for (int it = 0; it < iters; it++) {
            const int bi = it * KS + ksub, buf = it & 1;
            if (bi < wg_blocks) commit(bi, buf);
            if (bi + KS < wg_blocks) issue(bi + KS);
            __syncthreads();
            if (bi < n_blocks) {  // (beyond: none of this wave's rows sees a key of the block)
#pragma unroll
                for (int s = 0; s < NS; s++) kk[s] = *(const half8 *)&stg[ksub][buf][0][tok_row * KP + g4 * (D / 4) + 8 * s];
#pragma unroll
                for (int i = 0; i < 4; i++) vv[i] = *(const halfv *)&stg[ksub][buf][1][(4 * i + g4) * KP + c16 * NT];
                compute(bi);
            }
        }
    }
    // lane (c16, g4) holds O[row 4 g4 + i][columns c16 * NT .. + NT - 1] of every tile; the row's sum of weights is
    // spread over the four lanes (row, 0..3). With KS > 1 the waves that took the other shares of the blocks hand
    // their (m, l, O) over through LDS - every value in the slot of the lane that holds the same element - and the
    // wave with share 0 adds them in share order.
    __shared__ float s_m[KS > 1 ? KS : 1][NSUB][QT][16], s_l[KS > 1 ? KS : 1][NSUB][QT][16];
    __shared__ float s_o[KS > 1 ? KS - 1 : 1][KS > 1 ? NSUB : 1][QT][4 * NT][64];
#pragma unroll
    for (int t = 0; t < QT; t++) {
        l_run[t] += __shfl_xor(l_run[t], 16, 64);
        l_run[t] += __shfl_xor(l_run[t], 32, 64);
    }
    if constexpr (KS > 1) {
#pragma unroll
        for (int t = 0; t < QT; t++) {
            if (g4 == 0) {
                s_m[ksub][sub][t][c16] = m_run[t];
                s_l[ksub][sub][t][c16] = l_run[t];
            }
            if (ksub > 0) {
#pragma unroll
                for (int e = 0; e < NT; e++)
#pragma unroll
                    for (int i = 0; i < 4; i++) s_o[ksub - 1][sub][t][e * 4 + i][lane] = o[t][e][i];
            }
        }
        __syncthreads();
        if (ksub > 0) return;
    }
    if (idle) return;
#pragma unroll
    for (int t = 0; t < QT; t++) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int row = 4 * g4 + i, qi = r0 + 16 * t + row;
            float L, w[KS];
            if constexpr (KS > 1) {
                float M = s_m[0][sub][t][row];
#pragma unroll
                for (int k2 = 1; k2 < KS; k2++) M = fmaxf(M, s_m[k2][sub][t][row]);
                L = 0.f;
#pragma unroll
                for (int k2 = 0; k2 < KS; k2++) {
                    const float mk = s_m[k2][sub][t][row];
                    w[k2] = mk == -INFINITY ? 0.f : exp2f(mk - M);
                    L += s_l[k2][sub][t][row] * w[k2];
                }
            } else {
                L = __shfl(l_run[t], row, 64);
                w[0] = 1.f;
            }
            const float inv = L > 0.f ? 1.f / L : 0.f;
            if (qi >= query_len) continue;
            float *op = out + (size_t)qi * qs + (size_t)head * D + c16 * NT;
            float y[NT];
#pragma unroll
            for (int e = 0; e < NT; e++) {
                float acc = o[t][e][i] * w[0];
                if constexpr (KS > 1) {
#pragma unroll
                    for (int k2 = 1; k2 < KS; k2++) acc += s_o[k2 - 1][sub][t][e * 4 + i][lane] * w[k2];
                }
                y[e] = acc * inv;
            }
#pragma unroll
            for (int e = 0; e < NT; e += 4) *(float4 *)(op + e) = make_float4(y[e], y[e + 1], y[e + 2], y[e + 3]);
        }
    }
}

// Copies per-sequence block tables given as device pointers into a padded [batch, max_blocks] matrix.
__global__ void gather_tables_kernel(const int32_t *const *bt_ptrs, const int32_t *seq_lens, int32_t *matrix,
                                     int max_blocks, int block_size) {
    const int seq = blockIdx.x;
    const int nb = (seq_lens[seq] + block_size - 1) / block_size;
    const int32_t *src = bt_ptrs[seq];
    for (int i = threadIdx.x; i < max_blocks; i += blockDim.x) matrix[(size_t)seq * max_blocks + i] = i < nb ? src[i] : 0;
}

// grid = (num_q_heads, batch); block = D threads.
template <int D>
__global__ void __launch_bounds__(D) paged_merge_kernel(const float *__restrict__ partial,
                                                        const int32_t *__restrict__ kv_lens, float *__restrict__ out,
                                                        int num_q_heads, int max_splits, int tps) {
    const int qh = blockIdx.x, seq = blockIdx.y, d = threadIdx.x;
    const int kv_len = kv_lens[seq];
    const int ns = min((kv_len + tps - 1) / tps, max_splits);  // a length over the caller's bound: its first max_splits splits
    const float *pb = partial + ((size_t)seq * num_q_heads + qh) * max_splits * (D + 2);
    float M = -INFINITY;
    for (int s = 0; s < ns; s++) M = fmaxf(M, pb[(size_t)s * (D + 2)]);
    float L = 0.f, A = 0.f;
    for (int s = 0; s < ns; s++) {
        const float *ps = pb + (size_t)s * (D + 2);
        const float f = exp2f(ps[0] - M);
        L += ps[1] * f;
        A += ps[2 + d] * f;
    }
    out[((size_t)seq * num_q_heads + qh) * D + d] = (L > 0.f) ? A / L : 0.f;
}

// The rows of candidate trees: query row `row` of head qh has its context (pool positions < start, read by
// paged_decode_gqa_kernel<D, G, RG>) as split partials; this adds the tree's own keys, which sit at pool positions
// start .. start + n - 1 of the same sequence and are visible where the row's mask says so (medusa/tree.go:186-202),
// and normalises. info[row] = (block-table row, start, row index inside its tree, rows of the tree);
// grid = (num_q_heads, rows); block = D threads.
template <int D>
__global__ void __launch_bounds__(D) tree_merge_kernel(const float *__restrict__ partial, const float *__restrict__ q,
                                                       const _Float16 *__restrict__ pool, const int32_t *__restrict__ bt_matrix,
                                                       int max_blocks, const int4 *__restrict__ info,
                                                       const uint8_t *__restrict__ masks, const int32_t *__restrict__ mask_off,
                                                       float *__restrict__ out, int num_q_heads, int num_kv_heads, float scale,
                                                       int max_splits) {
    constexpr int MAXN = 64;  // rows of one tree (checked on the host)
    const int qh = blockIdx.x, row = blockIdx.y, d = threadIdx.x;
    const int4 inf = info[row];
    const int start = inf.y, r = inf.z, n = inf.w;
    const int kvh = qh / (num_q_heads / num_kv_heads);
    const int32_t *bt = bt_matrix + (size_t)inf.x * max_blocks;
    const uint8_t *mk = masks + mask_off[row] + (size_t)r * n;
    const size_t hs = (size_t)num_kv_heads * D, part = (size_t)HOT_BS * hs;
    __shared__ float s_q[D];
    __shared__ float s_s[MAXN];
    s_q[d] = q[((size_t)row * num_q_heads + qh) * D + d] * (scale * kLog2e);
    __syncthreads();
    if (d < n) {  // one key per thread: its score in the exp2 domain, -inf where the mask hides it
        float t = -INFINITY;
        if (mk[d]) {
            const int pos = start + d;
            const _Float16 *kp = pool + (size_t)bt[pos / HOT_BS] * 2 * part + (size_t)(pos % HOT_BS) * hs + (size_t)kvh * D;
            t = 0.f;
            for (int e = 0; e < D; e++) t = fmaf(s_q[e], (float)kp[e], t);
        }
        s_s[d] = t;
    }
    __syncthreads();
    const int ns = (start + TPW - 1) / TPW;
    const float *pb = partial + ((size_t)row * num_q_heads + qh) * max_splits * (D + 2);
    float M = -INFINITY;
    for (int s = 0; s < ns; s++) M = fmaxf(M, pb[(size_t)s * (D + 2)]);
    for (int j = 0; j < n; j++) M = fmaxf(M, s_s[j]);
    float L = 0.f, A = 0.f;
    for (int s = 0; s < ns; s++) {
        const float *ps = pb + (size_t)s * (D + 2);
        const float f = exp2f(ps[0] - M);
        L += ps[1] * f;
        A += ps[2 + d] * f;
    }
    for (int j = 0; j < n; j++) {
        if (s_s[j] == -INFINITY) continue;
        const int pos = start + j;
        const _Float16 *vp = pool + (size_t)bt[pos / HOT_BS] * 2 * part + part + (size_t)(pos % HOT_BS) * hs + (size_t)kvh * D;
        const float f = exp2f(s_s[j] - M);
        L += f;
        A = fmaf(f, (float)vp[d], A);
    }
    out[((size_t)row * num_q_heads + qh) * D + d] = (L > 0.f) ? A / L : 0.f;
}

// --------------------------------------------------------------------------------------------
// Dense causal prefill (Backend.SDPAPrefill, backend.go:389; math of backend/cpu/cpu.go:568-632 per query):
// FlashAttention-2 style. grid = (query tiles of 64, Hq); block = 256 = 4 waves of 16 queries.
// Per 32-key tile: K goes to LDS as f16 rows, V transposed ([d][key], so that a lane's eight keys of one column are
// 16 contiguous bytes); S = Q K^T and O += P V run on v_mfma_f32_16x16x32_f16 with every float32 operand split in
// two f16 halves (x = hi + lo, about 22 significant bits, float32 accumulation): Q and P always, K and V when they
// come as float32 (dense prefill; the products hi*hi + hi*lo + lo*hi, the lo*lo term is below float32's last bit),
// not when they are the f16 rows of the paged pool, which are exact. The softmax is online in the exp2 domain; P
// crosses from the MFMA output layout to the operand layout through a wave-private LDS tile. LDS row pitches are
// an odd number of 16-byte slots, so the 16 lanes of an operand read land in 16 different slots.
constexpr int FA_BQ = 64, FA_BK = 32;

template <int N>
__device__ __forceinline__ float row16_max(float t) {  // max over the 16 lanes of a row; every lane gets it
    t = fmaxf(t, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, t), 0xb1, 0xf, 0xf, false)));
    t = fmaxf(t, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, t), 0x4e, 0xf, 0xf, false)));
    t = fmaxf(t, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, t), 0x141, 0xf, 0xf, false)));
    t = fmaxf(t, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, t), 0x140, 0xf, 0xf, false)));
    return t;
}

// CAP: the scores (held in log2 units, score * log2 e) pass through cap2 * tanh(. / cap2) with
// cap2 = softcap * log2 e, which is softcap * tanh(score / softcap) in those units.
// PAGED: the keys and values are the rows of one sequence in an F16 paged pool (block table `paged.table`), and query
// row i attends to the first paged.kv_lens[i] of them (Backend.SDPAPagedDecodeMultiquery, backend.go:456-466: the
// later chunks of a prompt, kv_lens[i] = startPos + i + 1, and linear verification, runtime/block.go:881-890)
// instead of to rows 0..i of dense float32 K and V.
struct PagedSrc {
    const _Float16 *pool;
    const int32_t *table;
    const int32_t *kv_lens;
    int block_size;
};

template <int D, bool CAP = false, bool PAGED = false>
__global__ void __launch_bounds__(256) prefill_fa2_kernel(const float *__restrict__ q, const float *__restrict__ k,
                                                          const float *__restrict__ v, float *__restrict__ out, int S,
                                                          int num_q_heads, int num_kv_heads, float scale,
                                                          float softcap = 0.f, PagedSrc paged = PagedSrc()) {
    constexpr int KP = D + 8, VP = FA_BK + 8, PP = FA_BK + 4;  // halves per K row, halves per V^T row, floats per P row
    constexpr int NLO = PAGED ? 1 : 2;                           // [0]: hi halves, [1]: lo halves (float32 sources only)
    __shared__ __attribute__((aligned(16))) _Float16 Ks[NLO][FA_BK * KP];
    __shared__ __attribute__((aligned(16))) _Float16 Vt[NLO][D * VP];
    __shared__ __attribute__((aligned(16))) float Ps[4][16 * PP];
    __shared__ int len_max[5];  // PAGED: the longest key range among each wave's 16 queries, [4]: among all 64
    const int qt = blockIdx.x, h = blockIdx.y, kvh = h / (num_q_heads / num_kv_heads);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int c16 = lane & 15, g = lane >> 4;
    const int q0 = qt * FA_BQ + wave * 16;  // the wave's first query
    const size_t qs = (size_t)num_q_heads * D, ks = (size_t)num_kv_heads * D;
    int lim[4];  // keys 0 .. lim[i]-1 are visible to the lane's query row 4g + i
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int qi = q0 + 4 * g + i;
        lim[i] = PAGED ? (qi < S ? max(paged.kv_lens[qi], 0) : 0) : min(qi + 1, S);
    }
    if (PAGED) {
        if (tid < 5) len_max[tid] = 0;
        __syncthreads();
        const int m4 = max(max(lim[0], lim[1]), max(lim[2], lim[3]));
        atomicMax(&len_max[wave], m4);
        atomicMax(&len_max[4], m4);
        __syncthreads();
    }
    const int wave_keys = PAGED ? len_max[wave] : min(q0 + 15, S - 1) + 1;  // keys any of the wave's queries sees

    // Q as the A operand: lane (row c16, columns 32s + 8g .. + 7), pre-multiplied by scale*log2(e), hi + lo
    half8 qh[D / 32], ql[D / 32];
    {
        const int qi = min(q0 + c16, S - 1);
        const float *qp = q + (size_t)qi * qs + (size_t)h * D + 8 * g;
        const float f = scale * kLog2e;
#pragma unroll
        for (int s = 0; s < D / 32; s++) {
            const float4 a = *(const float4 *)(qp + 32 * s), b = *(const float4 *)(qp + 32 * s + 4);
            const float x[8] = {a.x * f, a.y * f, a.z * f, a.w * f, b.x * f, b.y * f, b.z * f, b.w * f};
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const HalfPair t = split_hl(x[e]);
                qh[s][e] = t.h;
                ql[s][e] = t.l;
            }
        }
    }
    float4v o[D / 16];
#pragma unroll
    for (int db = 0; db < D / 16; db++) o[db] = (float4v){0.f, 0.f, 0.f, 0.f};
    float m_run[4], l_run[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        m_run[i] = -INFINITY;
        l_run[i] = 0.f;
    }
    const int last_q = min(qt * FA_BQ + FA_BQ - 1, S - 1);
    const int n_keys = PAGED ? len_max[4] : last_q + 1;  // keys 0 .. n_keys-1 are visible to some query of the tile
    const int n_tiles = (n_keys + FA_BK - 1) / FA_BK;
    // A tile's rows as they come from memory: requested a tile ahead, so that their way is covered by the
    // arithmetic of the tile before (a thread's pieces: key idx % 32, columns 8 (idx / 32) .. + 7).
    constexpr int NIDX = FA_BK * (D / 8) / 256;
    static_assert(NIDX * 256 == FA_BK * (D / 8), "whole trips of the 256 threads over a tile");
    float4 rk[PAGED ? 1 : NIDX][2], rv[PAGED ? 1 : NIDX][2];
    half8 rkh[PAGED ? NIDX : 1], rvh[PAGED ? NIDX : 1];
    auto fetch = [&](int kt) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < NIDX; t++) {
            const int idx = tid + 256 * t;
            const int key = idx % FA_BK, d8 = (idx / FA_BK) * 8;  // (lanes run over keys: V^T's 2-byte stores fill whole rows)
            const int ki = kt * FA_BK + key;
            if constexpr (PAGED) {
                const half8 z = {0, 0, 0, 0, 0, 0, 0, 0};
                rkh[t] = z;
                rvh[t] = z;
                if (ki < n_keys) {
                    const size_t part = (size_t)paged.block_size * ks;  // a block's K rows, then its V rows
                    const _Float16 *kp = paged.pool + (size_t)paged.table[ki / paged.block_size] * 2 * part +
                                         (size_t)(ki % paged.block_size) * ks + (size_t)kvh * D + d8;
                    rkh[t] = *(const half8 *)kp;
                    rvh[t] = *(const half8 *)(kp + part);
                }
            } else {
                const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
                rk[t][0] = rk[t][1] = rv[t][0] = rv[t][1] = z;
                if (ki < S) {
                    const float *kp = k + (size_t)ki * ks + (size_t)kvh * D + d8, *vp = v + (size_t)ki * ks + (size_t)kvh * D + d8;
                    rk[t][0] = *(const float4 *)kp;
                    rk[t][1] = *(const float4 *)(kp + 4);
                    rv[t][0] = *(const float4 *)vp;
                    rv[t][1] = *(const float4 *)(vp + 4);
                }
            }
        }
    };
    // what fetch() brought, as f16 halves into the LDS tiles (K rows, V transposed)
    auto stash = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < NIDX; t++) {
            const int idx = tid + 256 * t;
            const int key = idx % FA_BK, d8 = (idx / FA_BK) * 8;
            half8 kh = {0, 0, 0, 0, 0, 0, 0, 0}, vh = kh, kl = kh, vl = kh;
            if constexpr (PAGED) {
                kh = rkh[t];
                vh = rvh[t];
            } else {
                const float4 k0 = rk[t][0], k1 = rk[t][1], v0 = rv[t][0], v1 = rv[t][1];
                const float kx[8] = {k0.x, k0.y, k0.z, k0.w, k1.x, k1.y, k1.z, k1.w};
                const float vx[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const HalfPair tk = split_hl(kx[e]), tv = split_hl(vx[e]);
                    kh[e] = tk.h; kl[e] = tk.l;
                    vh[e] = tv.h; vl[e] = tv.l;
                }
            }
            *(half8 *)(&Ks[0][key * KP + d8]) = kh;
#pragma unroll
            for (int e = 0; e < 8; e++) Vt[0][(d8 + e) * VP + key] = vh[e];
            if (!PAGED) {
                *(half8 *)(&Ks[NLO - 1][key * KP + d8]) = kl;
#pragma unroll
                for (int e = 0; e < 8; e++) Vt[NLO - 1][(d8 + e) * VP + key] = vl[e];
            }
        }
    };
    if (n_tiles > 0) fetch(0);
    for (int kt = 0; kt < n_tiles; kt++) {
        __syncthreads();  // the previous tile's reads are done
        stash();
        if (kt + 1 < n_tiles) fetch(kt + 1);
        __syncthreads();
        if (kt * FA_BK >= wave_keys) continue;  // every key of the tile is beyond what the wave's queries see
        // S = Q K^T for the wave's 16 queries x 32 keys: lane holds S[row 4g+i][key cb*16 + c16]
        float4v sc[FA_BK / 16];
#pragma unroll
        for (int cb = 0; cb < FA_BK / 16; cb++) {
            float4v acc = {0.f, 0.f, 0.f, 0.f};
            const int ko = (cb * 16 + c16) * KP + 8 * g;  // key cb*16 + c16, columns 32s + 8g .. + 7
#pragma unroll
            for (int s = 0; s < D / 32; s++) {
                const half8 b = *(const half8 *)(&Ks[0][ko + 32 * s]);
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(qh[s], b, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(ql[s], b, acc, 0, 0, 0);
                if (!PAGED) {
                    const half8 bl = *(const half8 *)(&Ks[NLO - 1][ko + 32 * s]);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(qh[s], bl, acc, 0, 0, 0);
                }
            }
            sc[cb] = acc;
        }
        if (CAP) {
            const float cap2 = softcap * kLog2e, inv_cap2 = 1.f / cap2;
#pragma unroll
            for (int cb = 0; cb < FA_BK / 16; cb++)
#pragma unroll
                for (int i = 0; i < 4; i++) sc[cb][i] = cap2 * tanhf(sc[cb][i] * inv_cap2);
        }
        // causal mask, online softmax per row
        float alpha[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float mx = -INFINITY;
#pragma unroll
            for (int cb = 0; cb < FA_BK / 16; cb++) {
                const int ki = kt * FA_BK + cb * 16 + c16;
                if (ki >= lim[i]) sc[cb][i] = -INFINITY;
                mx = fmaxf(mx, sc[cb][i]);
            }
            mx = row16_max<16>(mx);
            const float m_new = fmaxf(m_run[i], mx);
            // a row whose keys are all masked so far keeps m = -inf: exp2(-inf - -inf) must not be evaluated
            alpha[i] = (m_new == -INFINITY) ? 1.f : exp2f(m_run[i] - m_new);
            float rs = 0.f;
#pragma unroll
            for (int cb = 0; cb < FA_BK / 16; cb++) {
                const float pw = (sc[cb][i] == -INFINITY) ? 0.f : exp2f(sc[cb][i] - m_new);
                sc[cb][i] = pw;
                rs += pw;
            }
            // sum over the 16 key lanes
            rs += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, rs), 0xb1, 0xf, 0xf, false));
            rs += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, rs), 0x4e, 0xf, 0xf, false));
            rs += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, rs), 0x141, 0xf, 0xf, false));
            rs += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, rs), 0x140, 0xf, 0xf, false));
            l_run[i] = l_run[i] * alpha[i] + rs;
            m_run[i] = m_new;
        }
#pragma unroll
        for (int db = 0; db < D / 16; db++)
#pragma unroll
            for (int i = 0; i < 4; i++) o[db][i] *= alpha[i];
        // P: MFMA output layout -> operand layout through the wave's LDS tile
        float *pt = &Ps[wave][0];
#pragma unroll
        for (int cb = 0; cb < FA_BK / 16; cb++)
#pragma unroll
            for (int i = 0; i < 4; i++) pt[(4 * g + i) * PP + cb * 16 + c16] = sc[cb][i];
        // (wave-private tile: the wave's own LDS accesses are ordered)
        // P as the A operand: lane (row c16, keys 8g .. 8g + 7), hi + lo
        half8 ph, pl;
        {
            const float4 a = *(const float4 *)(pt + c16 * PP + 8 * g), b = *(const float4 *)(pt + c16 * PP + 8 * g + 4);
            const float x[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const HalfPair t = split_hl(x[e]);
                ph[e] = t.h;
                pl[e] = t.l;
            }
        }
        // O += P V: lane holds O[row 4g+i][d = db*16 + c16]; B operand: column d, keys 8g .. 8g + 7 of V^T
#pragma unroll
        for (int db = 0; db < D / 16; db++) {
            const int vo = (db * 16 + c16) * VP + 8 * g;
            const half8 vb = *(const half8 *)(&Vt[0][vo]);
            o[db] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ph, vb, o[db], 0, 0, 0);
            o[db] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pl, vb, o[db], 0, 0, 0);
            if (!PAGED) {
                const half8 vl = *(const half8 *)(&Vt[NLO - 1][vo]);
                o[db] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ph, vl, o[db], 0, 0, 0);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int qi = q0 + 4 * g + i;
        if (qi >= S) continue;
        const float inv = l_run[i] > 0.f ? 1.f / l_run[i] : 0.f;
        float *op = out + (size_t)qi * qs + (size_t)h * D + c16;
#pragma unroll
        for (int db = 0; db < D / 16; db++) op[db * 16] = o[db][i] * inv;
    }
}

// The partial sums of a call that must not allocate: one fixed area per device, shared by every such call on that
// device (calls that overlap there race). Host code never uses the array's name as an address: attn_noalloc_init
// asks the runtime where the current device keeps its copy, and that pointer is what the kernels get.
constexpr size_t FIXED_WS_BYTES = (size_t)8 << 20;
static __device__ __align__(256) unsigned char scratch[FIXED_WS_BYTES];

// Tokens per split of the streaming kernels: ATTN_TPW; half of it for grouped queries at heads of 64 / 128 (fewer
// kv heads, so fewer workgroups per token, and the matrix-core form's per-block work is small: measured faster at
// every batch tried); and down to a quarter of ATTN_TPW while that many splits would leave most of the chip idle
// (a single sequence). vx_pack_batch leaves a work list for each of the first two.
int split_tokens(vx_backend *be, int D, int G, int batch, int num_kv_heads, int max_kv_len) {
    static const int cus = [&] {
        int n = 0;
        return (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, be->device) == hipSuccess && n > 0) ? n : 256;
    }();
    int tps = TPW;
    if (G >= 2 && (D == 64 || D == 128)) tps = TPW / 2;
    while (tps > TPW / 4 && (size_t)batch * num_kv_heads * ceil_div(max_kv_len, tps) < (size_t)2 * cus) tps /= 2;
    return tps;
}
// Bytes of partial sums for that many splits: (maximum, sum, D values) per sequence, head and split; a single
// sequence's merged row behind them.
size_t split_bytes(int D, int batch, int num_q_heads, int max_splits) {
    const size_t partial_floats = ((size_t)batch * num_q_heads * max_splits * (D + 2) + 3) & ~(size_t)3;
    return (partial_floats + (batch == 1 ? (size_t)num_q_heads * D : 0)) * sizeof(float);
}

// fixed: the call takes the fixed area (and fails when it is too small) instead of the growable one
template <int D, int G>
int launch_hot(vx_backend *be, const float *q, const void *pool, const int32_t *bt_matrix, const int32_t *bt_rows,
               int max_blocks, const int32_t *kv_lens, float *out, int batch, int num_q_heads, int num_kv_heads,
               float scale, int max_kv_len, bool fixed) {
    const int tps = split_tokens(be, D, G, batch, num_kv_heads, max_kv_len);
    int max_splits = ceil_div(max_kv_len, tps);
    const size_t need = split_bytes(D, batch, num_q_heads, max_splits);
    const size_t partial_floats = ((size_t)batch * num_q_heads * max_splits * (D + 2) + 3) & ~(size_t)3;
    float *ws;
    if (fixed) {
        if (need > FIXED_WS_BYTES || !be->attn_fixed_ws) {
            set_error("vx_sdpa_paged_decode_ragged_noalloc: %d sequences x %d heads x %d splits of %d tokens need %zu bytes of "
                      "partial sums, the fixed area holds %zu", batch, num_q_heads, max_splits, tps, need, FIXED_WS_BYTES);
            return VX_ERR_INVALID;
        }
        ws = (float *)be->attn_fixed_ws;
    } else {
        int rc = ensure_ws(be, &be->attn_ws, &be->attn_ws_bytes, need, "attention");
        if (rc) return rc;
        ws = (float *)be->attn_ws;
    }
    // With a work list from vx_pack_batch for these lengths the grid's second dimension runs over its items
    // (at most max_splits per sequence, as max_kv_len bounds every length); otherwise over (split, sequence).
    const bool half_list = tps == TPW / 2;
    const size_t list_off = half_list ? (be->items.cap + 1) * 4 : 0, list_cap = half_list ? 2 * be->items.cap : be->items.cap;
    const bool listed = (tps == TPW || half_list) && be->items.valid && be->items.kv_lens == kv_lens &&
                        be->items.table_rows == bt_rows && be->items.batch == batch && (size_t)batch * max_splits <= list_cap &&
                        (size_t)batch * max_splits <= 65535;
    const int32_t *const list = listed ? be->items.buf + list_off : nullptr;
    dim3 grid(num_kv_heads, listed ? batch * max_splits : max_splits, listed ? 1 : batch);
    // (for measurements: the vector kernel walking the list with n workgroups per compute unit instead)
    static const int gy_env = getenv("VEXEL_HIP_ATTN_WG_PER_CU") ? atoi(getenv("VEXEL_HIP_ATTN_WG_PER_CU")) : 0;
    dim3 grid_walk = grid;
    if (listed && gy_env > 0) {
        static int cus = 0;
        if (cus == 0 && (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, be->device) != hipSuccess || cus <= 0)) cus = 256;
        grid_walk.y = (unsigned)std::max(1, std::min(batch * max_splits, ceil_div(cus * gy_env, num_kv_heads)));
    }
    // out == NULL leaves the result to vx_decode_ffn(attn = NULL): as split partial sums, and - where the shape
    // allows - already merged by the workgroups that finish last: prepared as that call's first operand, or, for
    // a single row, as plain floats behind the partial sums (what the matrix-vector product reads).
    MergeOut mg;
    float *plain = nullptr;
    const bool no_merge = !be->attn_merge;
    constexpr int GD = G * D;
    // whole merge units, of at most one chunk per wave of the merging workgroup (with more - 7 chunks per two KV heads
    // at 28 / 4 heads of 128 - the merge at the launch's tail costs what the separate merge launch does)
    const bool mergeable = num_kv_heads % MergeUnit<GD>::HPC == 0 && MergeUnit<GD>::CH <= 4;
    if (!out && !fixed && !no_merge && mergeable && be->attn_cnt && (size_t)batch * num_kv_heads <= VX_ATTN_CNT) {
        if (batch == 1) {
            mg.cnt = be->attn_cnt;
            mg.plain = plain = ws + partial_floats;
        } else {
            int mpad = 0;
            const int rc = prep_begin_chunked(be, batch, num_q_heads * D, &mg.pv, &mpad);
            if (rc == VX_OK) {
                mg.cnt = be->attn_cnt;
                mg.mpad = mpad;
            } else if (rc != VX_ERR_UNSUPPORTED)
                return rc;
        }
    }
    // grouped queries on heads of 64 or 128: the matrix-core form (VEXEL_HIP_ATTN_VECTOR_FORM=1: the vector form, to compare)
    static const bool vector_form = getenv("VEXEL_HIP_ATTN_VECTOR_FORM") != nullptr;
    bool launched = false;
    if constexpr (G >= 2 && (D == 64 || D == 128)) {  // (one query per K/V row: the vector form is the faster one, 110 against 119 us)
        if (!vector_form || G > 8) {
            paged_decode_gqa_kernel<D, G><<<grid, 256, 0, be->stream>>>(q, (const _Float16 *)pool, bt_matrix, bt_rows,
                                                                        max_blocks, kv_lens, ws, num_q_heads,
                                                                        num_kv_heads, scale, max_splits,
                                                                        list, mg, tps);
            launched = true;
        }
    }
    if constexpr (G <= 8) {  // (wider groups have the matrix-core form only)
        if (!launched)
            paged_decode_f16_kernel<D, G><<<grid_walk, 256, 0, be->stream>>>(q, (const _Float16 *)pool, bt_matrix, bt_rows,
                                                                        max_blocks, kv_lens, ws, num_q_heads,
                                                                        num_kv_heads, scale, max_splits,
                                                                        list, mg, tps);
    }
    VX_CHECK_LAUNCH();
    if (!fixed) be->split.batch = 0;  // (the fixed area is not where vx_decode_ffn looks for a split result)
    if (!out) {  // the caller merges: vx_decode_ffn(attn = NULL)
        be->split.merged = mg.cnt != nullptr && !plain;
        be->split.plain = plain;
        be->split.batch = batch;
        be->split.num_q_heads = num_q_heads;
        be->split.head_dim = D;
        be->split.max_splits = max_splits;
        be->split.tokens_per_split = tps;
        be->split.kv_lens = kv_lens;
        return VX_OK;
    }
    paged_merge_kernel<D><<<dim3(num_q_heads, batch), D, 0, be->stream>>>(ws, kv_lens, out, num_q_heads, max_splits, tps);
    VX_CHECK_LAUNCH();
    return VX_OK;
}

int run_generic(vx_backend *be, const AttnParams &p, int num_queries) {
    VX_REQUIRE(p.head_dim > 0 && p.head_dim <= 256, "attention: head_dim %d not in 1..256", p.head_dim);
    VX_REQUIRE(p.num_kv_heads > 0 && p.num_q_heads % p.num_kv_heads == 0,
               "attention: %d query heads not a multiple of %d kv heads", p.num_q_heads, p.num_kv_heads);
    if (num_queries == 0) return VX_OK;
    attn_generic_kernel<<<dim3(p.num_q_heads, num_queries), GEN_THREADS, 0, be->stream>>>(p);
    VX_CHECK_LAUNCH();
    return VX_OK;
}

// Ragged batched decode: hot kernel when the shape has an instantiation, generic otherwise.
int run_ragged(vx_backend *be, const float *q, const void *pool, int pool_is_f16, const int32_t *const *bt_ptrs,
               const int32_t *bt_matrix, const int32_t *bt_rows, int max_blocks, const int32_t *kv_lens, float *out,
               int batch, int block_size,
               int num_q_heads, int num_kv_heads, int head_dim, float scale, int max_kv_len, bool fixed = false) {
    VX_REQUIRE(num_kv_heads > 0 && num_q_heads % num_kv_heads == 0, "attention: bad head counts");
    VX_REQUIRE(block_size > 0 && max_kv_len > 0, "attention: bad block size / kv length");
    if (batch == 0) return VX_OK;
    const int G = num_q_heads / num_kv_heads;
    const bool hot = pool_is_f16 && ((uintptr_t)pool % 16) == 0 && block_size == HOT_BS && bt_matrix && !bt_ptrs;
#define VX_HOT(DD, GG)                                                                                         \
    if (hot && head_dim == DD && G == GG)                                                                      \
        return launch_hot<DD, GG>(be, q, pool, bt_matrix, bt_rows, max_blocks, kv_lens, out, batch, num_q_heads, \
                                  num_kv_heads, scale, max_kv_len, fixed);
    VX_HOT(128, 1) VX_HOT(128, 2) VX_HOT(128, 4) VX_HOT(128, 8)
    VX_HOT(64, 1) VX_HOT(64, 2) VX_HOT(64, 4) VX_HOT(64, 8)
    // group sizes that are no power of two (Qwen 2 7B: 28 / 4 heads, LLaMA 3.2 3B: 24 / 8, Qwen 2 1.5B: 12 / 2)
    VX_HOT(128, 3) VX_HOT(128, 5) VX_HOT(128, 6) VX_HOT(128, 7)
    VX_HOT(64, 3) VX_HOT(64, 5) VX_HOT(64, 6) VX_HOT(64, 7)
    // wide groups (12 and 16 query heads per KV head: the matrix-core tile's 16 rows)
    VX_HOT(128, 12) VX_HOT(128, 16)
    // heads of 256 (Gemma): 32 lanes per token; the K/V registers of a 16-token block leave room for 1 or 2 query heads
    VX_HOT(256, 1) VX_HOT(256, 2)
    // heads of 80 (Phi-2) and 96 (Phi-3 mini) on 16 lanes per token, 10 or 12 of them live
    VX_HOT(80, 1) VX_HOT(96, 1)
#undef VX_HOT
    if (fixed) {
        set_error("vx_sdpa_paged_decode_ragged_noalloc: only the geometries of the streaming kernel (see "
                  "vx_sdpa_paged_decode_split_supported) run without scratch allocation");
        return VX_ERR_UNSUPPORTED;
    }
    if (!out) {
        set_error("vx_sdpa_paged_decode_ragged: out = NULL (split form) needs an F16 pool with 16-token blocks and a "
                  "supported head geometry");
        return VX_ERR_UNSUPPORTED;
    }
    AttnParams p = {};
    p.q = q;
    p.out = out;
    p.k = pool;
    p.mode = MODE_PAGED;
    p.f16 = pool_is_f16;
    p.num_q_heads = num_q_heads;
    p.num_kv_heads = num_kv_heads;
    p.head_dim = head_dim;
    p.scale = scale;
    p.bt_ptrs = bt_ptrs;
    p.bt_matrix = bt_matrix;
    p.bt_rows = bt_rows;
    p.max_blocks = max_blocks;
    p.block_size = block_size;
    p.kv_lens = kv_lens;
    return run_generic(be, p, batch);
}

}  // namespace

namespace vx {
int attn_noalloc_init(vx_backend *be) {
    void *p = nullptr;
    VX_CHECK_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));  // the current device's copy of the array
    be->attn_fixed_ws = p;
    return VX_OK;
}
}  // namespace vx

extern "C" {

static int sdpa_dense(vx_backend *be, const float *q, const float *k, const float *v, float *out, int kv_len,
                      int num_q_heads, int num_kv_heads, int head_dim, float scale, float softcap, int kv_head_stride) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(q && k && v && out && kv_len >= 1, "vx_sdpa: bad arguments");
    VX_REQUIRE(softcap >= 0.f, "vx_sdpa_softcap: negative softcap");
    AttnParams p = {};
    p.softcap = softcap;
    p.q = q;
    p.out = out;
    p.k = k;
    p.v = v;
    p.mode = MODE_CONTIG;
    p.num_q_heads = num_q_heads;
    p.num_kv_heads = num_kv_heads;
    p.head_dim = head_dim;
    p.scale = scale;
    p.kv_head_stride = kv_head_stride;
    p.kv_len = kv_len;
    return run_generic(be, p, 1);
}

int vx_sdpa(vx_backend *be, const float *q, const float *k, const float *v, float *out, int kv_len, int num_q_heads,
            int num_kv_heads, int head_dim, float scale, int kv_head_stride) {
    return sdpa_dense(be, q, k, v, out, kv_len, num_q_heads, num_kv_heads, head_dim, scale, 0.f, kv_head_stride);
}

int vx_sdpa_softcap(vx_backend *be, const float *q, const float *k, const float *v, float *out, int kv_len,
                    int num_q_heads, int num_kv_heads, int head_dim, float scale, float softcap, int kv_head_stride) {
    return sdpa_dense(be, q, k, v, out, kv_len, num_q_heads, num_kv_heads, head_dim, scale, softcap, kv_head_stride);
}

static int sdpa_prefill_dense(vx_backend *be, const float *q, const float *k, const float *v, float *out, int seq_len,
                              int num_q_heads, int num_kv_heads, int head_dim, float scale, float softcap) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(q && k && v && out && seq_len >= 0, "vx_sdpa_prefill: bad arguments");
    VX_REQUIRE(num_kv_heads > 0 && num_q_heads % num_kv_heads == 0, "vx_sdpa_prefill: bad head counts");
    VX_REQUIRE(softcap >= 0.f, "vx_sdpa_prefill_softcap: negative softcap");
    if (seq_len == 0) return VX_OK;
    if ((head_dim == 64 || head_dim == 128) && ((uintptr_t)k % 16) == 0 && ((uintptr_t)v % 16) == 0) {
        const dim3 grid(ceil_div(seq_len, FA_BQ), num_q_heads);
        if (softcap > 0.f) {
            if (head_dim == 128)
                prefill_fa2_kernel<128, true><<<grid, 256, 0, be->stream>>>(q, k, v, out, seq_len, num_q_heads, num_kv_heads, scale, softcap);
            else
                prefill_fa2_kernel<64, true><<<grid, 256, 0, be->stream>>>(q, k, v, out, seq_len, num_q_heads, num_kv_heads, scale, softcap);
        } else if (head_dim == 128)
            prefill_fa2_kernel<128><<<grid, 256, 0, be->stream>>>(q, k, v, out, seq_len, num_q_heads, num_kv_heads, scale);
        else
            prefill_fa2_kernel<64><<<grid, 256, 0, be->stream>>>(q, k, v, out, seq_len, num_q_heads, num_kv_heads, scale);
        VX_CHECK_LAUNCH();
        return VX_OK;
    }
    AttnParams p = {};
    p.softcap = softcap;
    p.q = q;
    p.out = out;
    p.k = k;
    p.v = v;
    p.mode = MODE_PREFILL;
    p.num_q_heads = num_q_heads;
    p.num_kv_heads = num_kv_heads;
    p.head_dim = head_dim;
    p.scale = scale;
    return run_generic(be, p, seq_len);
}

int vx_sdpa_prefill(vx_backend *be, const float *q, const float *k, const float *v, float *out, int seq_len,
                    int num_q_heads, int num_kv_heads, int head_dim, float scale) {
    return sdpa_prefill_dense(be, q, k, v, out, seq_len, num_q_heads, num_kv_heads, head_dim, scale, 0.f);
}

int vx_sdpa_prefill_softcap(vx_backend *be, const float *q, const float *k, const float *v, float *out, int seq_len,
                            int num_q_heads, int num_kv_heads, int head_dim, float scale, float softcap) {
    return sdpa_prefill_dense(be, q, k, v, out, seq_len, num_q_heads, num_kv_heads, head_dim, scale, softcap);
}

static int paged_single(vx_backend *be, const float *q, const void *kv_pool, int f16, const int32_t *block_table,
                        float *out, int num_blocks, int block_size, int num_q_heads, int num_kv_heads, int head_dim,
                        float scale, int tokens_in_last_block) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(q && kv_pool && block_table && out, "vx_sdpa_paged_decode: null pointer");
    VX_REQUIRE(num_blocks >= 1 && block_size >= 1 && tokens_in_last_block >= 1 && tokens_in_last_block <= block_size,
               "vx_sdpa_paged_decode: bad block counts");
    AttnParams p = {};
    p.q = q;
    p.out = out;
    p.k = kv_pool;
    p.mode = MODE_PAGED;
    p.f16 = f16;
    p.num_q_heads = num_q_heads;
    p.num_kv_heads = num_kv_heads;
    p.head_dim = head_dim;
    p.scale = scale;
    p.block_table = block_table;
    p.block_size = block_size;
    p.kv_len = (num_blocks - 1) * block_size + tokens_in_last_block;
    return run_generic(be, p, 1);
}

int vx_sdpa_paged_decode(vx_backend *be, const float *q, const void *kv_pool, const int32_t *block_table, float *out,
                         int num_blocks, int block_size, int num_q_heads, int num_kv_heads, int head_dim, float scale,
                         int tokens_in_last_block) {
    return paged_single(be, q, kv_pool, 0, block_table, out, num_blocks, block_size, num_q_heads, num_kv_heads,
                        head_dim, scale, tokens_in_last_block);
}

int vx_sdpa_paged_decode_f16(vx_backend *be, const float *q, const void *kv_pool, const int32_t *block_table,
                             float *out, int num_blocks, int block_size, int num_q_heads, int num_kv_heads,
                             int head_dim, float scale, int tokens_in_last_block) {
    return paged_single(be, q, kv_pool, 1, block_table, out, num_blocks, block_size, num_q_heads, num_kv_heads,
                        head_dim, scale, tokens_in_last_block);
}

int vx_sdpa_paged_decode_batched(vx_backend *be, const float *q, const void *kv_pool, int pool_is_f16,
                                 const int32_t *const *block_tables, float *out, int batch_size, int max_blocks,
                                 int block_size, int num_q_heads, int num_kv_heads, int head_dim, float scale,
                                 const int32_t *seq_lens) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(q && kv_pool && block_tables && out && seq_lens, "vx_sdpa_paged_decode_batched: null pointer");
    VX_REQUIRE(!be->capturing, "vx_sdpa_paged_decode_batched takes host arrays and cannot be captured");
    if (batch_size == 0) return VX_OK;
    size_t pbytes = (size_t)batch_size * sizeof(void *), lbytes = (size_t)batch_size * sizeof(int32_t);
    VX_REQUIRE(pbytes + lbytes <= be->misc_ws_bytes, "vx_sdpa_paged_decode_batched: batch too large");
    int max_len = 0;
    for (int i = 0; i < batch_size; i++) {
        VX_REQUIRE(seq_lens[i] >= 1, "vx_sdpa_paged_decode_batched: sequence %d has length %d", i, seq_lens[i]);
        max_len = seq_lens[i] > max_len ? seq_lens[i] : max_len;
    }
    char *dev = (char *)be->misc_ws;
    VX_CHECK_HIP(hipMemcpyAsync(dev, block_tables, pbytes, hipMemcpyHostToDevice, be->stream));
    VX_CHECK_HIP(hipMemcpyAsync(dev + pbytes, seq_lens, lbytes, hipMemcpyHostToDevice, be->stream));
    VX_CHECK_HIP(hipStreamSynchronize(be->stream));  // host arrays belong to the caller after return
    const int32_t *d_lens = (const int32_t *)(dev + pbytes);
    // gather the per-sequence tables into one padded matrix when it fits the staging buffer
    const size_t moff = (pbytes + lbytes + 255) / 256 * 256;
    const size_t mbytes = (size_t)batch_size * max_blocks * sizeof(int32_t);
    if (max_blocks >= 1 && moff + mbytes <= be->misc_ws_bytes) {
        int32_t *matrix = (int32_t *)(dev + moff);
        gather_tables_kernel<<<batch_size, 256, 0, be->stream>>>((const int32_t *const *)dev, d_lens, matrix, max_blocks,
                                                                block_size);
        VX_CHECK_LAUNCH();
        return run_ragged(be, q, kv_pool, pool_is_f16, nullptr, matrix, nullptr, max_blocks, d_lens, out, batch_size,
                          block_size, num_q_heads, num_kv_heads, head_dim, scale, max_len);
    }
    return run_ragged(be, q, kv_pool, pool_is_f16, (const int32_t *const *)dev, nullptr, nullptr, max_blocks, d_lens,
                      out, batch_size, block_size, num_q_heads, num_kv_heads, head_dim, scale, max_len);
}

int vx_sdpa_paged_decode_ragged(vx_backend *be, const float *q, const void *kv_pool, int pool_is_f16,
                                const int32_t *block_tables, const int32_t *table_rows, const int32_t *kv_lens,
                                float *out, int batch, int max_blocks, int block_size, int num_q_heads,
                                int num_kv_heads, int head_dim, float scale, int max_kv_len) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(q && kv_pool && block_tables && kv_lens, "vx_sdpa_paged_decode_ragged: null pointer");
    VX_REQUIRE(max_kv_len <= max_blocks * block_size, "vx_sdpa_paged_decode_ragged: max_kv_len %d exceeds table capacity %d",
               max_kv_len, max_blocks * block_size);
    return run_ragged(be, q, kv_pool, pool_is_f16, nullptr, block_tables, table_rows, max_blocks, kv_lens, out, batch,
                      block_size,
                      num_q_heads, num_kv_heads, head_dim, scale, max_kv_len);
}

int vx_sdpa_paged_decode_ragged_noalloc(vx_backend *be, const float *q, const void *kv_pool, int pool_is_f16,
                                        const int32_t *block_tables, const int32_t *table_rows, const int32_t *kv_lens,
                                        float *out, int batch, int max_blocks, int block_size, int num_q_heads,
                                        int num_kv_heads, int head_dim, float scale, int max_kv_len) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(q && kv_pool && block_tables && kv_lens && out, "vx_sdpa_paged_decode_ragged_noalloc: null pointer");
    VX_REQUIRE(batch >= 0 && max_kv_len > 0 && max_kv_len <= max_blocks * block_size,
               "vx_sdpa_paged_decode_ragged_noalloc: max_kv_len %d not in 1..table capacity %d", max_kv_len, max_blocks * block_size);
    return run_ragged(be, q, kv_pool, pool_is_f16, nullptr, block_tables, table_rows, max_blocks, kv_lens, out, batch,
                      block_size, num_q_heads, num_kv_heads, head_dim, scale, max_kv_len, true);
}

size_t vx_sdpa_paged_decode_ragged_noalloc_bytes(vx_backend *be, int batch, int num_q_heads, int num_kv_heads, int head_dim,
                                                 int max_kv_len, size_t *capacity) {
    if (capacity) *capacity = FIXED_WS_BYTES;
    if (!be || batch < 1 || max_kv_len < 1 || !vx_sdpa_paged_decode_split_supported(1, HOT_BS, num_q_heads, num_kv_heads, head_dim))
        return 0;
    if (enter(be) != VX_OK) return 0;
    const int tps = split_tokens(be, head_dim, num_q_heads / num_kv_heads, batch, num_kv_heads, max_kv_len);
    return split_bytes(head_dim, batch, num_q_heads, ceil_div(max_kv_len, tps));
}

int vx_sdpa_paged_decode_split_supported(int pool_is_f16, int block_size, int num_q_heads, int num_kv_heads,
                                         int head_dim) {
    if (!pool_is_f16 || block_size != HOT_BS || num_kv_heads <= 0 || num_q_heads % num_kv_heads != 0) return 0;
    const int G = num_q_heads / num_kv_heads;
    return ((head_dim == 128 || head_dim == 64) && G >= 1 && G <= 8) || (head_dim == 128 && (G == 12 || G == 16)) ||
           (head_dim == 256 && G <= 2) ||
           ((head_dim == 80 || head_dim == 96) && G == 1);
}

int vx_sdpa_paged_decode_multiquery(vx_backend *be, const float *q, const void *kv_pool, int pool_is_f16,
                                    const int32_t *block_table, float *out, const int32_t *kv_lens, int num_blocks,
                                    int block_size, int num_q_heads, int num_kv_heads, int head_dim, float scale,
                                    int query_len) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(q && kv_pool && block_table && out && kv_lens, "vx_sdpa_paged_decode_multiquery: null pointer");
    VX_REQUIRE(num_blocks >= 1 && block_size >= 1 && query_len >= 0, "vx_sdpa_paged_decode_multiquery: bad counts");
    VX_REQUIRE(head_dim > 0 && num_kv_heads > 0 && num_q_heads % num_kv_heads == 0, "vx_sdpa_paged_decode_multiquery: bad head counts");
    // Chunks of a prompt and verification rows over an F16 pool: the matrix-core kernels (16-token blocks: a tile of
    // 16 query rows per wave straight from the pool; other block sizes: K/V tiles of 32 keys staged in LDS for 64
    // queries). A handful of rows, other head sizes and float32 pools keep the one-workgroup-per-query kernel.
    static const bool lds_tiles = getenv("VEXEL_HIP_MQ_LDS_TILES") != nullptr;  // (the LDS-tiled kernel instead, to compare)
    if (pool_is_f16 && query_len >= 16 && (head_dim == 64 || head_dim == 128) && ((uintptr_t)kv_pool % 16) == 0 &&
        block_size == HOT_BS && ((uintptr_t)q % 16) == 0 && ((uintptr_t)out % 16) == 0 && !lds_tiles) {
        constexpr int QT = 1;
        const int G = num_q_heads / num_kv_heads, combos = G * ceil_div(query_len, 16 * QT);
        // the blocks of a row tile shared out over 1, 2 or 4 waves: two waves per SIMD and more cover each other's
        // dependent chains (scores, softmax, weights, values), fewer leave the matrix cores waiting
        const long waves = (long)combos * num_kv_heads;
        const int share = waves >= 2048 ? 1 : (waves >= 1024 ? 2 : 4);
        const _Float16 *pool = (const _Float16 *)kv_pool;
        const int max_keys = num_blocks * block_size;
#define VX_MQ(DD, KK, NS)                                                                                                 \
    if (head_dim == DD && share == KK)                                                                                    \
        paged_mq_kernel<DD, QT, KK, NS><<<dim3(ceil_div(combos, NS), num_kv_heads), 64 * NS * KK, 0, be->stream>>>(         \
            q, pool, block_table, kv_lens, out, query_len, max_keys, num_q_heads, num_kv_heads, scale);
        // (heads of 128 with four shares: two pairs a workgroup, so that a wave keeps 256 registers)
        VX_MQ(128, 1, 4) VX_MQ(128, 2, 4) VX_MQ(128, 4, 2) VX_MQ(64, 1, 4) VX_MQ(64, 2, 4) VX_MQ(64, 4, 4)
#undef VX_MQ
        VX_CHECK_LAUNCH();
        return VX_OK;
    }
    if (pool_is_f16 && query_len >= 16 && (head_dim == 64 || head_dim == 128) && ((uintptr_t)kv_pool % 8) == 0) {
        PagedSrc src = {(const _Float16 *)kv_pool, block_table, kv_lens, block_size};
        dim3 grid(ceil_div(query_len, FA_BQ), num_q_heads);
        if (head_dim == 128)
            prefill_fa2_kernel<128, false, true><<<grid, 256, 0, be->stream>>>(q, nullptr, nullptr, out, query_len, num_q_heads,
                                                                               num_kv_heads, scale, 0.f, src);
        else
            prefill_fa2_kernel<64, false, true><<<grid, 256, 0, be->stream>>>(q, nullptr, nullptr, out, query_len, num_q_heads,
                                                                              num_kv_heads, scale, 0.f, src);
        VX_CHECK_LAUNCH();
        return VX_OK;
    }
    AttnParams p = {};
    p.q = q;
    p.out = out;
    p.k = kv_pool;
    p.mode = MODE_PAGED;
    p.f16 = pool_is_f16;
    p.num_q_heads = num_q_heads;
    p.num_kv_heads = num_kv_heads;
    p.head_dim = head_dim;
    p.scale = scale;
    p.block_table = block_table;
    p.block_size = block_size;
    p.kv_lens = kv_lens;
    return run_generic(be, p, query_len);
}

int vx_sdpa_paged_tree(vx_backend *be, const float *q, const void *kv_pool, int pool_is_f16,
                       const int32_t *block_table, float *out, const uint8_t *tree_mask, int tree_base, int block_size,
                       int num_q_heads, int num_kv_heads, int head_dim, float scale, int query_len) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(q && kv_pool && block_table && out && tree_mask, "vx_sdpa_paged_tree: null pointer");
    VX_REQUIRE(tree_base >= 0 && block_size >= 1 && query_len >= 0, "vx_sdpa_paged_tree: bad counts");
    AttnParams p = {};
    p.q = q;
    p.out = out;
    p.k = kv_pool;
    p.mode = MODE_PAGED;
    p.f16 = pool_is_f16;
    p.num_q_heads = num_q_heads;
    p.num_kv_heads = num_kv_heads;
    p.head_dim = head_dim;
    p.scale = scale;
    p.block_table = block_table;
    p.block_size = block_size;
    p.tree_mask = tree_mask;
    p.tree_base = tree_base;
    p.query_len = query_len;
    return run_generic(be, p, query_len);
}

int vx_sdpa_paged_tree_rows_per_entry(int pool_is_f16, int block_size, int num_q_heads, int num_kv_heads, int head_dim) {
    if (!pool_is_f16 || block_size != HOT_BS || num_kv_heads <= 0 || num_q_heads % num_kv_heads != 0) return 0;
    if (head_dim != 128 && head_dim != 64) return 0;
    const int G = num_q_heads / num_kv_heads;
    return G <= 8 ? 16 / G : 0;  // 16 queries (row, head) per K/V row fill the matrix-core tile: 16, 8, 5, 4, 3, 2, 2, 2 rows
}

int vx_sdpa_paged_tree_batched(vx_backend *be, const float *q, const void *kv_pool, const int32_t *block_tables,
                               int max_blocks, const int32_t *entry_table_rows, const int32_t *entry_kv_lens, int entries,
                               const int32_t *row_info, const uint8_t *tree_masks, const int32_t *mask_offsets, float *out,
                               int rows, int max_tree_rows, int num_q_heads, int num_kv_heads, int head_dim, float scale,
                               int max_kv_len) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(q && kv_pool && block_tables && entry_table_rows && entry_kv_lens && row_info && tree_masks && mask_offsets && out,
               "vx_sdpa_paged_tree_batched: null pointer");
    const int rg_max = vx_sdpa_paged_tree_rows_per_entry(1, HOT_BS, num_q_heads, num_kv_heads, head_dim);
    if (rg_max == 0) {
        set_error("vx_sdpa_paged_tree_batched: head geometry %d/%d x %d has no batched form", num_q_heads, num_kv_heads, head_dim);
        return VX_ERR_UNSUPPORTED;
    }
    // entries of rg_max rows, or - for small trees, which would mostly pad them - of half as many where that is whole
    const int rg = entries > 0 ? rows / entries : rg_max;
    VX_REQUIRE(entries >= 0 && rows == entries * rg && (rg == rg_max || (rg_max % 2 == 0 && rg == rg_max / 2)),
               "vx_sdpa_paged_tree_batched: %d rows are not %d entries of %d rows%s", rows, entries, rg_max,
               rg_max % 2 == 0 ? " or of half as many" : "");
    VX_REQUIRE(max_tree_rows >= 1 && max_tree_rows <= 64 && max_tree_rows <= head_dim,
               "vx_sdpa_paged_tree_batched: a tree of %d rows (at most 64)", max_tree_rows);
    VX_REQUIRE(((uintptr_t)kv_pool % 16) == 0 && max_kv_len >= 0, "vx_sdpa_paged_tree_batched: bad pool alignment / length");
    if (rows == 0) return VX_OK;
    const int max_splits = max_kv_len > 0 ? ceil_div(max_kv_len, TPW) : 1;
    const size_t need = (size_t)rows * num_q_heads * max_splits * (head_dim + 2) * sizeof(float);
    rc = ensure_ws(be, &be->attn_ws, &be->attn_ws_bytes, need, "attention");
    if (rc) return rc;
    be->split.batch = 0;
    const _Float16 *pool = (const _Float16 *)kv_pool;
    float *ws = (float *)be->attn_ws;
    const int G = num_q_heads / num_kv_heads;
    const dim3 grid(num_kv_heads, max_splits, entries);
    if (max_kv_len > 0) {
#define VX_TREE(DD, GG, RR)                                                                                              \
    if (head_dim == DD && G == GG && rg == RR)                                                                            \
        paged_decode_gqa_kernel<DD, GG, RR><<<grid, 256, 0, be->stream>>>(q, pool, block_tables, entry_table_rows, max_blocks, \
                                                                        entry_kv_lens, ws, num_q_heads, num_kv_heads, scale, \
                                                                        max_splits, nullptr, MergeOut{}, TPW);
#define VX_TREES(DD)                                                                                                       \
    VX_TREE(DD, 1, 16) VX_TREE(DD, 1, 8) VX_TREE(DD, 2, 8) VX_TREE(DD, 2, 4) VX_TREE(DD, 3, 5) VX_TREE(DD, 4, 4)         \
    VX_TREE(DD, 4, 2) VX_TREE(DD, 5, 3) VX_TREE(DD, 6, 2) VX_TREE(DD, 6, 1) VX_TREE(DD, 7, 2) VX_TREE(DD, 7, 1)           \
    VX_TREE(DD, 8, 2) VX_TREE(DD, 8, 1)
        VX_TREES(128) VX_TREES(64)
#undef VX_TREES
#undef VX_TREE
        VX_CHECK_LAUNCH();
    }
    const dim3 mgrid(num_q_heads, rows);
    if (head_dim == 128)
        tree_merge_kernel<128><<<mgrid, 128, 0, be->stream>>>(ws, q, pool, block_tables, max_blocks, (const int4 *)row_info,
                                                             tree_masks, mask_offsets, out, num_q_heads, num_kv_heads, scale,
                                                             max_splits);
    else
        tree_merge_kernel<64><<<mgrid, 64, 0, be->stream>>>(ws, q, pool, block_tables, max_blocks, (const int4 *)row_info,
                                                           tree_masks, mask_offsets, out, num_q_heads, num_kv_heads, scale,
                                                           max_splits);
    VX_CHECK_LAUNCH();
    return VX_OK;
}

}  // extern "C"
