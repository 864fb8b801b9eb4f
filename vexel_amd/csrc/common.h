// Internal declarations shared by the HIP translation units of libvexel_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include <string>
#include <unordered_map>
#include <vector>

#include "vexel_hip.h"

namespace vx {

void set_error(const char *fmt, ...);

#define VX_CHECK_HIP(expr)                                                                  \
    do {                                                                                    \
        hipError_t _e = (expr);                                                             \
        if (_e != hipSuccess) {                                                             \
            vx::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), __FILE__, __LINE__); \
            return VX_ERR_HIP;                                                              \
        }                                                                                   \
    } while (0)

#define VX_REQUIRE(cond, ...)            \
    do {                                 \
        if (!(cond)) {                   \
            vx::set_error(__VA_ARGS__);  \
            return VX_ERR_INVALID;       \
        }                                \
    } while (0)

// Checks the launch that was just issued (invalid configuration etc.).
#define VX_CHECK_LAUNCH() VX_CHECK_HIP(hipGetLastError())

struct PoolChunk {
    char *base;
    size_t size;
    size_t used;
};

}  // namespace vx

// chunk-parallel prepares: up to 512 rows x 64 chunks of 256 columns; two [64][512] float arrays of per-chunk sums of squares
#define VX_ROPE_TAB_ROWS 64
#define VX_ATTN_CNT 16384
#define VX_ROPE_TAB_PAIRS 128
#define VX_PREP_SYNC_ROWS 512
#define VX_PREP_SYNC_CHUNKS 64
#define VX_PREP_SYNC_BYTES (2 * VX_PREP_SYNC_CHUNKS * VX_PREP_SYNC_ROWS * 4)

struct vx_backend {
    int device = 0;
    hipStream_t stream = nullptr;
    bool capturing = false;
    const char *last_matmul = "";  // kernel family of the last quantized matmul launch (vx_last_matmul_kernel)

    // per-step pool (vx_alloc / vx_reset_pool)
    std::vector<vx::PoolChunk> chunks;
    size_t cur_chunk = 0;
    // permanent allocations (vx_alloc_permanent / vx_free)
    std::unordered_map<void *, size_t> permanent;

    // load-time repacked copies of quantized matrices for the decode-batch GEMM (qstream.hip), keyed by the raw
    // matrix' device address; each value is that file's record of the copy
    std::unordered_map<const void *, void *> packed;

    // library-owned scratch, grown on demand outside graph capture; scratch_gen counts the reallocations
    // (a captured graph holds the old addresses)
    uint64_t scratch_gen = 0;
    void *gemm_ws = nullptr;     // prepared (split, tiled) activations for the quantized GEMM
    size_t gemm_ws_bytes = 0;
    int prep_m = 0, prep_k = 0;  // shape of the activation currently prepared in gemm_ws
    int rowfac_slot = 0;         // which of the two row-factor arrays at the head of gemm_ws is current
    void *prep_sync = nullptr;   // per-chunk sums of squares of the chunk-parallel RMSNorm prepares (two slots)
    int prep_norm_k = 0;         // > 0: the prepared activation is x*w of an RMSNorm over that many columns whose
    float prep_norm_eps = 0.f;   //      1/rms is still to be taken from the current slot of prep_sync
    void *part_ws = nullptr;     // split-K partial sums
    size_t part_ws_bytes = 0;
    void *part_ws2 = nullptr;    // a second one: the V projection's, where V is a launch of its own beside Q|K
    size_t part_ws2_bytes = 0;
    // cos / sin of every (row, pair) of the step's positions (vx_rope_table_prepare): [VX_ROPE_TAB_ROWS][head_dim/2]
    // float2, valid while the key below matches and the library has written nothing since (write_epoch)
    void *rope_tab = nullptr;
    const int32_t *rope_tab_pos = nullptr;
    int rope_tab_rows = 0, rope_tab_dim = 0;
    float rope_tab_theta = 0.f;
    uint64_t rope_tab_epoch = 0, write_epoch = 1;
    // cos / sin of vx_paged_kv_copy_shifted's rotation per pair, kept while (shift, theta, head_dim) stay the same
    void *shift_tab = nullptr;
    int shift_tab_shift = 0, shift_tab_dim = 0;
    float shift_tab_theta = 0.f;
    void *attn_ws = nullptr;     // split-KV partial results
    void *attn_fixed_ws = nullptr;  // this device's copy of the fixed-size partial-sum area (never allocated or freed)
    // attention left in split form by vx_sdpa_paged_decode_ragged(out = NULL), to be merged by vx_decode_ffn
    struct {
        int batch = 0, num_q_heads = 0, head_dim = 0, max_splits = 0, tokens_per_split = 0;
        const int32_t *kv_lens = nullptr;
        int merged = 0;  // the attention kernel also left the merged rows as the prepared activation (gemm_ws)
        const float *plain = nullptr;  // a single row: the attention kernel also left the merged row here, as floats
    } split;
    // the decode attention kernel merges its own splits where the geometry allows (vx_backend_set_attn_merge; the
    // initial value is off when VEXEL_HIP_NO_ATTN_MERGE is set in the environment at vx_backend_create)
    bool attn_merge = true;
    int32_t *attn_cnt = nullptr;  // arrival counters of the merging attention kernel, VX_ATTN_CNT of them, zero between launches
    size_t attn_ws_bytes = 0;
    // Work lists of the ragged decode attention, written on the device by vx_pack_batch next to kv_lens:
    // buf[0] = number of items, then from buf[4] one record of four ints per item (batch index, split, kv
    // length, block-table row), full splits first, then the sequences' partial last splits from the longest
    // down; items of ATTN_TPW tokens, with room for `cap` of them, and behind that room (from buf[4 (cap + 1)])
    // the same for items of ATTN_TPW / 2 tokens. Valid for attention calls that pass the same kv_lens and table-row pointers and batch, until the
    // library is asked to write into the kv_lens array by other means.
    struct {
        int32_t *buf = nullptr;
        size_t bytes = 0;
        const int32_t *kv_lens = nullptr;
        const int32_t *table_rows = nullptr;
        int batch = 0;
        size_t cap = 0;
        bool valid = false;
    } items;
    float *ones = nullptr;       // 64 floats of 1.0 on the device (row factors of an unscaled activation)
    void *sample_ws = nullptr;   // probabilities and sort keys of vx_sample_rows
    size_t sample_ws_bytes = 0;
    void *misc_ws = nullptr;     // small device staging (pointer tables, argmax result)
    size_t misc_ws_bytes = 0;
    void *host_stage = nullptr;  // pinned host staging
    size_t host_stage_bytes = 0;

    hipEvent_t ev0 = nullptr, ev1 = nullptr;
};

struct vx_graph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
};

namespace vx {

// qstream.hip: drops the packed copy of the raw matrix at `raw` (if any) / every packed copy of the backend / the
// copies of matrices that [dst, dst + bytes) overlaps.
void stream_drop_packed(vx_backend *be, const void *raw);
void stream_drop_all(vx_backend *be);
void stream_written(vx_backend *be, const void *dst, size_t bytes);

constexpr int ATTN_TPW = 512;  // tokens of one (sequence, kv head) that one attention workgroup takes

// Drops the attention work list when [dst, dst + bytes) overlaps the kv_lens array it was built from.
inline void items_written(vx_backend *be, const void *dst, size_t bytes) {
    be->write_epoch++;  // the library wrote into a caller's buffer: a kept RoPE table may describe other positions now
    if (!be->packed.empty()) stream_written(be, dst, bytes);  // a packed copy of rewritten rows is stale
    if (!be->items.valid) return;
    const char *a = (const char *)dst, *k = (const char *)be->items.kv_lens;
    if (a < k + (size_t)be->items.batch * 4 && k < a + bytes) be->items.valid = false;
}

// Makes be->device current on the calling thread (Go moves goroutines across OS threads).
int enter(vx_backend *be);
// Ensures a library scratch buffer holds at least `bytes`; fails during capture if it must grow.
int ensure_ws(vx_backend *be, void **ptr, size_t *cap, size_t bytes, const char *what);
// Looks up, once per backend and with its device current, where that device keeps the fixed partial-sum area of
// vx_sdpa_paged_decode_ragged_noalloc (attention.hip); called by vx_backend_create.
int attn_noalloc_init(vx_backend *be);

// qmatvec.hip: out[n] = a . W[n] (+ residual[n]) for one activation row; VX_ERR_UNSUPPORTED (nothing launched, no
// error text) when the shape is outside the kernel's range.
int run_matvec(vx_backend *be, int fmt, const float *a, const void *b, float *out, const float *residual, int n, int k);
// Where the matrix-vector kernel takes its activation row from: x itself; x * norm_w with the results divided
// by rms(x) (RMSNorm folded in); or the attention output of one query merged from its split-KV partials.
// RoPE (interleaved pairs over the whole head) and the paged K/V store as the epilogue of a single row's fused
// Q|K|V matrix-vector product: rows [0, qd) are Q, [qd, qd + kvd) K, then V. q_out == nullptr: none.
struct MatvecRope {
    float *q_out = nullptr;
    void *pool = nullptr;          // F16 paged pool of the layer
    const int32_t *slot = nullptr; // the row's slot in the pool (device)
    const float2 *cs_tab = nullptr; // (cos, sin) of the row's position per pair (vx_rope_table_prepare)
    int qd = 0, kvd = 0, head_dim = 0, block_size = 0;
};
struct MatvecSource {
    MatvecRope rope;
    const float *x = nullptr;
    const float *norm_w = nullptr;
    float eps = 0.f;
    const float *attn_partial = nullptr;
    const int32_t *kv_len = nullptr;
    int head_dim = 0, max_splits = 0, tokens_per_split = 0;
};
// Whether run_matvec_fused would take these matrices (format, K, alignment).
bool matvec_ok(int fmt, const void *const *ws, const int *ns, int nw, int k);
// Up to three matrices of one format and K with their rows concatenated (out has the summed height); pair != 0:
// two matrices of equal height n, out[i] = silu(W0[i] . a) * (W1[i] . a), i < n.
int run_matvec_fused(vx_backend *be, int fmt, const void *const *ws, const int *ns, int nw, int k, const MatvecSource &src,
                     float *out, const float *residual, int pair);

static inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
static inline int64_t ceil_div64(int64_t a, int64_t b) { return (a + b - 1) / b; }

}  // namespace vx
