// Continuous-batching step metadata built on the device (vx_pack_batch).
//
// Host restatement of what this replaces: the per-sequence loop of
// inference/runtime/decode.go:642-650 calling GPUBlockPool.StoreKV for every sequence
// (inference/runtime/gpu_block_pool.go:234-252: ensure blocks up to (endPos-1)/blockSize by
// popping the free list's tail, slot = (table[pos/bs], pos%bs)) and the length bookkeeping
// of gpu_block_pool.go:318-320,354-363. Because the host loop visits sequences in batch
// order and every layer's free list evolves identically, sequence i's new blocks are the
// entries free[F-1-rank_i-j], rank_i = exclusive prefix sum of the blocks needed by the
// sequences before it. Two prefix scans (blocks needed, new tokens) give every output.
#include "common.h"

using namespace vx;

namespace {

constexpr int PK_THREADS = 1024;

// Exclusive scan over blockDim.x values held one per thread; returns the exclusive prefix and
// writes the total to *total (same value in every thread). Each wave scans its 64 values by shuffles, the first wave
// then the 16 waves' sums (sm: at least PK_THREADS / 64 ints).
__device__ int block_exclusive_scan(int v, int *sm, int *total) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    constexpr int NWAVES = PK_THREADS / 64;
    int incl = v;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const int t = __shfl_up(incl, off, 64);
        if (lane >= off) incl += t;
    }
    __syncthreads();  // (whoever still reads sm from an earlier use is done)
    if (lane == 63) sm[wave] = incl;
    __syncthreads();
    if (wave == 0) {
        int w = lane < NWAVES ? sm[lane] : 0;
#pragma unroll
        for (int off = 1; off < NWAVES; off <<= 1) {
            const int t = __shfl_up(w, off, 64);
            if (lane >= off) w += t;
        }
        if (lane < NWAVES) sm[lane] = w;          // inclusive sums of the waves
    }
    __syncthreads();
    const int before = wave > 0 ? sm[wave - 1] : 0;
    *total = sm[NWAVES - 1];
    __syncthreads();  // (the caller may write sm next)
    return before + incl - v;
}

__global__ void __launch_bounds__(PK_THREADS) pack_batch_kernel(
    const int32_t *seq_slots, const int32_t *positions, const int32_t *q_lens, int batch, int total_tokens,
    int32_t *block_tables, int max_blocks, int32_t *num_blocks, int32_t *free_list, int32_t *free_count,
    int block_size, int32_t *cu_seqlens, int32_t *token_pos, int32_t *slot_mapping, int32_t *kv_lens,
    int32_t *status, int32_t *items, int items_cap) {
    __shared__ int sm[PK_THREADS];
    __shared__ int s_cu[PK_THREADS + 1];
    const int tid = threadIdx.x;
    const bool act = tid < batch;
    int slot = 0, pos = 0, ql = 0, have = 0, need = 0;
    if (act) {
        slot = seq_slots[tid];
        pos = positions[tid];
        ql = q_lens ? q_lens[tid] : 1;
        have = num_blocks[slot];
        int end = pos + ql;
        int want = end > 0 ? (end - 1) / block_size + 1 : 0;
        need = want > have ? want - have : 0;
    }
    int total_need, total_q;
    const int rank = block_exclusive_scan(need, sm, &total_need);
    const int cu = block_exclusive_scan(ql, sm, &total_q);
    const int F = *free_count;
    bool fail = total_need > F || total_q != total_tokens;
    if (act && have + need > max_blocks) fail = true;
    // any thread's failure fails the step
    const bool any_fail = __syncthreads_or(fail ? 1 : 0) != 0;
    if (any_fail) {
        if (tid == 0) {
            *status = 1;
            if (items) {
                items[0] = 0;
                items[(items_cap + 1) * 4] = 0;
            }
        }
        return;
    }
    if (items) {
        // The attention work lists: one item per ATTN_TPW tokens of a sequence, and a second list in items of half
        // that for the kernels that take half as many tokens per workgroup (grouped queries). Equal (full) items
        // first, in batch order; then the partial last items from the longest down, so that the kernel's last
        // workgroups are its smallest. The second list sits behind the first one's capacity.
        const int len = act ? pos + ql : 0;
        for (int which = 0; which < 2; which++) {
            const int tpw = which == 0 ? ATTN_TPW : ATTN_TPW / 2;
            const int cap = which == 0 ? items_cap : 2 * items_cap;
            int32_t *list = which == 0 ? items : items + (items_cap + 1) * 4;
            const int full = len / tpw, rest = len % tpw;
            int total_full;
            const int off = block_exclusive_scan(full, sm, &total_full);
            sm[tid] = rest;
            __syncthreads();
            int before = 0, partials = 0;  // partial items ahead of this one; partial items in all
            if (act || tid == 0) {  // (the threads without a sequence write nothing below)
                for (int j = 0; j < batch; j++) {
                    const int rj = sm[j];
                    partials += rj > 0;
                    before += (rj > rest) || (rj == rest && rj > 0 && j < tid);
                }
            }
            __syncthreads();
            const int n_items = total_full + partials;
            if (act && n_items <= cap) {
                int4 *rec = (int4 *)(list + 4);  // one 16-byte record per item: everything a workgroup needs to start
                for (int s2 = 0; s2 < full; s2++) rec[off + s2] = make_int4(tid, s2, len, slot);
                if (rest > 0) rec[total_full + before] = make_int4(tid, full, len, slot);
            }
            if (tid == 0) list[0] = n_items <= cap ? n_items : -1;  // -1: the list did not fit, not to be used
        }
    }
    if (act) {
        for (int j = 0; j < need; j++)
            block_tables[(size_t)slot * max_blocks + have + j] = free_list[F - 1 - (rank + j)];
        num_blocks[slot] = have + need;
        kv_lens[tid] = pos + ql;
        s_cu[tid] = cu;
        cu_seqlens[tid] = cu;
    }
    if (tid == 0) {
        *free_count = F - total_need;
        *status = 0;
        s_cu[batch] = total_q;
        cu_seqlens[batch] = total_q;
    }
    __syncthreads();
    for (int t = tid; t < total_q; t += PK_THREADS) {
        // binary search: largest i with s_cu[i] <= t
        int lo = 0, hi = batch - 1;
        while (lo < hi) {
            int mid = (lo + hi + 1) >> 1;
            if (s_cu[mid] <= t)
                lo = mid;
            else
                hi = mid - 1;
        }
        const int p = positions[lo] + (t - s_cu[lo]);
        token_pos[t] = p;
        const int sl = seq_slots[lo];
        slot_mapping[t] = block_tables[(size_t)sl * max_blocks + p / block_size] * block_size + p % block_size;
    }
}

}  // namespace

extern "C" int vx_pack_batch(vx_backend *be, const int32_t *seq_slots, const int32_t *positions,
                             const int32_t *q_lens, int batch, int total_tokens, int32_t *block_tables,
                             int max_blocks, int32_t *num_blocks, int32_t *free_list, int32_t *free_count,
                             int block_size, int32_t *cu_seqlens, int32_t *token_pos, int32_t *slot_mapping,
                             int32_t *kv_lens, int32_t *status) {
    int rc = enter(be);
    if (rc) return rc;
    be->write_epoch++;  // positions and slots change
    VX_REQUIRE(seq_slots && positions && block_tables && num_blocks && free_list && free_count && cu_seqlens &&
                   token_pos && slot_mapping && kv_lens && status,
               "vx_pack_batch: null pointer");
    VX_REQUIRE(batch >= 1 && batch <= PK_THREADS, "vx_pack_batch: batch %d not in 1..%d", batch, PK_THREADS);
    VX_REQUIRE(block_size >= 1 && max_blocks >= 1 && total_tokens >= 0, "vx_pack_batch: bad sizes");
    // room for the attention work list: every sequence at the longest context its block table allows
    const size_t per_seq = ((size_t)max_blocks * block_size + ATTN_TPW - 1) / ATTN_TPW;
    const size_t cap = (size_t)batch * per_seq;
    int32_t *items = nullptr;
    be->items.valid = false;
    if (batch <= 32767 && per_seq <= 65535 &&
        ensure_ws(be, (void **)&be->items.buf, &be->items.bytes, (3 * cap + 2) * 4 * sizeof(int32_t), "attention work list") == VX_OK)
        items = be->items.buf;
    pack_batch_kernel<<<1, PK_THREADS, 0, be->stream>>>(seq_slots, positions, q_lens, batch, total_tokens,
                                                        block_tables, max_blocks, num_blocks, free_list, free_count,
                                                        block_size, cu_seqlens, token_pos, slot_mapping, kv_lens,
                                                        status, items, (int)cap);
    VX_CHECK_LAUNCH();
    if (items) {
        be->items.kv_lens = kv_lens;
        be->items.table_rows = seq_slots;
        be->items.batch = batch;
        be->items.cap = cap;
        be->items.valid = true;
    }
    return VX_OK;
}

namespace {
__global__ void decode_advance_kernel(int32_t *tokens, int32_t *positions, const int32_t *next_tokens,
                                      int32_t *out_log, int32_t *step_counter, int batch) {
    const int i = threadIdx.x;
    const int step = *step_counter;
    __syncthreads();
    if (i < batch) {
        const int t = next_tokens[i];
        out_log[(size_t)step * batch + i] = t;
        tokens[i] = t;
        positions[i] += 1;
    }
    if (i == 0) *step_counter = step + 1;
}
}  // namespace

extern "C" int vx_decode_advance(vx_backend *be, int32_t *tokens, int32_t *positions, const int32_t *next_tokens,
                                 int32_t *out_log, int32_t *step_counter, int batch) {
    int rc = enter(be);
    if (rc) return rc;
    be->write_epoch++;  // positions move on
    VX_REQUIRE(tokens && positions && next_tokens && out_log && step_counter, "vx_decode_advance: null pointer");
    VX_REQUIRE(batch >= 1 && batch <= PK_THREADS, "vx_decode_advance: batch %d not in 1..%d", batch, PK_THREADS);
    decode_advance_kernel<<<1, PK_THREADS, 0, be->stream>>>(tokens, positions, next_tokens, out_log, step_counter,
                                                            batch);
    VX_CHECK_LAUNCH();
    return VX_OK;
}
