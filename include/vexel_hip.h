/*
 * vexel_hip.h -- C ABI of libvexel_hip.so, an MI355X (gfx950) compute backend for
 * vexel's batched-decode path.
 *
 * Every entry point replaces one method of the Go interfaces in
 * inference/backend/backend.go of keithballinger/vexel (cited per function as
 * backend.go:LINE). A cgo shim binds them 1:1. Conventions:
 *   - every device pointer argument is a raw device address (the shim passes
 *     DevicePtr.Addr()+DevicePtr.Offset(), tensor/device.go:38-51);
 *   - functions return VX_OK (0) or an error code; vx_last_error() gives the text.
 *     The Go methods return nothing: the shim panics on non-zero, as the Metal
 *     backend panics on a missing pipeline (backend/metal/backend.go:775);
 *   - all work is enqueued on the backend's single HIP stream (FIFO, like the one
 *     Metal command queue); only vx_sync, vx_to_host and vx_argmax wait for it;
 *   - the library is not re-entrant: one thread at a time per backend, which is how
 *     the reference's scheduler goroutine uses it (scheduler/scheduler.go:126-165).
 */
#ifndef VEXEL_HIP_H
#define VEXEL_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct vx_backend vx_backend;

enum {
    VX_OK = 0,
    VX_ERR_INVALID = 1,     /* bad argument (shape, alignment, null pointer) */
    VX_ERR_OOM = 2,         /* device allocation failed */
    VX_ERR_HIP = 3,         /* a HIP runtime call failed */
    VX_ERR_UNSUPPORTED = 4  /* unknown weight format, or a fused form the given shapes do not have */
};

/* Weight formats for the generic entry points (GGUF block layouts,
 * inference/pkg/gguf/dequant.go). */
enum { VX_Q4_0 = 1, VX_Q8_0 = 2, VX_Q4_K = 3, VX_Q6_K = 4, VX_Q5_0 = 5, VX_Q5_K = 6, VX_BF16 = 7 };

/* ---- lifetime / errors ------------------------------------------------------ */
/* metal.NewBackend (backend/metal/backend.go:238-409); Backend.Device (backend.go:311) */
int vx_backend_create(int device_id, vx_backend **out);
void vx_backend_destroy(vx_backend *be);
/* Whether the ragged decode attention kernel merges the partial results of a sequence's splits itself (the workgroup
 * that finishes a sequence's columns last does it; default) or leaves them to a merge step of the consumer
 * (on = 0). Both give the same bits; the in-kernel form saves a launch per layer and orders its memory traffic by
 * properties of this GPU family's caches rather than by HIP's memory model, so the switch exists to fall back and
 * to compare. The environment variable VEXEL_HIP_NO_ATTN_MERGE, read at vx_backend_create, sets the initial value
 * to off. No counterpart in the reference. */
int vx_backend_set_attn_merge(vx_backend *be, int on);
int vx_backend_device(const vx_backend *be);
const char *vx_last_error(void);

/* ---- memory (backend.go:313-331, 8-10, 38-43) ------------------------------- */
/* Backend.Alloc: buffer from the per-step pool, recycled by vx_reset_pool. NULL on failure. */
void *vx_alloc(vx_backend *be, size_t bytes);
/* AllocPermanent (runtime/gpu_block_pool.go:73-81, runtime/block.go:445-447): survives resets. */
void *vx_alloc_permanent(vx_backend *be, size_t bytes);
/* Backend.Free: releases a permanent buffer; a pool buffer is left to the next reset. */
void vx_free(vx_backend *be, void *ptr);
/* PoolResetter.ResetPool (backend.go:8-10): every vx_alloc buffer becomes reusable. */
void vx_reset_pool(vx_backend *be);
/* Backend.ToDevice / ToHost: the host buffer may be reused as soon as the call returns. */
int vx_to_device(vx_backend *be, void *dst, const void *src_host, size_t bytes);
int vx_to_host(vx_backend *be, void *dst_host, const void *src, size_t bytes);
/* Backend.Sync */
int vx_sync(vx_backend *be);
/* BufferCopier.CopyBuffer / CopyBufferBatched (backend.go:38-43): device to device. */
int vx_copy_buffer(vx_backend *be, const void *src, size_t src_off, void *dst, size_t dst_off, size_t bytes);
/* Batcher (backend.go:25-34): one in-order stream needs no batching or barriers; kept
 * so the shim can satisfy the interface. */
int vx_begin_batch(vx_backend *be);
int vx_end_batch(vx_backend *be);
int vx_memory_barrier(vx_backend *be);

/* ---- dense F32 kernels (backend.go:337-389) --------------------------------- */
int vx_matmul(vx_backend *be, const float *a, const float *b, float *out, int m, int n, int k);             /* :338 */
int vx_matmul_transposed(vx_backend *be, const float *a, const float *b, float *out, int m, int n, int k); /* :341 */
int vx_rmsnorm(vx_backend *be, const float *x, const float *weight, float *out, int rows, int cols, float eps); /* :345 */
/* :352. k may be NULL. rope_dim 0 = full head_dim. */
int vx_rope(vx_backend *be, float *q, float *k, int head_dim, int num_heads, int num_kv_heads, int seq_len,
            int start_pos, int rope_dim, float theta, int rope_neox);
/* RoPEShift of the CPU backend (backend/cpu/backend.go:244-276, interface.go:37-44): every K vector of
 * k[num_tokens, num_kv_heads, head_dim] is rotated by the angle of position `shift` (interleaved pairs), which
 * turns RoPE(p) into RoPE(p + shift); shift 0 changes nothing. */
int vx_rope_shift(vx_backend *be, float *k, int head_dim, int num_kv_heads, int num_tokens, int shift, float theta);
int vx_silu(vx_backend *be, const float *x, float *out, int n);                           /* :356 */
int vx_silu_mul(vx_backend *be, const float *gate, const float *up, float *out, int n);   /* :360 */
int vx_softmax(vx_backend *be, const float *x, float *out, int rows, int cols);           /* :364 */
int vx_add(vx_backend *be, const float *a, const float *b, float *out, int n);            /* :367 */
int vx_mul(vx_backend *be, const float *a, const float *b, float *out, int n);            /* :370 */
/* :374. ids int32 on device; an id outside [0,vocab) leaves its output row untouched. */
int vx_embedding(vx_backend *be, const int32_t *ids, int num_tokens, const float *table, float *out,
                 int vocab_size, int dim);
/* :382. K/V head-major [numKVHeads, kv_head_stride/headDim, headDim]. */
int vx_sdpa(vx_backend *be, const float *q, const float *k, const float *v, float *out, int kv_len,
            int num_q_heads, int num_kv_heads, int head_dim, float scale, int kv_head_stride);
/* :389. Q/K/V/out token-major [seqLen, heads, headDim], causal. */
int vx_sdpa_prefill(vx_backend *be, const float *q, const float *k, const float *v, float *out, int seq_len,
                    int num_q_heads, int num_kv_heads, int head_dim, float scale);

/* ---- optional interfaces of other architectures (backend.go:205-263; CPU bodies in backend/cpu/cpu.go) ---- */
/* LayerNormOps.LayerNorm (backend.go:207-212, cpu.go:404-436): (x - mean) / sqrt(var + eps) * weight + bias per
 * row, var = the mean squared deviation (divisor cols). */
int vx_layernorm(vx_backend *be, const float *x, const float *weight, const float *bias, float *out, int rows,
                 int cols, float eps);
/* GELUOps (backend.go:216-226, cpu.go:440-473): 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))); gelu(gate) * up. */
int vx_gelu(vx_backend *be, const float *x, float *out, int n);
int vx_gelu_mul(vx_backend *be, const float *gate, const float *up, float *out, int n);
/* BiasOps.AddBias (backend.go:249-253, cpu.go:476-487): out[r][c] = x[r][c] + bias[c]; out may be x. */
int vx_add_bias(vx_backend *be, const float *x, const float *bias, float *out, int rows, int cols);
/* ScaleOps.ScaleBuffer (backend.go:257-261, cpu.go:558-563): buf[i] *= scale in place. */
int vx_scale_buffer(vx_backend *be, float *buf, float scale, int n);
/* SoftCapAttentionOps (backend.go:231-241, cpu.go:705-841): vx_sdpa / vx_sdpa_prefill whose scaled scores pass
 * through softcap * tanh(score / softcap) before the softmax; softcap 0 is the plain kernel. */
int vx_sdpa_softcap(vx_backend *be, const float *q, const float *k, const float *v, float *out, int kv_len,
                    int num_q_heads, int num_kv_heads, int head_dim, float scale, float softcap, int kv_head_stride);
int vx_sdpa_prefill_softcap(vx_backend *be, const float *q, const float *k, const float *v, float *out, int seq_len,
                            int num_q_heads, int num_kv_heads, int head_dim, float scale, float softcap);
/* ModelRuntime.ApplyFinalLogitSoftCap (runtime/model.go:336-350; the reference runs it on the host copy of the logits
 * a request is sampled from): logits[i] = cap * tanh(logits[i] / cap) in float64, in place; cap <= 0 = off. */
int vx_logit_softcap(vx_backend *be, float *logits, int n, float cap);
/* ScaledRoPEOps.RoPEWithFreqs (backend.go:247-249, cpu.go:308-375): RoPE over the whole head with pair j turning
 * by position * freqs[j] (head_dim / 2 floats on the device). k may be NULL. */
int vx_rope_with_freqs(vx_backend *be, float *q, float *k, const float *freqs, int head_dim, int num_heads,
                       int num_kv_heads, int seq_len, int start_pos, int rope_neox);

/* ---- Medusa prediction heads (inference/medusa/heads.go) ---- */
/* Heads.ForwardAll (heads.go:83-128) for `rows` (<= 8) hidden states at once: for every head h,
 * intermediate[h][r] = SiLU(hidden[r] . FC1[h]) and logits[h][r] = intermediate[h][r] . FC2[h], with SiLU(x) =
 * x / (1 + exp(-x)). fc1 [heads][hidden][hidden] and fc2 [heads][hidden][vocab] are float32 with the input index
 * first, as Head.FC1 / FC2 hold them; hidden [rows][hidden]; intermediate [heads][rows][hidden] (caller's scratch);
 * logits [heads][rows][vocab]. hidden and vocab must be multiples of 4. */
int vx_medusa_forward(vx_backend *be, const float *hidden, const float *fc1, const float *fc2, float *intermediate,
                      float *logits, int rows, int num_heads, int hidden_size, int vocab_size);
/* topK (heads.go:146-171) per row of x [rows][n]: the indices of the k largest values, largest first, a tie to the
 * lower index; out_idx [rows][k] int32, out_val [rows][k] (may be NULL) on the device; k <= min(n, 256). Values not above -MaxFloat32
 * and NaN are never taken: the index is then -1. */
int vx_topk_rows(vx_backend *be, const float *x, int rows, int n, int k, int32_t *out_idx, float *out_val);

/* ArgmaxOps.Argmax (backend.go:199-203): first index of the strict maximum; waits for the stream. */
int vx_argmax(vx_backend *be, const float *input, int n, int *out_index);

/* ---- QuantizedMatMul (backend.go:47-81): C[M,N] = A[M,K] * B^T, B raw GGUF blocks --- */
int vx_matmul_q4_0(vx_backend *be, const float *a, const void *b, float *out, int m, int n, int k); /* :50 */
int vx_matmul_q4_k(vx_backend *be, const float *a, const void *b, float *out, int m, int n, int k); /* :55 */
int vx_matmul_q6_k(vx_backend *be, const float *a, const void *b, float *out, int m, int n, int k); /* :60 */
int vx_matmul_q8_0(vx_backend *be, const float *a, const void *b, float *out, int m, int n, int k); /* :75 */
/* Not in any benchmark config. Q5_K and Q5_0 (pkg/gguf/dequant.go:423-500, 100-145) run on the same two kernels
 * as the formats above (the streaming matrix-vector kernel for one row, the MFMA kernel for more); BF16
 * (dequant.go:215-228) has one wave per weight row on the exact values only. */
int vx_matmul_q5_k(vx_backend *be, const float *a, const void *b, float *out, int m, int n, int k); /* :65 */
int vx_matmul_q5_0(vx_backend *be, const float *a, const void *b, float *out, int m, int n, int k); /* :70 */
int vx_matmul_bf16(vx_backend *be, const float *a, const void *b, float *out, int m, int n, int k); /* :80 */

/* ---- PagedKVOps (backend.go:415-466) ----------------------------------------- */
/* Pool layout per physical block: K[blockSize,numKVHeads,headDim] then V[same]
 * (runtime/gpu_block_pool.go:15-19). */
int vx_reshape_paged_kv(vx_backend *be, const float *src, void *dst_base, const int32_t *page_table,
                        const int32_t *block_offsets, int num_tokens, int num_kv_heads, int head_dim,
                        int block_size, int is_value);                                             /* :424 */
int vx_reshape_paged_kv_f16(vx_backend *be, const float *src, void *dst_base, const int32_t *page_table,
                            const int32_t *block_offsets, int num_tokens, int num_kv_heads, int head_dim,
                            int block_size, int is_value);                                         /* :457 */
int vx_sdpa_paged_decode(vx_backend *be, const float *q, const void *kv_pool, const int32_t *block_table,
                         float *out, int num_blocks, int block_size, int num_q_heads, int num_kv_heads,
                         int head_dim, float scale, int tokens_in_last_block);                     /* :432 */
int vx_sdpa_paged_decode_f16(vx_backend *be, const float *q, const void *kv_pool, const int32_t *block_table,
                             float *out, int num_blocks, int block_size, int num_q_heads, int num_kv_heads,
                             int head_dim, float scale, int tokens_in_last_block);                 /* :436 */
/* :447. block_tables: host array of batch_size device pointers; seq_lens: host array.
 * pool_is_f16 selects the pool element type (the Go method is called on an F32 pool). */
int vx_sdpa_paged_decode_batched(vx_backend *be, const float *q, const void *kv_pool, int pool_is_f16,
                                 const int32_t *const *block_tables, float *out, int batch_size, int max_blocks,
                                 int block_size, int num_q_heads, int num_kv_heads, int head_dim, float scale,
                                 const int32_t *seq_lens);
/* :463. kv_lens: device int32[query_len]; query i attends to positions < kv_lens[i]. */
int vx_sdpa_paged_decode_multiquery(vx_backend *be, const float *q, const void *kv_pool, int pool_is_f16,
                                    const int32_t *block_table, float *out, const int32_t *kv_lens,
                                    int num_blocks, int block_size, int num_q_heads, int num_kv_heads,
                                    int head_dim, float scale, int query_len);

/* ---- batched-decode entry points the reference lacks ------------------------- */
/* (its batch is a host loop, runtime/decode.go:623-650; these run the whole batch in one
 * launch and are defined per sequence by the sequential semantics above.) */

/* gguf.Dequantize on the device (pkg/gguf/dequant.go:503-538), bit-exact; used for the
 * loader rule that keeps token_embd in F32 (runtime/loader.go:275-288). n % block == 0. */
int vx_dequantize(vx_backend *be, int fmt, const void *src, float *dst, int64_t n);

/* Any of the four formats, with an optional fused residual: out = (residual ? residual : 0) + A*B^T.
 * The add is the same single float32 add Backend.Add would do (runtime/block.go:990,1077). */
int vx_matmul_quant(vx_backend *be, int fmt, const float *a, const void *b, float *out, const float *residual,
                    int m, int n, int k);

/* "Prepare once, multiply many": the MFMA path consumes activations in a split, tiled f16 form
 * kept in a backend-owned slot. A prepare call fills the slot from an [m,k] activation; every
 * following vx_matmul_quant_prepared with the same (m,k) multiplies that activation by one more
 * weight (Q/K/V share one, gate/up share one). k must be a multiple of 256 and pointers
 * 16-byte aligned. Results equal vx_matmul_quant on the same values bit for bit.
 *   vx_prepare_act       a itself
 *   vx_rmsnorm_prepare   Backend.RMSNorm(x, weight) (backend.go:345); also stored to out when out != NULL
 *   vx_silu_mul_prepare  Backend.SiLUMul(gate, up) (backend.go:360); also stored to out when out != NULL
 *   vx_gelu_mul_prepare  GELUMul(gate, up) (backend.go:222-224; GeGLU layers); also stored to out when out != NULL
 *   vx_gelu_prepare      GELU(x) (backend.go:216-220; the GELU MLP's fc1 output); also stored to out when out != NULL
 * vx_matmul_quant_prepared with out == NULL (and residual == NULL) issues the projection's launch alone, as the
 * fused decode blocks do: the sums of its K slices stay in a backend workspace that only the library reads. That
 * form exists to time the launch by itself; it returns nothing to the caller. */
int vx_prepare_act(vx_backend *be, const float *a, int m, int k);
int vx_rmsnorm_prepare(vx_backend *be, const float *x, const float *weight, float *out, int rows, int cols, float eps);
int vx_silu_mul_prepare(vx_backend *be, const float *gate, const float *up, float *out, int rows, int cols);
int vx_gelu_mul_prepare(vx_backend *be, const float *gate, const float *up, float *out, int rows, int cols);
int vx_gelu_prepare(vx_backend *be, const float *x, float *out, int rows, int cols);
int vx_matmul_quant_prepared(vx_backend *be, int fmt, const void *b, float *out, const float *residual, int m,
                             int n, int k);
/* 1 when the [n,k] matrix can take the prepared MFMA path: k % 256 == 0, a 16-byte aligned pointer, and rows
 * that are a multiple of 16 bytes (Q6_K: the whole matrix is, e.g. n % 8 == 0). */
int vx_matmul_quant_has_fast_path(int fmt, const void *b, int n, int k);
/* Which kernel family the backend's last quantized matmul launch took ("qmatvec_kernel", "qstream_kernel",
 * "qtiles_kernel", "qgemm_wave_kernel", "qgemm_rows_kernel", "qgemm_kernel", "qrow4_kernel",
 * "qgemm_fallback_kernel"; "" before the first). No counterpart in the reference; for tests and reports that must
 * know that the path they measure is the one a default configuration runs. */
const char *vx_last_matmul_kernel(vx_backend *be);

/* Fused decode blocks (the reference's FusedOps idea, backend.go:128-158, re-cut for the batched
 * paged path). They compute what the unfused call sequence computes, with each projection group
 * (Q|K|V, gate|up) as one launch and the split-K partial sums consumed directly by the next stage
 * instead of being reduced, stored and re-read. Results are deterministic and independent of the
 * batch a row sits in; against the unfused sequence they differ only by the float32 summation order
 * of the split-K slices (a group is sliced by its summed width). *_supported() is 1 when the weights allow it (same format within a group,
 * MFMA path available, rows of 16, widths that are multiples of 256 and fit one workgroup's LDS);
 * otherwise the entry points return VX_ERR_UNSUPPORTED before doing anything. */
typedef struct vx_qweight {
    int fmt;          /* VX_Q4_0 ... */
    const void *data; /* raw GGUF blocks on the device, [n,k] */
    int n, k;
} vx_qweight;

/* Load-time repack for decode batches. No counterpart in the reference, whose loader hands GGUF rows to the kernels
 * as they are (runtime/loader.go:79-200): vx_qweight_pack makes a second copy of a Q4_0, Q8_0, Q4_K, Q6_K, Q5_0 or Q5_K matrix
 * (n % 16 == 0, k % 256 == 0; VX_ERR_UNSUPPORTED otherwise, nothing changed) in the order the matrix cores consume it
 * (Q4_0 and Q8_0: a permutation of the rows' bytes, 18 / 34 per 32 elements either way; Q4_K: the codes with the
 * sub-blocks' scale and min products d * sc, dmin * m as float32, 6 bits per weight; Q6_K: one byte per code and the
 * float32 products d * sc per 16 elements, 10 bits per weight; Q5_0: one byte per code in the Q8_0 form, 8.5 bits;
 * Q5_K: one byte per code and the products as for Q4_K, 10 bits), kept by the backend under the matrix' address until
 * vx_qweight_unpack, vx_free of the matrix, a library write into its bytes or vx_backend_destroy. While it exists,
 * every quantized matmul entry point and fused decode block that is given the matrix (by the same data pointer, alone
 * or as part of a Q|K|V or gate|up group) with 2 .. 64 activation rows (Q4_K, Q5_K: 2 .. 32) streams the packed copy, and with more than 64 rows reads
 * it tile by tile; other row counts read the GGUF rows, which stay where they are. vx_dequantize_packed: gguf.Dequantize of the packed copy
 * (pkg/gguf/dequant.go:16-145, 272-470), bit for bit what vx_dequantize gives for the rows. */
int vx_qweight_pack(vx_backend *be, const vx_qweight *w);
int vx_qweight_unpack(vx_backend *be, const vx_qweight *w);
int vx_qweight_is_packed(vx_backend *be, const vx_qweight *w);
int vx_dequantize_packed(vx_backend *be, const vx_qweight *w, float *dst);

/* RMSNorm(x, norm_weight) -> Q|K|V projections (one launch) -> RoPE at positions[r] -> rotated Q to
 * q_out [rows,Hq*D], rotated K and V scattered into the pool at slot_mapping[r]
 * (runtime/block.go:834-868). With x_prepared != 0 the normalised activation left prepared by the
 * previous vx_decode_ffn (next_norm_weight) is used and x / norm_weight are ignored. wq and wk share a format;
 * wv may have another one (the K-quant mixes keep attn_v in Q6_K): with packed copies of Q4_K or Q5_K beside Q6_K and at
 * most 32 rows one launch still computes the three (its row groups shared out between the two formats), otherwise V is
 * a launch of its own between the shared prepare and the shared RoPE + store. */
int vx_decode_attn_qkv_supported(const vx_qweight *wq, const vx_qweight *wk, const vx_qweight *wv, int head_dim);
/* Optional, once per decode step before the layers' vx_decode_attn_qkv calls: works out cos / sin of every (row,
 * dimension pair) for positions[0 .. rows-1] (up to 64 rows, heads up to 256) and keeps them in the backend. While the
 * table stands, a vx_decode_attn_qkv call with the same positions pointer, at most 32 rows, an unbiased interleaved
 * whole-head RoPE and weights laid out for a single K slice rotates and stores its rows inside the projection launch
 * (one launch per layer less), with the same arithmetic; a call whose projection leaves K slices' sums (more rows, the
 * formats with a min term, V in another format) reads its cos / sin from the table in the RoPE + store launch that
 * follows. The table falls when the library writes to a caller's
 * buffer (vx_pack_batch, vx_decode_advance, vx_to_device, vx_copy_buffer); a caller that changes the positions by
 * other means must call this again (or not at all: without a table nothing changes). No counterpart in the reference,
 * which recomputes the angles in every layer (backend/cpu/cpu.go:226-303). */
int vx_rope_table_prepare(vx_backend *be, const int32_t *positions, int rows, int head_dim, float theta);
int vx_decode_attn_qkv(vx_backend *be, const float *x, const float *norm_weight, float eps, int x_prepared,
                       const vx_qweight *wq, const vx_qweight *wk, const vx_qweight *wv, int rows,
                       const int32_t *positions, const int32_t *slot_mapping, void *kv_pool, int pool_is_f16,
                       int num_q_heads, int num_kv_heads, int head_dim, int block_size, float theta, float *q_out);
/* The same for projections with biases (added before the rotation, as block.go:555-560 then :497-503 do) and with
 * Backend.RoPE's ropeDim / ropeNeox: Qwen 2's layer (Q/K/V biases, split pairs) on the fused path. NULL biases,
 * rope_dim 0 and rope_neox 0 are vx_decode_attn_qkv. */
int vx_decode_attn_qkv_ex(vx_backend *be, const float *x, const float *norm_weight, float eps, int x_prepared,
                          const vx_qweight *wq, const vx_qweight *wk, const vx_qweight *wv, const float *q_bias,
                          const float *k_bias, const float *v_bias, int rows, const int32_t *positions,
                          const int32_t *slot_mapping, void *kv_pool, int pool_is_f16, int num_q_heads, int num_kv_heads,
                          int head_dim, int block_size, float theta, int rope_dim, int rope_neox, float *q_out);
/* vx_decode_attn_qkv_ex for the first chunk of a prompt (runtime/block.go:834-868 at startPos 0): the same block, and
 * the rotated K rows and the V rows also as dense floats, k_out / v_out [rows, Hkv*D] (not yet rounded to the pool's
 * type), which the causal attention of that chunk reads (SDPAPrefill, block.go:893-895). k_out = v_out = NULL: exactly
 * vx_decode_attn_qkv_ex. */
int vx_prefill_attn_qkv(vx_backend *be, const float *x, const float *norm_weight, float eps, int x_prepared,
                        const vx_qweight *wq, const vx_qweight *wk, const vx_qweight *wv, const float *q_bias,
                        const float *k_bias, const float *v_bias, int rows, const int32_t *positions,
                        const int32_t *slot_mapping, void *kv_pool, int pool_is_f16, int num_q_heads, int num_kv_heads,
                        int head_dim, int block_size, float theta, int rope_dim, int rope_neox, float *q_out, float *k_out,
                        float *v_out);

/* x += attn*Wo^T; h = RMSNorm(x, ffn_norm_weight); x += (SiLU(h*W1^T) * (h*W3^T)) * W2^T
 * (runtime/block.go:981-1077), x [rows,hidden] updated in place. attn may be NULL when the call follows a
 * vx_sdpa_paged_decode_ragged with out = NULL for the same rows: the split-KV partials are merged here. When next_norm_weight != NULL,
 * RMSNorm(x, next_norm_weight) of the updated x is left prepared for the next vx_decode_attn_qkv
 * (x_prepared = 1) or vx_matmul_quant_prepared (the output head). */
int vx_decode_ffn_supported(const vx_qweight *wo, const vx_qweight *w1, const vx_qweight *w3, const vx_qweight *w2);
int vx_decode_ffn(vx_backend *be, const float *attn, float *x, const vx_qweight *wo, const float *ffn_norm_weight,
                  float eps, const vx_qweight *w1, const vx_qweight *w3, const vx_qweight *w2, int rows,
                  const float *next_norm_weight);

/* RoPE with one position per row (row r rotated as Backend.RoPE with seqLen=1,
 * startPos=positions[r]) fused with the paged scatter of K and V:
 * slot_mapping[r] = physBlock*blockSize + offset (runtime/gpu_block_pool.go:250-252).
 * q [rows,Hq,D] is rotated in place; k is rotated and stored; v is stored. */
int vx_rope_store_paged(vx_backend *be, float *q, const float *k, const float *v, const int32_t *positions,
                        const int32_t *slot_mapping, void *kv_pool, int pool_is_f16, int rows,
                        int num_q_heads, int num_kv_heads, int head_dim, int block_size, float theta);
/* The same with Backend.RoPE's ropeDim / ropeNeox (backend.go:352): the first rope_dim dimensions of a head turn
 * (0 = all), in pairs (j, j + rope_dim/2) when rope_neox; the others are stored as they are. */
int vx_rope_store_paged_ex(vx_backend *be, float *q, const float *k, const float *v, const int32_t *positions,
                           const int32_t *slot_mapping, void *kv_pool, int pool_is_f16, int rows, int num_q_heads,
                           int num_kv_heads, int head_dim, int block_size, float theta, int rope_dim, int rope_neox);

/* Ragged batched paged attention with all metadata on the device: block_tables is a
 * padded int32 [rows, max_blocks] matrix; sequence i uses row table_rows[i] (row i when
 * table_rows is NULL); kv_lens int32[batch]. One query per sequence. max_kv_len bounds
 * the launch (>= every kv_lens[i]; the lengths live on the device, so the host cannot check the promise: the
 * streaming kernels attend a longer sequence over its first max_kv_len tokens, rounded up to whole splits, and stay
 * inside their buffers; max_blocks * block_size is always a safe value). With out = NULL the result stays in the backend as per-split partial
 * sums for the next vx_decode_ffn(attn = NULL) to merge (one launch less); that form exists only where
 * vx_sdpa_paged_decode_split_supported() is 1, otherwise the call returns VX_ERR_UNSUPPORTED. Where a workgroup's
 * columns (query heads per KV head x head_dim) divide 256 or are a multiple of it, 2 to 64 rows, the workgroup that
 * finishes a sequence's 256 columns last also merges them, splits in index order, and writes them as the output
 * projection's prepared operand (no merge launch at all); any call between the two that prepares another
 * activation makes vx_decode_ffn merge from the partial sums as before. A call with out = NULL therefore replaces
 * whatever activation the backend held prepared (vx_prepare_act, vx_rmsnorm_prepare, ...): prepare again before a
 * vx_matmul_quant_prepared that is not the vx_decode_ffn this call is for.
 * That is also where the streaming split-KV kernel runs (F16 pool, 16-token blocks): heads of 64 or 128 with 1 to 8
 * query heads per KV head, heads of 256 with 1 or 2, heads of 80 or 96 with 1; other geometries take the generic
 * kernel (any head_dim <= 256), same results, far slower. */
int vx_sdpa_paged_decode_split_supported(int pool_is_f16, int block_size, int num_q_heads, int num_kv_heads,
                                         int head_dim);
int vx_sdpa_paged_decode_ragged(vx_backend *be, const float *q, const void *kv_pool, int pool_is_f16,
                                const int32_t *block_tables, const int32_t *table_rows, const int32_t *kv_lens,
                                float *out, int batch, int max_blocks, int block_size, int num_q_heads,
                                int num_kv_heads, int head_dim, float scale, int max_kv_len);
/* vx_sdpa_paged_decode_ragged for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc): the same kernels, same arguments and bit-identical results, with
 * the per-split partial sums in a fixed 8 MiB area that every device holds from the moment the library is loaded
 * until the process ends, instead of the backend's growable scratch. It has no counterpart in the reference. The
 * call allocates and frees nothing. It needs out != NULL and a geometry of the streaming kernel
 * (vx_sdpa_paged_decode_split_supported() == 1), else VX_ERR_UNSUPPORTED; batch * num_q_heads * splits *
 * (head_dim + 2) * 4 bytes must fit the area, else VX_ERR_INVALID with the sizes in vx_last_error(). splits =
 * ceil(max_kv_len / t), where t, the tokens one workgroup takes, is what the allocating entry point uses for the
 * same call (so that the results are the same bits): 512; 256 with two or more query heads per KV head at heads
 * of 64 or 128; and halved again, down to 128, while batch * num_kv_heads * splits would be under twice the
 * device's compute units. Examples: 32 sequences x 32 heads of 128 up to 4096 tokens take 4.3 MB; 32 sequences
 * x 32 / 8 heads of 128 up to 4096 tokens take 8.5 MB and are refused. vx_sdpa_paged_decode_ragged_noalloc_bytes
 * gives the exact need of a call (0 for a geometry the entry point does not take) and, through *capacity when
 * that is not NULL, the size of the area. All calls on one device, from any backend, share the area: two of
 * them in flight at once race. */
int vx_sdpa_paged_decode_ragged_noalloc(vx_backend *be, const float *q, const void *kv_pool, int pool_is_f16,
                                        const int32_t *block_tables, const int32_t *table_rows, const int32_t *kv_lens,
                                        float *out, int batch, int max_blocks, int block_size, int num_q_heads,
                                        int num_kv_heads, int head_dim, float scale, int max_kv_len);

size_t vx_sdpa_paged_decode_ragged_noalloc_bytes(vx_backend *be, int batch, int num_q_heads, int num_kv_heads, int head_dim,
                                                 int max_kv_len, size_t *capacity);

/* Tree verification (medusa/tree.go:186-202 mask rule): query i attends to every pool
 * position < tree_base and to position tree_base+j iff tree_mask[i*query_len+j] != 0
 * (uint8 on device). */
int vx_sdpa_paged_tree(vx_backend *be, const float *q, const void *kv_pool, int pool_is_f16,
                       const int32_t *block_table, float *out, const uint8_t *tree_mask, int tree_base,
                       int block_size, int num_q_heads, int num_kv_heads, int head_dim, float scale,
                       int query_len);

/* Tree verification for many sequences in two launches. The query rows come in entries of
 * vx_sdpa_paged_tree_rows_per_entry() consecutive rows (16 / G for G query heads per KV head; 0: this geometry
 * has no batched form) or, where that number is even, of half as many (rows / entries says which: fewer rows of
 * padding for small trees, the context read twice as often); the rows of an entry belong to one tree, whose sequence is block-table row entry_table_rows[e] with entry_kv_lens[e] tokens
 * before the tree. A tree's own keys sit at pool positions kv_len .. kv_len + n - 1 of its sequence (stored
 * before the call). row_info: int32[rows][4] = (block-table row, kv_len, row index inside its tree, rows n of the
 * tree); row i of a tree sees key j where tree_masks[mask_offsets[row] + i*n + j] != 0 (medusa/tree.go:186-202).
 * Rows that only pad an entry repeat a real row. F16 pool with 16-token blocks; all arrays on the device. The
 * context is read once per entry (not once per row); no counterpart in the reference, which verifies one path. */
int vx_sdpa_paged_tree_rows_per_entry(int pool_is_f16, int block_size, int num_q_heads, int num_kv_heads, int head_dim);
int vx_sdpa_paged_tree_batched(vx_backend *be, const float *q, const void *kv_pool, const int32_t *block_tables,
                               int max_blocks, const int32_t *entry_table_rows, const int32_t *entry_kv_lens,
                               int entries, const int32_t *row_info, const uint8_t *tree_masks,
                               const int32_t *mask_offsets, float *out, int rows, int max_tree_rows,
                               int num_q_heads, int num_kv_heads, int head_dim, float scale, int max_kv_len);

/* Copies num_tokens token rows (K and V of every KV head) from src_slots[i] to dst_slots[i] of one layer's paged
 * pool (device int32 arrays, slot = physical block * block_size + offset; the two sets must not overlap) and
 * rotates the K rows by the angle of position `shift` on the way: RoPEShift (backend/cpu/backend.go:244-276,
 * interleaved pairs) applied where the reference applies it to a gathered copy when it reads a cached fragment
 * (kv/paged_cache.go:225-283). An F16 pool keeps the rotated K rounded to half precision. shift 0 is a plain copy. */
int vx_paged_kv_copy_shifted(vx_backend *be, void *kv_pool, int pool_is_f16, const int32_t *src_slots,
                             const int32_t *dst_slots, int num_tokens, int num_kv_heads, int head_dim, int block_size,
                             int shift, float theta);

/* Moves token rows (K and V of every KV head) inside one layer's paged pool: slot = physical block *
 * block_size + offset in the block. Chain c is the moves chain_offsets[c] .. chain_offsets[c+1]-1 (device
 * int32 arrays), applied in order, so a later move of a chain may read what an earlier one wrote; different
 * chains must not touch the same slots. No counterpart in the reference, whose verification keeps one path
 * that is contiguous already (scheduler/medusa_scheduler.go:852-861 only truncates); after a whole tree has
 * been verified the accepted path's rows have to move up before the truncation. */
int vx_paged_kv_move(vx_backend *be, void *kv_pool, int pool_is_f16, const int32_t *chain_offsets,
                     const int32_t *src_slots, const int32_t *dst_slots, int num_chains, int num_kv_heads,
                     int head_dim, int block_size);

/* Row-wise argmax on the device: out_idx[r] = ArgmaxOps.Argmax(logits + r*n, n). No wait. */
int vx_argmax_rows(vx_backend *be, const float *logits, int rows, int n, int32_t *out_idx);

/* Sampler.Sample (pkg/sampler/sampler.go:48-204) for every row of logits[rows, n] on the device: temperature
 * scaling, softmax, top-k (0 or >= n: off), top-p (<= 0 or >= 1: off) and the draw, with the row's uniform number
 * in [0, 1) given by the caller in place of the reference's rand.Float32(). temperature 0 is Argmax. All sums are
 * float32 in the reference's order, so the token is the reference's for the same draw; among equal probabilities
 * at the nucleus boundary the lower index stays (the reference's sort leaves that open). All arrays on the device;
 * out_idx int32[rows]. No wait. */
int vx_sample_rows(vx_backend *be, const float *logits, int rows, int n, const float *temperature,
                   const int32_t *top_k, const float *top_p, const float *uniform, int32_t *out_idx);

/* Continuous-batching step metadata built on the device by prefix scans
 * (host restatement: scheduler/scheduler.go:290-303 + runtime/gpu_block_pool.go:234-252,
 * 359-363). Inputs (device int32): seq_slots[batch] = row of each sequence in the
 * block-table matrix, positions[batch] = first new position, q_lens[batch] = new tokens
 * (NULL = 1 each). free_list[free_cap] / free_count[1] are the pool's free stack; blocks
 * are popped from the tail in batch order exactly as the per-sequence StoreKV calls would.
 * Outputs (device int32): cu_seqlens[batch+1], token_pos[T], slot_mapping[T], kv_lens[batch],
 * block tables updated in place, status[1] = 0 or 1 if the pool ran out of blocks.
 * total_tokens = sum(q_lens) is given by the caller (T).
 * The call also leaves, inside the backend, a work list for vx_sdpa_paged_decode_ragged: one item per 512 tokens
 * of every sequence, equal items first, the partial last items from the longest down. An attention call that
 * passes this kv_lens array, seq_slots as its table_rows and the same batch walks the list (no empty workgroups inside its grid, the smallest last);
 * the list is dropped when the array is written through vx_to_device / vx_copy_buffer, freed, or the pool is
 * reset. A caller that rewrites kv_lens with kernels of its own must do so in another array. */
int vx_pack_batch(vx_backend *be, const int32_t *seq_slots, const int32_t *positions, const int32_t *q_lens,
                  int batch, int total_tokens, int32_t *block_tables, int max_blocks, int32_t *num_blocks,
                  int32_t *free_list, int32_t *free_count, int block_size, int32_t *cu_seqlens,
                  int32_t *token_pos, int32_t *slot_mapping, int32_t *kv_lens, int32_t *status);

/* End of a device-driven decode step (host restatement: scheduler/scheduler.go:432-446 greedy arm +
 * scheduler/sequence.go:136-141): out_log[step*batch + i] = next_tokens[i] where step = *step_counter,
 * then tokens[i] = next_tokens[i], positions[i] += 1, *step_counter += 1. All device int32. */
int vx_decode_advance(vx_backend *be, int32_t *tokens, int32_t *positions, const int32_t *next_tokens,
                      int32_t *out_log, int32_t *step_counter, int batch);

/* Stream capture of a decode step into a hipGraph (replaces the Metal command-buffer
 * batching of runtime/decode.go:426-431). Between begin and end every vx_* compute call
 * is recorded instead of run; vx_graph_launch replays the recording. */
typedef struct vx_graph vx_graph;
int vx_graph_begin_capture(vx_backend *be);
int vx_graph_end_capture(vx_backend *be, vx_graph **out);
int vx_graph_launch(vx_backend *be, vx_graph *g);
/* A recording holds the addresses of the library's own scratch buffers (prepared activations, split-K and
 * split-KV partial sums, the attention work list) and of the packed copies of quantized matrices. The buffers move
 * when a later eager call needs more room than any call before it, the copies come and go with vx_qweight_pack /
 * vx_qweight_unpack / vx_free; the counter returned here goes up by one each time either happens. A caller that keeps a graph
 * records the counter after vx_graph_end_capture and captures again, instead of launching, once it has changed.
 * No counterpart in the reference (its command buffers are rebuilt every step). */
uint64_t vx_scratch_generation(const vx_backend *be);
/* The caller makes sure no replay of the graph is still running (vx_sync). */
void vx_graph_destroy(vx_graph *g);

/* Wall-clock helpers on the backend stream (HIP events), for benchmarks. */
int vx_timer_start(vx_backend *be);
int vx_timer_stop_ms(vx_backend *be, float *ms);

#ifdef __cplusplus
}
#endif
#endif /* VEXEL_HIP_H */
