/*
 * vexel_host.h -- C API of libvexel_host.so: the host-side drivers of the batched-decode
 * path (block pool bookkeeping, layer executor, decode / prefill drivers), written in C++
 * above the C ABI of vexel_hip.h. In a Go build these are the Go packages themselves
 * (inference/runtime); this library exists so the same logic can be built, tested and
 * benchmarked where no Go toolchain is present. Each function names the Go method it mirrors.
 */
#ifndef VEXEL_HOST_H
#define VEXEL_HOST_H

#include <stdint.h>

#include "vexel_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

enum { VH_OK = 0, VH_ERR = 1 };

/* runtime.ModelConfig (inference/runtime/config.go) fields the path needs + pool sizing */
typedef struct vh_config {
    int num_layers, hidden, num_heads, num_kv_heads, head_dim, ffn, vocab;
    float eps, rope_theta;
    int block_size;          /* 16 in the reference (runtime/model.go:321) */
    int pool_blocks;         /* physical blocks per layer (GPUBlockPool.maxBlocks) */
    int max_seqs;            /* rows of the device block-table matrix */
    int max_blocks_per_seq;  /* columns of the device block-table matrix */
    int max_batch;           /* rows of the activation buffers */
    int kv_fp16;             /* 1 = F16 pool (runtime/model.go:311), 0 = F32 */
} vh_config;

typedef vx_qweight vh_qweight;  /* tensor.Tensor with a QuantProfile: raw GGUF blocks on the device */
/* vh_qweight.fmt for a plain float32 [n,k] matrix (a dequantized or tied output head, runtime/loader.go:187-203,
 * 596-600); accepted for the output head only. */
enum { VH_F32 = 0 };

typedef struct vh_layer_weights {  /* the BlockRuntime fields used by ExecuteWithPagedKV */
    const float *attn_norm, *ffn_norm;
    vh_qweight wq, wk, wv, wo, w1, w2, w3;
} vh_layer_weights;

/* The architecture switches of runtime/config.go:14-62,120-131 and block.go:245-254,339-340. All zero = LLaMA. */
enum { VH_NORM_RMS = 0, VH_NORM_LAYER = 1 };                  /* NormType */
enum { VH_MLP_SWIGLU = 0, VH_MLP_GELU = 1, VH_MLP_GEGLU = 2 }; /* MLPType */
typedef struct vh_arch {
    int norm_type, mlp_type;
    int parallel_residual;   /* x + attn(norm(x)) + mlp(norm(x)); with the GELU MLP only (block.go:972-976) */
    int rope_dim;            /* rotated dimensions of a head, 0 = all (RoPEDim) */
    int rope_neox;           /* pairs (j, j + rope_dim/2) instead of (2j, 2j+1) */
    int post_norms;          /* HasPostNorms: RMSNorm of the attention and MLP outputs before the residual */
    float attn_softcap;      /* AttentionLogitSoftCap: applied where block.go applies it on the paged path, the
                                first prefill chunk (block.go:891-892) */
    float embedding_scale;   /* EmbeddingScale, <= 0 = none (decode.go:197-205) */
    float final_softcap;     /* FinalLogitSoftCap (model.go:336-350): applied, as in the reference, to the logits a
                                request is sampled from (scheduler.go:772-773), not to what vh_prefill and
                                vh_decode_batched return, and not before a greedy arg-max */
} vh_arch;
typedef struct vh_layer_extras {  /* the BlockRuntime tensors beside vh_layer_weights (block.go:266-283); NULL = absent */
    const float *attn_norm_bias, *ffn_norm_bias;
    const float *wq_bias, *wk_bias, *wv_bias, *wo_bias, *w1_bias, *w2_bias;
    const float *post_attn_norm, *post_ffn_norm;
} vh_layer_extras;

typedef struct vh_model vh_model;

const char *vh_last_error(void);

/* NewModelRuntime + CreateGPUBlockPool (runtime/model.go:305-327): allocates the per-layer
 * KV pool, the device mirror of the block tables and the activation buffers. */
int vh_model_create(vx_backend *be, const vh_config *cfg, vh_model **out);
void vh_model_destroy(vh_model *m);
void vh_model_get_config(const vh_model *m, vh_config *out);  /* the configuration the model was created with */
/* Decode uses vx_decode_attn_qkv / vx_decode_ffn wherever they support the weights (default on).
 * Off = the one-call-per-operation sequence of runtime/block.go; the two agree to float32
 * summation order. */
void vh_model_set_fused(vh_model *m, int on);
int vh_model_set_layer(vh_model *m, int layer, const vh_layer_weights *w);
/* A model with any switch or extra tensor set runs ExecuteWithPagedKV's general sequence, one backend call per
 * operation (block.go:834-1077), in vh_prefill, vh_decode_batched, vh_decode_graph, vh_verify_tree and the scheduler,
 * except where a half of the layer is LLaMA's up to Q/K/V biases and the RoPE form: an RMSNorm in front of Q|K|V
 * without a bias lets the fused attention block serve the first half, and a second half without post-norms, biases,
 * GELU / GeGLU or a parallel residual takes the fused FFN block. With the GELU MLP a layer's w3 may be empty.
 * All pointers are float32 device vectors that outlive the model's use of them. */
int vh_model_set_architecture(vh_model *m, const vh_arch *arch);
void vh_model_get_architecture(const vh_model *m, vh_arch *out);
int vh_model_set_layer_extras(vh_model *m, int layer, const vh_layer_extras *extras);
int vh_model_set_final_norm_bias(vh_model *m, const float *bias);  /* Model.FinalNormBias (model.go:36, 207-219) */
/* embedding: F32 [vocab,hidden] on the device (loader rule, runtime/loader.go:275-288) */
int vh_model_set_head(vh_model *m, const float *embedding, const float *final_norm, const vh_qweight *lm_head);
void *vh_kv_pool(vh_model *m, int layer);  /* device base of a layer's block pool */
/* Device arrays the last decode step ran on: the block-table matrix [slots, max_blocks_per_seq], the matrix
 * row of every batch entry and the kv lengths (int32 each). For measuring or re-running the step's attention
 * call in isolation; contents change with every step. */
void vh_step_buffers(vh_model *m, const int32_t **block_tables, const int32_t **table_rows, const int32_t **kv_lens);

/* GPUBlockPool (runtime/gpu_block_pool.go) */
int vh_pool_create_sequence(vh_model *m, int64_t seq_id);                       /* :126 */
int vh_pool_delete_sequence(vh_model *m, int64_t seq_id);                       /* :138 */
int vh_pool_truncate_sequence(vh_model *m, int64_t seq_id, int new_len);        /* :162 */
int vh_pool_has_sequence(vh_model *m, int64_t seq_id);                          /* :193 */
int vh_pool_share_blocks(vh_model *m, int64_t src, int64_t dst, int num_tokens);/* :572 */
void vh_pool_block_stats(vh_model *m, int *total, int *free_blocks, int *shared);/* :610 (per layer x numLayers) */
/* Named fragments (kv/fragment.go:18-101, kv/paged_cache.go:285-343): the K/V of a finished sequence kept under a
 * name and put at the end of other sequences without running the model over those tokens again.
 *   vh_fragment_cache   PagedKVCache.CacheContent: the sequence's blocks get one more reference each and stay alive
 *                       after the sequence is deleted; a fragment of the same name is released first; an unknown
 *                       sequence caches nothing.
 *   vh_fragment_insert  PagedKVCache.InsertFragment: *num_tokens = tokens added (0 and VH_OK for an unknown name;
 *                       an unknown sequence is created). insert_pos must be the sequence's length. The reference
 *                       shares the blocks and rotates K by insert_pos at every read; here the rows are copied once
 *                       into the sequence's own blocks with K rotated (vx_paged_kv_copy_shifted), so attention reads
 *                       the pool as it is.
 *   vh_fragment_delete  FragmentCache.Delete; vh_fragment_tokens: CachedFragment.NumTokens or -1;
 *   vh_fragment_count   len(FragmentCache.List()). */
int vh_fragment_cache(vh_model *m, const char *name, int64_t seq_id);
int vh_fragment_insert(vh_model *m, int64_t seq_id, const char *name, int insert_pos, int *num_tokens);
int vh_fragment_delete(vh_model *m, const char *name);
int vh_fragment_tokens(vh_model *m, const char *name);
int vh_fragment_count(vh_model *m);
int vh_pool_seq_len(vh_model *m, int64_t seq_id);
/* copies the sequence's block table (identical for every layer) into out; returns its length or -1 */
int vh_pool_block_table(vh_model *m, int64_t seq_id, int32_t *out, int cap);
/* installs a given block table / length for a sequence whose KV was written directly into the
 * pool (synthetic pre-filled contexts of the benchmark configs); the blocks leave the free list */
int vh_pool_adopt_blocks(vh_model *m, int64_t seq_id, const int32_t *blocks, int num_blocks, int seq_len);
/* reads the device mirror back and compares it with the host state: 1 equal, 0 different, <0 error */
int vh_pool_device_matches_host(vh_model *m);

/* ModelRuntime.DecodeWithPagedKVBatched (runtime/decode.go:612-654): one token per sequence.
 * logits_out: host [batch,vocab] or NULL; argmax_out: host [batch] or NULL. */
int vh_decode_batched(vh_model *m, const int32_t *tokens, const int64_t *seq_ids, const int32_t *positions,
                      int batch, float *logits_out, int32_t *argmax_out);
/* Sampler.Sample (pkg/sampler/sampler.go:48-77) on the device for the `rows` rows of logits the last
 * vh_decode_batched left there, one (temperature, top_k, top_p, uniform draw in [0, 1)) per row from host arrays;
 * temperature 0 is the greedy choice. tokens_out: host int32[rows]. */
int vh_sample_last_logits(vh_model *m, int rows, const float *temperature, const int32_t *top_k, const float *top_p,
                          const float *uniform, int32_t *tokens_out);
/* Speculative verification of a whole candidate tree for each of n_seqs sequences in one forward pass, greedy
 * acceptance and rollback. The reference's runTreeMedusaDecodeStep (scheduler/medusa_scheduler.go:733-861)
 * handles one sequence and verifies only the most confident path with VerifySpeculativeWithPagedKV
 * (runtime/decode.go:1446-1569); here every path is verified at once under the ancestor mask of
 * medusa/tree.go:186-202, and each root-to-node path sees exactly what that linear verification shows it.
 *   Sequence i: input_tokens[i] goes to position start_pos[i], which must be the sequence's KV length; its
 *   n_nodes[i] candidates follow in CandidateTree.Linearize order (tree.go:144-178), tokens and parent indices
 *   (-1 = child of the input token) concatenated over the sequences in node_tokens / parent_idx.
 *   Acceptance: from the argmax of the input token's logits, descend into the child whose token equals the
 *   current argmax (first such child), continue with that node's argmax; the argmax nobody matches is the
 *   final token. accepted_nodes receives the accepted node indices (within the sequence's tree, path order)
 *   at the sequence's offset in the concatenated node arrays; num_accepted[i] and final_tokens[i] per sequence.
 *   Rollback (medusa_scheduler.go:852-861): the accepted nodes' K/V rows move to the positions after the input
 *   token and the sequence is truncated to start_pos + 1 + accepted (gpu_block_pool.go:162-190).
 * logits_out: host [n_seqs + sum n_nodes, vocab] (per sequence: input token row, then node rows) or NULL. */
int vh_verify_tree(vh_model *m, int n_seqs, const int64_t *seq_ids, const int32_t *input_tokens,
                   const int32_t *start_pos, const int32_t *n_nodes, const int32_t *node_tokens,
                   const int32_t *parent_idx, int32_t *num_accepted, int32_t *accepted_nodes, int32_t *final_tokens,
                   float *logits_out);
/* ModelRuntime.PrefillWithPagedKV (runtime/decode.go:961-1096) when all_logits == 0: logits of the
 * last token -> logits_out[vocab]. VerifySpeculativeWithPagedKV (decode.go:1446-1569) when
 * all_logits != 0: logits of every position -> logits_out[n,vocab]. */
int vh_prefill(vh_model *m, const int32_t *tokens, int n, int64_t seq_id, int start_pos, int all_logits,
               float *logits_out);
/* Greedy decode of `steps` tokens for a fixed batch with the step captured in a hipGraph and all
 * per-step metadata built on the device. out_tokens: host [steps,batch]. The host pool state is
 * advanced by the same rule afterwards. use_graph = 0 runs the same device-driven step eagerly. */
int vh_decode_graph(vh_model *m, const int32_t *first_tokens, const int64_t *seq_ids, const int32_t *positions,
                    int batch, int steps, int use_graph, int32_t *out_tokens, float *ms_per_step);

/* ---- GGUF checkpoints (inference/pkg/gguf/gguf.go; loader rule of inference/runtime/loader.go) ---------- */
#define VH_GGUF_MAX_DIMS 4
typedef struct vh_gguf vh_gguf;
typedef struct vh_gguf_tensor {  /* gguf.TensorInfo (gguf.go:200-207) plus where its bytes are */
    const char *name;            /* owned by the reader */
    int n_dims;
    uint64_t dims[VH_GGUF_MAX_DIMS]; /* file order: dims[0] is the innermost dimension (K of an [N,K] matrix) */
    uint32_t type;               /* gguf.TensorType (gguf.go:38-60) */
    uint64_t offset;             /* from the start of the data section */
    uint64_t n_bytes;            /* ceil(elements / block) * bytes per block (gguf.go:594-604) */
    const void *data;            /* host address inside the file mapping; NULL when the file ends before it */
} vh_gguf_tensor;
typedef struct vh_gguf_config {  /* File.extractModelConfig (gguf.go:504-582); 0 = key absent */
    char architecture[64];
    int num_layers, hidden, num_heads, num_kv_heads, ffn, context_length, vocab, rope_dim_count, head_dim;
    float rope_theta;            /* 10000 when absent */
    float rms_eps;
    float attn_softcap, final_softcap; /* <arch>.attn_logit_softcapping / final_logit_softcapping (gguf.go:560-566) */
} vh_gguf_config;
/* gguf.Open (gguf.go:249-335): magic, version 2..3, metadata, tensor table, aligned data offset. The file is
 * mapped read-only; nothing is copied until a tensor is used. */
int vh_gguf_open(const char *path, vh_gguf **out);
void vh_gguf_close(vh_gguf *g);
uint32_t vh_gguf_version(const vh_gguf *g);
int64_t vh_gguf_data_offset(const vh_gguf *g);
int vh_gguf_num_tensors(const vh_gguf *g);
int vh_gguf_tensor_at(const vh_gguf *g, int i, vh_gguf_tensor *out);
int vh_gguf_find_tensor(const vh_gguf *g, const char *name, vh_gguf_tensor *out);  /* File.GetTensor (gguf.go:584-591) */
int vh_gguf_num_metadata(const vh_gguf *g);
const char *vh_gguf_metadata_key(const vh_gguf *g, int i);                         /* file order */
int vh_gguf_meta_type(const vh_gguf *g, const char *key);                          /* gguf.MetadataType, -1 if absent */
uint32_t vh_gguf_meta_u32(const vh_gguf *g, const char *key);                      /* MetadataValue.AsUint32 (gguf.go:158-169) */
uint64_t vh_gguf_meta_u64(const vh_gguf *g, const char *key);                      /* AsUint64 (:172-181) */
float vh_gguf_meta_f32(const vh_gguf *g, const char *key);                         /* AsFloat32 (:189-198) */
const char *vh_gguf_meta_str(const vh_gguf *g, const char *key);                   /* NULL unless a string */
int64_t vh_gguf_meta_array_len(const vh_gguf *g, const char *key);                 /* -1 unless an array */
int vh_gguf_get_config(const vh_gguf *g, vh_gguf_config *out);
/* gguf.GetLayerTensorName (pkg/gguf/loader.go:121-228), LLaMA-family names; others pass through. */
int vh_gguf_tensor_name(const char *hf_name, char *out, size_t cap);

typedef struct vh_load_options {  /* what the checkpoint does not say: the KV pool and batch geometry */
    int block_size;               /* 0 = 16 */
    int pool_blocks, max_seqs, max_blocks_per_seq, max_batch, kv_fp16;
} vh_load_options;
/* ModelRuntime.LoadWeightsGGUF + CopyWeightsToDevice (runtime/loader.go:28-212, 560-700). general.architecture
 * selects the switches as ModelConfigFromGGUF does (runtime/config.go:388-470): llama / mistral; qwen2 (Q/K/V biases,
 * split-pair RoPE); gemma and gemma2 (GeGLU, embeddings times sqrt(hidden); gemma2 also post-norms and the soft
 * caps); phi / phi2 (LayerNorm and biases, GELU MLP, parallel residual, partial split-pair RoPE, the fused
 * attn_qkv matrix used in place as three row ranges, loader.go:610-640). Any other architecture is refused. For
 * all of them: Q4_0 / Q8_0 / Q4_K / Q6_K / Q5_0 / Q5_K / BF16 projection matrices and output head go to the
 * device as raw blocks, token_embd and the norm vectors as float32 (F32, F16 or one of those types in the file), a missing
 * output.weight is the embedding. One difference: a Q4_0 output head stays Q4_0 here, where the reference
 * dequantizes it to float32 at load (same values, float32 summation order aside). The model owns the device
 * copies; vh_model_destroy frees them. */
int vh_model_load_gguf(vx_backend *be, const char *path, const vh_load_options *opt, vh_model **out);
/* Hands a vx_alloc_permanent buffer to the model, which frees it in vh_model_destroy. */
void vh_model_adopt_buffer(vh_model *m, void *device_ptr);

/* ---- continuous-batching scheduler (inference/scheduler/scheduler.go, sequence.go; pkg/sampler/sampler.go) ---- */
enum { VH_SEQ_PENDING = 0, VH_SEQ_PREFILL = 1, VH_SEQ_DECODING = 2, VH_SEQ_FINISHED = 3 };  /* sequence.go:15-20 */
typedef struct vh_scheduler vh_scheduler;
typedef struct vh_sched_config {  /* scheduler.Config (scheduler.go:24-36) */
    int max_batch_size;           /* ready sequences per step */
    int max_tokens;               /* generation limit per sequence, 0 = none */
    int eos_token;                /* the stop token (scheduler.go:110-116) */
    int prefill_chunk;            /* 0 = a prompt is prefilled in one call (scheduler.go:483-500); > 0 = in pieces of
                                     this many tokens, one piece per step */
} vh_sched_config;
int vh_sched_create(vh_model *m, const vh_sched_config *cfg, vh_scheduler **out);
void vh_sched_destroy(vh_scheduler *s);
/* Scheduler.AddSequence (scheduler.go:645-677) with the prompt already tokenized; max_tokens 0 = the scheduler's. */
int vh_sched_add_sequence(vh_scheduler *s, int64_t seq_id, const int32_t *prompt, int n, int max_tokens);
/* Sequence.SetSamplingParams (sequence.go:150-160); temperature 0 = greedy. The uniform draws come from a
 * SplitMix64 stream started at seed. */
int vh_sched_set_sampling(vh_scheduler *s, int64_t seq_id, float temperature, int top_k, float top_p, uint64_t seed);
int vh_sched_remove_sequence(vh_scheduler *s, int64_t seq_id);             /* scheduler.go:679-699 */
int vh_sched_sequence_count(const vh_scheduler *s);                        /* scheduler.go:702-706 */
int vh_sched_state(const vh_scheduler *s, int64_t seq_id);                 /* VH_SEQ_*, -1 if unknown */
int vh_sched_position(const vh_scheduler *s, int64_t seq_id);
int vh_sched_generated(const vh_scheduler *s, int64_t seq_id, int32_t *out, int cap);
/* One Scheduler.step (scheduler.go:166-201): ready sequences in ascending id (the reference's map order is
 * unspecified), prompts fed first, then one batched decode; *tokens_out = tokens generated. */
int vh_sched_step(vh_scheduler *s, int *tokens_out);
/* sampler.Argmax (sampler.go:80-91) and Sampler.Sample (sampler.go:48-77) on host logits, the uniform draw r given. */
int vh_argmax(const float *logits, int n);
int vh_sample(const float *logits, int n, float temperature, int top_k, float top_p, float r);

#ifdef __cplusplus
}
#endif
#endif
