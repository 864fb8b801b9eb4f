"""HipBackend: Python mirror of vexel's Go backend interfaces over the C ABI.

Method names and argument order follow inference/backend/backend.go (Backend :309-390,
QuantizedMatMul :47-81, PagedKVOps :415-466, BufferCopier :38-43, ArgmaxOps :199-203,
PoolResetter :8-10) in snake_case. Device pointers are plain integers (device addresses),
as tensor.DevicePtr.Addr()+Offset() would be. A non-zero status raises VexelError, where
the Go shim would panic. Host data goes in and out as numpy arrays; nothing here computes.
"""
import ctypes as C

import numpy as np

from . import lib as _l


class VxQWeight(C.Structure):
    """vx_qweight of include/vexel_hip.h."""
    _fields_ = [("fmt", C.c_int), ("data", C.c_void_p), ("n", C.c_int), ("k", C.c_int)]


class VexelError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("vexel_hip error %d: %s" % (code, msg))
        self.code = code


class HipBackend:
    def __init__(self, device=0):
        self._lib = _l.load()
        h = C.c_void_p()
        rc = self._lib.vx_backend_create(device, C.byref(h))
        if rc != 0:
            raise VexelError(rc, self._lib.vx_last_error().decode())
        self._h = h

    def close(self):
        if self._h:
            self._lib.vx_backend_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _ck(self, rc):
        if rc != 0:
            raise VexelError(rc, self._lib.vx_last_error().decode())

    def lib_call(self, name, *args):
        """Calls a C-ABI function that takes no backend handle and returns its int result."""
        return getattr(self._lib, name)(*args)

    def call(self, name, *args):
        """Calls C-ABI function `name` with the backend handle prepended; raises on error."""
        self._ck(getattr(self._lib, name)(self._h, *args))

    def set_attn_merge(self, on):
        """vx_backend_set_attn_merge: the decode attention kernel merges its own splits (default) or not."""
        self.call("vx_backend_set_attn_merge", int(bool(on)))

    def last_matmul_kernel(self):
        """vx_last_matmul_kernel: the kernel family of the last quantized matmul launch."""
        return self._lib.vx_last_matmul_kernel(self._h).decode()

    def scratch_generation(self):
        """How often the library's own scratch buffers have moved (a kept graph is stale once this changes)."""
        return int(self._lib.vx_scratch_generation(self._h))

    # ---- memory
    def alloc(self, nbytes):
        p = self._lib.vx_alloc(self._h, nbytes)
        if not p and nbytes > 0:
            raise VexelError(_l.VX_ERR_OOM, self._lib.vx_last_error().decode())
        return p or 0

    def alloc_permanent(self, nbytes):
        p = self._lib.vx_alloc_permanent(self._h, nbytes)
        if not p and nbytes > 0:
            raise VexelError(_l.VX_ERR_OOM, self._lib.vx_last_error().decode())
        return p or 0

    def free(self, ptr):
        self._lib.vx_free(self._h, ptr)

    def reset_pool(self):
        self._lib.vx_reset_pool(self._h)

    def to_device(self, dst, src):
        src = np.ascontiguousarray(src)
        self.call("vx_to_device", dst, src.ctypes.data, src.nbytes)

    def to_host(self, dst, src):
        assert dst.flags["C_CONTIGUOUS"]
        self.call("vx_to_host", dst.ctypes.data, src, dst.nbytes)

    def sync(self):
        self.call("vx_sync")

    def copy_buffer(self, src, src_off, dst, dst_off, size):
        self.call("vx_copy_buffer", src, src_off, dst, dst_off, size)

    def begin_batch(self):
        self.call("vx_begin_batch")

    def end_batch(self):
        self.call("vx_end_batch")

    def memory_barrier(self):
        self.call("vx_memory_barrier")

    # helpers for tests / drivers (not part of the Go interface)
    def upload(self, arr, permanent=False):
        arr = np.ascontiguousarray(arr)
        p = (self.alloc_permanent if permanent else self.alloc)(max(arr.nbytes, 4))
        if arr.nbytes:
            self.to_device(p, arr)
        return p

    def download(self, ptr, shape, dtype):
        out = np.empty(shape, dtype=dtype)
        if out.nbytes:
            self.to_host(out, ptr)
        return out

    # ---- Backend compute
    def matmul(self, a, b, out, m, n, k):
        self.call("vx_matmul", a, b, out, m, n, k)

    def matmul_transposed(self, a, b, out, m, n, k):
        self.call("vx_matmul_transposed", a, b, out, m, n, k)

    def rmsnorm(self, x, weight, out, rows, cols, eps):
        self.call("vx_rmsnorm", x, weight, out, rows, cols, eps)

    def rope(self, q, k, head_dim, num_heads, num_kv_heads, seq_len, start_pos, rope_dim, theta, rope_neox):
        self.call("vx_rope", q, k, head_dim, num_heads, num_kv_heads, seq_len, start_pos, rope_dim, theta,
                  int(bool(rope_neox)))

    def silu(self, x, out, n):
        self.call("vx_silu", x, out, n)

    def silu_mul(self, gate, up, out, n):
        self.call("vx_silu_mul", gate, up, out, n)

    def softmax(self, x, out, rows, cols):
        self.call("vx_softmax", x, out, rows, cols)

    def add(self, a, b, out, n):
        self.call("vx_add", a, b, out, n)

    def mul(self, a, b, out, n):
        self.call("vx_mul", a, b, out, n)

    def embedding(self, ids, num_tokens, table, out, vocab_size, dim):
        self.call("vx_embedding", ids, num_tokens, table, out, vocab_size, dim)

    def sdpa(self, q, k, v, out, kv_len, num_q_heads, num_kv_heads, head_dim, scale, kv_head_stride):
        self.call("vx_sdpa", q, k, v, out, kv_len, num_q_heads, num_kv_heads, head_dim, scale, kv_head_stride)

    def sdpa_prefill(self, q, k, v, out, seq_len, num_q_heads, num_kv_heads, head_dim, scale):
        self.call("vx_sdpa_prefill", q, k, v, out, seq_len, num_q_heads, num_kv_heads, head_dim, scale)

    # ---- Medusa heads (medusa/heads.go)
    def medusa_forward(self, hidden, fc1, fc2, intermediate, logits, rows, num_heads, hidden_size, vocab_size):
        self.call("vx_medusa_forward", hidden, fc1, fc2, intermediate, logits, rows, num_heads, hidden_size, vocab_size)

    def topk_rows(self, x, rows, n, k, out_idx, out_val=None):
        self.call("vx_topk_rows", x, rows, n, k, out_idx, out_val)

    # ---- optional interfaces (backend.go:205-263)
    def layernorm(self, x, weight, bias, out, rows, cols, eps):
        self.call("vx_layernorm", x, weight, bias, out, rows, cols, eps)

    def gelu(self, x, out, n):
        self.call("vx_gelu", x, out, n)

    def gelu_mul(self, gate, up, out, n):
        self.call("vx_gelu_mul", gate, up, out, n)

    def add_bias(self, x, bias, out, rows, cols):
        self.call("vx_add_bias", x, bias, out, rows, cols)

    def logit_softcap(self, logits, n, cap):
        self.call("vx_logit_softcap", logits, n, cap)

    def scale_buffer(self, buf, scale, n):
        self.call("vx_scale_buffer", buf, scale, n)

    def sdpa_softcap(self, q, k, v, out, kv_len, num_q_heads, num_kv_heads, head_dim, scale, softcap, kv_head_stride):
        self.call("vx_sdpa_softcap", q, k, v, out, kv_len, num_q_heads, num_kv_heads, head_dim, scale, softcap,
                  kv_head_stride)

    def sdpa_prefill_softcap(self, q, k, v, out, seq_len, num_q_heads, num_kv_heads, head_dim, scale, softcap):
        self.call("vx_sdpa_prefill_softcap", q, k, v, out, seq_len, num_q_heads, num_kv_heads, head_dim, scale, softcap)

    def rope_with_freqs(self, q, k, freqs, head_dim, num_heads, num_kv_heads, seq_len, start_pos, neox):
        self.call("vx_rope_with_freqs", q, k, freqs, head_dim, num_heads, num_kv_heads, seq_len, start_pos,
                  int(bool(neox)))

    def argmax(self, inp, n):
        r = C.c_int()
        self.call("vx_argmax", inp, n, C.byref(r))
        return r.value

    # ---- QuantizedMatMul
    def matmul_q4_0(self, a, b, out, m, n, k):
        self.call("vx_matmul_q4_0", a, b, out, m, n, k)

    def matmul_q4_k(self, a, b, out, m, n, k):
        self.call("vx_matmul_q4_k", a, b, out, m, n, k)

    def matmul_q6_k(self, a, b, out, m, n, k):
        self.call("vx_matmul_q6_k", a, b, out, m, n, k)

    def matmul_q8_0(self, a, b, out, m, n, k):
        self.call("vx_matmul_q8_0", a, b, out, m, n, k)

    def matmul_q5_k(self, a, b, out, m, n, k):
        self.call("vx_matmul_q5_k", a, b, out, m, n, k)

    def matmul_q5_0(self, a, b, out, m, n, k):
        self.call("vx_matmul_q5_0", a, b, out, m, n, k)

    def matmul_bf16(self, a, b, out, m, n, k):
        self.call("vx_matmul_bf16", a, b, out, m, n, k)

    # ---- PagedKVOps
    def reshape_paged_kv(self, src, dst_base, page_table, block_offsets, num_tokens, num_kv_heads, head_dim,
                         block_size, is_value):
        self.call("vx_reshape_paged_kv", src, dst_base, page_table, block_offsets, num_tokens, num_kv_heads,
                  head_dim, block_size, int(bool(is_value)))

    def reshape_paged_kv_f16(self, src, dst_base, page_table, block_offsets, num_tokens, num_kv_heads, head_dim,
                             block_size, is_value):
        self.call("vx_reshape_paged_kv_f16", src, dst_base, page_table, block_offsets, num_tokens, num_kv_heads,
                  head_dim, block_size, int(bool(is_value)))

    def sdpa_paged_decode(self, q, kv_pool, block_table, out, num_blocks, block_size, num_q_heads, num_kv_heads,
                          head_dim, scale, tokens_in_last_block):
        self.call("vx_sdpa_paged_decode", q, kv_pool, block_table, out, num_blocks, block_size, num_q_heads,
                  num_kv_heads, head_dim, scale, tokens_in_last_block)

    def sdpa_paged_decode_f16(self, q, kv_pool, block_table, out, num_blocks, block_size, num_q_heads,
                              num_kv_heads, head_dim, scale, tokens_in_last_block):
        self.call("vx_sdpa_paged_decode_f16", q, kv_pool, block_table, out, num_blocks, block_size, num_q_heads,
                  num_kv_heads, head_dim, scale, tokens_in_last_block)

    def sdpa_paged_decode_batched(self, q, kv_pool, block_tables, out, batch_size, max_blocks, block_size,
                                  num_q_heads, num_kv_heads, head_dim, scale, seq_lens, pool_is_f16=False):
        """block_tables: list of device pointers; seq_lens: list of ints (host), as the Go method takes."""
        ptrs = (C.c_void_p * batch_size)(*block_tables)
        lens = (C.c_int32 * batch_size)(*seq_lens)
        self.call("vx_sdpa_paged_decode_batched", q, kv_pool, int(bool(pool_is_f16)), ptrs, out, batch_size,
                  max_blocks, block_size, num_q_heads, num_kv_heads, head_dim, scale, lens)

    def sdpa_paged_decode_multiquery(self, q, kv_pool, block_table, out, kv_lens, num_blocks, block_size,
                                     num_q_heads, num_kv_heads, head_dim, scale, query_len, pool_is_f16=False):
        self.call("vx_sdpa_paged_decode_multiquery", q, kv_pool, int(bool(pool_is_f16)), block_table, out,
                  kv_lens, num_blocks, block_size, num_q_heads, num_kv_heads, head_dim, scale, query_len)

    # ---- batched extensions
    def dequantize(self, fmt, src, dst, n):
        self.call("vx_dequantize", fmt, src, dst, n)

    def matmul_quant(self, fmt, a, b, out, residual, m, n, k):
        self.call("vx_matmul_quant", fmt, a, b, out, residual, m, n, k)

    def prepare_act(self, a, m, k):
        self.call("vx_prepare_act", a, m, k)

    def rmsnorm_prepare(self, x, weight, out, rows, cols, eps):
        self.call("vx_rmsnorm_prepare", x, weight, out, rows, cols, eps)

    def silu_mul_prepare(self, gate, up, out, rows, cols):
        self.call("vx_silu_mul_prepare", gate, up, out, rows, cols)

    def gelu_mul_prepare(self, gate, up, out, rows, cols):
        self.call("vx_gelu_mul_prepare", gate, up, out, rows, cols)

    def gelu_prepare(self, x, out, rows, cols):
        self.call("vx_gelu_prepare", x, out, rows, cols)

    def matmul_quant_prepared(self, fmt, b, out, residual, m, n, k):
        self.call("vx_matmul_quant_prepared", fmt, b, out, residual, m, n, k)

    @staticmethod
    def qweight(fmt, data, n, k):
        """vx_qweight for the fused decode entry points (data: device pointer of the raw blocks)."""
        return VxQWeight(fmt, data, n, k)

    def qweight_pack(self, w):
        """vx_qweight_pack: True when a packed copy was made, False when the format or shape has none."""
        rc = self._lib.vx_qweight_pack(self._h, C.byref(w))
        if rc == _l.VX_ERR_UNSUPPORTED:
            return False
        self._ck(rc)
        return True

    def qweight_unpack(self, w):
        self.call("vx_qweight_unpack", C.byref(w))

    def qweight_is_packed(self, w):
        return bool(self._lib.vx_qweight_is_packed(self._h, C.byref(w)))

    def dequantize_packed(self, w, dst):
        self.call("vx_dequantize_packed", C.byref(w), dst)

    def decode_attn_qkv_supported(self, wq, wk, wv, head_dim):
        return bool(self._lib.vx_decode_attn_qkv_supported(C.byref(wq), C.byref(wk), C.byref(wv), head_dim))

    def decode_attn_qkv(self, x, norm_weight, eps, x_prepared, wq, wk, wv, rows, positions, slot_mapping, kv_pool,
                        pool_is_f16, num_q_heads, num_kv_heads, head_dim, block_size, theta, q_out):
        self.call("vx_decode_attn_qkv", x, norm_weight, eps, int(bool(x_prepared)), C.byref(wq), C.byref(wk),
                  C.byref(wv), rows, positions, slot_mapping, kv_pool, int(bool(pool_is_f16)), num_q_heads,
                  num_kv_heads, head_dim, block_size, theta, q_out)

    def rope_table_prepare(self, positions, rows, head_dim, theta):
        self.call("vx_rope_table_prepare", positions, rows, head_dim, theta)

    def decode_attn_qkv_ex(self, x, norm_weight, eps, x_prepared, wq, wk, wv, q_bias, k_bias, v_bias, rows, positions,
                           slot_mapping, kv_pool, pool_is_f16, num_q_heads, num_kv_heads, head_dim, block_size, theta,
                           rope_dim, rope_neox, q_out):
        self.call("vx_decode_attn_qkv_ex", x, norm_weight, eps, int(bool(x_prepared)), C.byref(wq), C.byref(wk),
                  C.byref(wv), q_bias, k_bias, v_bias, rows, positions, slot_mapping, kv_pool, int(bool(pool_is_f16)),
                  num_q_heads, num_kv_heads, head_dim, block_size, theta, rope_dim, int(bool(rope_neox)), q_out)

    def prefill_attn_qkv(self, x, norm_weight, eps, x_prepared, wq, wk, wv, q_bias, k_bias, v_bias, rows, positions,
                         slot_mapping, kv_pool, pool_is_f16, num_q_heads, num_kv_heads, head_dim, block_size, theta,
                         rope_dim, rope_neox, q_out, k_out, v_out):
        self.call("vx_prefill_attn_qkv", x, norm_weight, eps, int(bool(x_prepared)), C.byref(wq), C.byref(wk),
                  C.byref(wv), q_bias, k_bias, v_bias, rows, positions, slot_mapping, kv_pool, int(bool(pool_is_f16)),
                  num_q_heads, num_kv_heads, head_dim, block_size, theta, rope_dim, int(bool(rope_neox)), q_out, k_out,
                  v_out)

    def decode_ffn_supported(self, wo, w1, w3, w2):
        return bool(self._lib.vx_decode_ffn_supported(C.byref(wo), C.byref(w1), C.byref(w3), C.byref(w2)))

    def decode_ffn(self, attn, x, wo, ffn_norm_weight, eps, w1, w3, w2, rows, next_norm_weight=None):
        self.call("vx_decode_ffn", attn, x, C.byref(wo), ffn_norm_weight, eps, C.byref(w1), C.byref(w3),
                  C.byref(w2), rows, next_norm_weight)

    def rope_store_paged(self, q, k, v, positions, slot_mapping, kv_pool, pool_is_f16, rows, num_q_heads,
                         num_kv_heads, head_dim, block_size, theta, rope_dim=0, rope_neox=False):
        self.call("vx_rope_store_paged_ex", q, k, v, positions, slot_mapping, kv_pool, int(bool(pool_is_f16)), rows,
                  num_q_heads, num_kv_heads, head_dim, block_size, theta, rope_dim, int(bool(rope_neox)))

    def sdpa_paged_decode_ragged(self, q, kv_pool, pool_is_f16, block_tables, kv_lens, out, batch, max_blocks,
                                 block_size, num_q_heads, num_kv_heads, head_dim, scale, max_kv_len, table_rows=None):
        self.call("vx_sdpa_paged_decode_ragged", q, kv_pool, int(bool(pool_is_f16)), block_tables, table_rows,
                  kv_lens, out, batch, max_blocks, block_size, num_q_heads, num_kv_heads, head_dim, scale, max_kv_len)

    def sdpa_paged_decode_ragged_noalloc(self, q, kv_pool, pool_is_f16, block_tables, kv_lens, out, batch, max_blocks,
                                         block_size, num_q_heads, num_kv_heads, head_dim, scale, max_kv_len,
                                         table_rows=None):
        self.call("vx_sdpa_paged_decode_ragged_noalloc", q, kv_pool, int(bool(pool_is_f16)), block_tables, table_rows,
                  kv_lens, out, batch, max_blocks, block_size, num_q_heads, num_kv_heads, head_dim, scale, max_kv_len)

    def sdpa_paged_decode_ragged_noalloc_bytes(self, batch, num_q_heads, num_kv_heads, head_dim, max_kv_len):
        """(bytes of partial sums the call needs, size of the fixed area)."""
        cap = C.c_size_t(0)
        need = self._lib.vx_sdpa_paged_decode_ragged_noalloc_bytes(self._h, batch, num_q_heads, num_kv_heads, head_dim,
                                                                    max_kv_len, C.byref(cap))
        return int(need), int(cap.value)

    def sdpa_paged_tree(self, q, kv_pool, pool_is_f16, block_table, out, tree_mask, tree_base, block_size,
                        num_q_heads, num_kv_heads, head_dim, scale, query_len):
        self.call("vx_sdpa_paged_tree", q, kv_pool, int(bool(pool_is_f16)), block_table, out, tree_mask,
                  tree_base, block_size, num_q_heads, num_kv_heads, head_dim, scale, query_len)

    def rope_shift(self, k, head_dim, num_kv_heads, num_tokens, shift, theta):
        self.call("vx_rope_shift", k, head_dim, num_kv_heads, num_tokens, shift, theta)

    def sample_rows(self, logits, rows, n, temperature, top_k, top_p, uniform, out_idx):
        self.call("vx_sample_rows", logits, rows, n, temperature, top_k, top_p, uniform, out_idx)

    def paged_kv_move(self, kv_pool, pool_is_f16, chain_offsets, src_slots, dst_slots, num_chains, num_kv_heads,
                      head_dim, block_size):
        self.call("vx_paged_kv_move", kv_pool, int(bool(pool_is_f16)), chain_offsets, src_slots, dst_slots,
                  num_chains, num_kv_heads, head_dim, block_size)

    def argmax_rows(self, logits, rows, n, out_idx):
        self.call("vx_argmax_rows", logits, rows, n, out_idx)

    def pack_batch(self, seq_slots, positions, q_lens, batch, total_tokens, block_tables, max_blocks, num_blocks,
                   free_list, free_count, block_size, cu_seqlens, token_pos, slot_mapping, kv_lens, status):
        self.call("vx_pack_batch", seq_slots, positions, q_lens, batch, total_tokens, block_tables, max_blocks,
                  num_blocks, free_list, free_count, block_size, cu_seqlens, token_pos, slot_mapping, kv_lens,
                  status)

    # ---- graph capture / timing
    def graph_begin_capture(self):
        self.call("vx_graph_begin_capture")

    def graph_end_capture(self):
        g = C.c_void_p()
        self.call("vx_graph_end_capture", C.byref(g))
        return g

    def graph_launch(self, g):
        self.call("vx_graph_launch", g)

    def graph_destroy(self, g):
        self._lib.vx_graph_destroy(g)

    def timer_start(self):
        self.call("vx_timer_start")

    def timer_stop_ms(self):
        ms = C.c_float()
        self.call("vx_timer_stop_ms", C.byref(ms))
        return ms.value
