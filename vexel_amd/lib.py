"""ctypes binding of libvexel_hip.so: one Python callable per C-ABI symbol of
include/vexel_hip.h. Loading fails loudly when the library has not been built; there
is no CPU fallback anywhere in this package."""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libvexel_hip.so")

VX_OK, VX_ERR_INVALID, VX_ERR_OOM, VX_ERR_HIP, VX_ERR_UNSUPPORTED = 0, 1, 2, 3, 4
VX_Q4_0, VX_Q8_0, VX_Q4_K, VX_Q6_K = 1, 2, 3, 4

_vp, _i, _f, _sz, _i64 = C.c_void_p, C.c_int, C.c_float, C.c_size_t, C.c_int64

# name -> (restype, argtypes); mirrors include/vexel_hip.h declaration by declaration
SIGNATURES = {
    "vx_backend_create": (_i, [_i, C.POINTER(_vp)]),
    "vx_backend_destroy": (None, [_vp]),
    "vx_backend_device": (_i, [_vp]),
    "vx_backend_set_attn_merge": (_i, [_vp, _i]),
    "vx_last_error": (C.c_char_p, []),
    "vx_scratch_generation": (C.c_uint64, [_vp]),
    "vx_alloc": (_vp, [_vp, _sz]),
    "vx_alloc_permanent": (_vp, [_vp, _sz]),
    "vx_free": (None, [_vp, _vp]),
    "vx_reset_pool": (None, [_vp]),
    "vx_to_device": (_i, [_vp, _vp, _vp, _sz]),
    "vx_to_host": (_i, [_vp, _vp, _vp, _sz]),
    "vx_sync": (_i, [_vp]),
    "vx_copy_buffer": (_i, [_vp, _vp, _sz, _vp, _sz, _sz]),
    "vx_begin_batch": (_i, [_vp]),
    "vx_end_batch": (_i, [_vp]),
    "vx_memory_barrier": (_i, [_vp]),
    "vx_matmul": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i]),
    "vx_matmul_transposed": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i]),
    "vx_rmsnorm": (_i, [_vp, _vp, _vp, _vp, _i, _i, _f]),
    "vx_rope": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _f, _i]),
    "vx_silu": (_i, [_vp, _vp, _vp, _i]),
    "vx_silu_mul": (_i, [_vp, _vp, _vp, _vp, _i]),
    "vx_softmax": (_i, [_vp, _vp, _vp, _i, _i]),
    "vx_add": (_i, [_vp, _vp, _vp, _vp, _i]),
    "vx_mul": (_i, [_vp, _vp, _vp, _vp, _i]),
    "vx_embedding": (_i, [_vp, _vp, _i, _vp, _vp, _i, _i]),
    "vx_sdpa": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _f, _i]),
    "vx_sdpa_prefill": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _f]),
    "vx_argmax": (_i, [_vp, _vp, _i, C.POINTER(_i)]),
    "vx_medusa_forward": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i]),
    "vx_topk_rows": (_i, [_vp, _vp, _i, _i, _i, _vp, _vp]),
    "vx_logit_softcap": (_i, [_vp, _vp, _i, _f]),
    "vx_layernorm": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _f]),
    "vx_gelu": (_i, [_vp, _vp, _vp, _i]),
    "vx_gelu_mul": (_i, [_vp, _vp, _vp, _vp, _i]),
    "vx_add_bias": (_i, [_vp, _vp, _vp, _vp, _i, _i]),
    "vx_scale_buffer": (_i, [_vp, _vp, _f, _i]),
    "vx_sdpa_softcap": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _f, _f, _i]),
    "vx_sdpa_prefill_softcap": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _f, _f]),
    "vx_rope_with_freqs": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i]),
    "vx_matmul_q4_0": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i]),
    "vx_matmul_q4_k": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i]),
    "vx_matmul_q6_k": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i]),
    "vx_matmul_q8_0": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i]),
    "vx_matmul_q5_k": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i]),
    "vx_matmul_q5_0": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i]),
    "vx_matmul_bf16": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i]),
    "vx_reshape_paged_kv": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i]),
    "vx_reshape_paged_kv_f16": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i]),
    "vx_sdpa_paged_decode": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _f, _i]),
    "vx_sdpa_paged_decode_f16": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _f, _i]),
    "vx_sdpa_paged_decode_batched": (_i, [_vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i, _i, _i, _f, _vp]),
    "vx_sdpa_paged_decode_multiquery": (_i, [_vp, _vp, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _i, _f, _i]),
    "vx_dequantize": (_i, [_vp, _i, _vp, _vp, _i64]),
    "vx_matmul_quant": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _i, _i, _i]),
    "vx_prepare_act": (_i, [_vp, _vp, _i, _i]),
    "vx_rmsnorm_prepare": (_i, [_vp, _vp, _vp, _vp, _i, _i, _f]),
    "vx_silu_mul_prepare": (_i, [_vp, _vp, _vp, _vp, _i, _i]),
    "vx_gelu_mul_prepare": (_i, [_vp, _vp, _vp, _vp, _i, _i]),
    "vx_gelu_prepare": (_i, [_vp, _vp, _vp, _i, _i]),
    "vx_matmul_quant_prepared": (_i, [_vp, _i, _vp, _vp, _vp, _i, _i, _i]),
    "vx_matmul_quant_has_fast_path": (_i, [_i, _vp, _i, _i]),
    "vx_last_matmul_kernel": (C.c_char_p, [_vp]),
    "vx_rope_table_prepare": (_i, [_vp, _vp, _i, _i, _f]),
    "vx_decode_attn_qkv_supported": (_i, [_vp, _vp, _vp, _i]),
    "vx_decode_attn_qkv_ex": (_i, [_vp, _vp, _vp, _f, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _i,
                                   _f, _i, _i, _vp]),
    "vx_decode_attn_qkv": (_i, [_vp, _vp, _vp, _f, _i, _vp, _vp, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _i, _f, _vp]),
    "vx_prefill_attn_qkv": (_i, [_vp, _vp, _vp, _f, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _i,
                                 _f, _i, _i, _vp, _vp, _vp]),
    "vx_decode_ffn_supported": (_i, [_vp, _vp, _vp, _vp]),
    "vx_qweight_pack": (_i, [_vp, _vp]),
    "vx_qweight_unpack": (_i, [_vp, _vp]),
    "vx_qweight_is_packed": (_i, [_vp, _vp]),
    "vx_dequantize_packed": (_i, [_vp, _vp, _vp]),
    "vx_decode_ffn": (_i, [_vp, _vp, _vp, _vp, _vp, _f, _vp, _vp, _vp, _i, _vp]),
    "vx_rope_store_paged": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _f]),
    "vx_rope_store_paged_ex": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _f, _i, _i]),
    "vx_sdpa_paged_decode_split_supported": (_i, [_i, _i, _i, _i, _i]),
    "vx_sdpa_paged_decode_ragged": (_i, [_vp, _vp, _vp, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _f, _i]),
    "vx_sdpa_paged_decode_ragged_noalloc": (_i, [_vp, _vp, _vp, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _f, _i]),
    "vx_sdpa_paged_decode_ragged_noalloc_bytes": (_sz, [_vp, _i, _i, _i, _i, _i, C.POINTER(_sz)]),
    "vx_sdpa_paged_tree": (_i, [_vp, _vp, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _i, _f, _i]),
    "vx_argmax_rows": (_i, [_vp, _vp, _i, _i, _vp]),
    "vx_sdpa_paged_tree_rows_per_entry": (_i, [_i, _i, _i, _i, _i]),
    "vx_sdpa_paged_tree_batched": (_i, [_vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _f, _i]),
    "vx_rope_shift": (_i, [_vp, _vp, _i, _i, _i, _i, _f]),
    "vx_sample_rows": (_i, [_vp, _vp, _i, _i, _vp, _vp, _vp, _vp, _vp]),
    "vx_paged_kv_copy_shifted": (_i, [_vp, _vp, _i, _vp, _vp, _i, _i, _i, _i, _i, _f]),
    "vx_paged_kv_move": (_i, [_vp, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i]),
    "vx_pack_batch": (_i, [_vp, _vp, _vp, _vp, _i, _i, _vp, _i, _vp, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp]),
    "vx_decode_advance": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i]),
    "vx_graph_begin_capture": (_i, [_vp]),
    "vx_graph_end_capture": (_i, [_vp, C.POINTER(_vp)]),
    "vx_graph_launch": (_i, [_vp, _vp]),
    "vx_graph_destroy": (None, [_vp]),
    "vx_timer_start": (_i, [_vp]),
    "vx_timer_stop_ms": (_i, [_vp, C.POINTER(_f)]),
}

_lib = None


def load():
    """Loads the shared library (dlopen only: no GPU call is made) and binds every symbol."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("%s is missing: build it with `python -m vexel_amd.build` "
                               "(there is no CPU fallback)" % LIB_PATH)
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)  # AttributeError if the symbol is not exported
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib
