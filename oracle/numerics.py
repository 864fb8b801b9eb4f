"""ctypes binding of oracle/vexel_oracle.c (test infrastructure only).

Each wrapper takes/returns numpy arrays and cites the reference function the C code
restates. Nothing here is used by the shipped library.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libvexel_oracle.so")

FMT_Q4_0, FMT_Q8_0, FMT_Q4_K, FMT_Q6_K, FMT_Q5_0, FMT_Q5_K, FMT_BF16 = 1, 2, 3, 4, 5, 6, 7
BLOCK_ELEMS = {FMT_Q4_0: 32, FMT_Q8_0: 32, FMT_Q4_K: 256, FMT_Q6_K: 256, FMT_Q5_0: 32, FMT_Q5_K: 256, FMT_BF16: 1}
BLOCK_BYTES = {FMT_Q4_0: 18, FMT_Q8_0: 34, FMT_Q4_K: 144, FMT_Q6_K: 210, FMT_Q5_0: 22, FMT_Q5_K: 176, FMT_BF16: 2}


def build(force=False):
    """Compile the oracle with gcc (a few hundred ms)."""
    if force or not os.path.exists(_LIB_PATH) or (
            os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "vexel_oracle.c"))):
        subprocess.check_call(["make", "-C", _HERE, "-s", "-B"])


def _load():
    build()
    lib = C.CDLL(_LIB_PATH)
    lib.vxo_f16_to_f32.restype = C.c_float
    lib.vxo_f16_to_f32.argtypes = [C.c_uint16]
    lib.vxo_f16_to_f32_cpu.restype = C.c_float
    lib.vxo_f16_to_f32_cpu.argtypes = [C.c_uint16]
    lib.vxo_f32_to_f16.restype = C.c_uint16
    lib.vxo_f32_to_f16.argtypes = [C.c_float]
    lib.vxo_argmax.restype = C.c_int
    lib.vxo_matmul_quant_via_dequant.restype = C.c_int
    return lib


_lib = _load()


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _u8(a):
    return np.ascontiguousarray(a, dtype=np.uint8)


# ---------------------------------------------------------------- half precision
def f16_to_f32(h):
    """dequant.go:231-261"""
    return float(_lib.vxo_f16_to_f32(int(h) & 0xFFFF))


def f16_to_f32_cpu(h):
    """cpu.go:962-992"""
    return float(_lib.vxo_f16_to_f32_cpu(int(h) & 0xFFFF))


def f32_to_f16(x):
    """Metal `(half)x`, metal_bridge_darwin.m:8641 (round to nearest even)."""
    return int(_lib.vxo_f32_to_f16(C.c_float(float(x))))


def f32_to_f16_array(x):
    x = _f32(x)
    out = np.empty(x.shape, dtype=np.uint16)
    _lib.vxo_f32_to_f16_n(_p(x), _p(out), C.c_int64(x.size))
    return out


def f16_to_f32_array(h):
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, dtype=np.float32)
    _lib.vxo_f16_to_f32_n(_p(h), _p(out), C.c_int64(h.size))
    return out


# ---------------------------------------------------------------- dequant
_DEQ = {FMT_Q4_0: "vxo_dequant_q4_0", FMT_Q8_0: "vxo_dequant_q8_0",
        FMT_Q4_K: "vxo_dequant_q4_k", FMT_Q6_K: "vxo_dequant_q6_k", FMT_Q5_0: "vxo_dequant_q5_0",
        FMT_Q5_K: "vxo_dequant_q5_k", FMT_BF16: "vxo_dequant_bf16"}


def dequantize(fmt, data, n):
    """gguf.Dequantize, dequant.go:503-538 (Q4_0/Q8_0/Q4_K/Q6_K/Q5_0/Q5_K/BF16 arms)."""
    data = _u8(data).reshape(-1)
    out = np.empty(n, dtype=np.float32)
    getattr(_lib, _DEQ[fmt])(_p(data), C.c_int64(data.size), C.c_int64(n), _p(out))
    return out


def dequantize_f16(data, n):
    data = _u8(data).reshape(-1)
    out = np.empty(n, dtype=np.float32)
    _lib.vxo_dequant_f16(_p(data), C.c_int64(data.size), C.c_int64(n), _p(out))
    return out


def get_scale_min_k4(j, q12):
    q12 = _u8(q12)
    sc, mn = C.c_uint8(), C.c_uint8()
    _lib.vxo_get_scale_min_k4(C.c_int(j), _p(q12), C.byref(sc), C.byref(mn))
    return sc.value, mn.value


# ---------------------------------------------------------------- matmul
def matmul_f32(a, b, m, n, k):
    """cpu.go:106-145"""
    a, b = _f32(a), _f32(b)
    out = np.empty((m, n), dtype=np.float32)
    _lib.vxo_matmul_f32(_p(a), _p(b), _p(out), m, n, k)
    return out


def matmul_t_f32(a, b, m, n, k):
    """cpu.go:158-197"""
    a, b = _f32(a), _f32(b)
    out = np.empty((m, n), dtype=np.float32)
    _lib.vxo_matmul_t_f32(_p(a), _p(b), _p(out), m, n, k)
    return out


_ROW_THREADS = 1
_ROW_POOL = None


def set_row_threads(n):
    """Long test runs only: the quantized matmuls cut their weight rows into n slices computed side by side. Every
    output element is still the same loop over the same numbers in the same order, so the bits do not change;
    only the wall time does. (The reference itself runs these loops on one core at M = 1.)"""
    global _ROW_THREADS, _ROW_POOL
    from concurrent.futures import ThreadPoolExecutor
    if _ROW_POOL is not None:
        _ROW_POOL.shutdown()
        _ROW_POOL = None
    _ROW_THREADS = max(1, int(n))
    if _ROW_THREADS > 1:
        _ROW_POOL = ThreadPoolExecutor(max_workers=_ROW_THREADS)


def _rows_parallel(fn, bq, m, n, k, row_bytes):
    """fn(weight bytes of rows [r0, r1), r1 - r0) -> [m, r1 - r0] on slices of the weight rows"""
    t = _ROW_THREADS
    if t <= 1 or n < 4 * t or m * n * k < (1 << 22):
        return fn(bq, n)
    rows = _u8(bq).reshape(n, row_bytes)
    cuts = [n * i // t for i in range(t + 1)]
    parts = list(_ROW_POOL.map(lambda i: fn(rows[cuts[i]:cuts[i + 1]], cuts[i + 1] - cuts[i]), range(t)))
    return np.concatenate(parts, axis=1)


def matmul_q4_0(a, bq, m, n, k):
    """cpu.go:842-911"""
    a, bq = _f32(a), _u8(bq)
    assert bq.size == n * (k // 32) * 18

    def run(rows, nr):
        rows = _u8(rows)
        out = np.empty((m, nr), dtype=np.float32)
        _lib.vxo_matmul_q4_0(_p(a), _p(rows), _p(out), m, nr, k)
        return out
    return _rows_parallel(run, bq, m, n, k, k // 32 * 18)


def matmul_quant(fmt, a, bq, m, n, k):
    """Reference CPU semantics of MatMulQ*: native loop for Q4_0 (cpu.go:842-911);
    gguf.Dequantize + matMulTransposedNaive for the others (cpu.go:916-945 panic,
    loader.go:216-271, cpu.go:158-197)."""
    if fmt == FMT_Q4_0:
        return matmul_q4_0(a, bq, m, n, k)
    a, bq = _f32(a), _u8(bq)
    assert bq.size == n * (k // BLOCK_ELEMS[fmt]) * BLOCK_BYTES[fmt]

    def run(rows, nr):
        rows = _u8(rows)
        out = np.empty((m, nr), dtype=np.float32)
        rc = _lib.vxo_matmul_quant_via_dequant(fmt, _p(a), _p(rows), _p(out), m, nr, k)
        assert rc == 0
        return out
    return _rows_parallel(run, bq, m, n, k, k // BLOCK_ELEMS[fmt] * BLOCK_BYTES[fmt])


def matmul_quant_via_dequant(fmt, a, bq, m, n, k):
    a, bq = _f32(a), _u8(bq)
    out = np.empty((m, n), dtype=np.float32)
    rc = _lib.vxo_matmul_quant_via_dequant(fmt, _p(a), _p(bq), _p(out), m, n, k)
    assert rc == 0
    return out


# ---------------------------------------------------------------- elementwise
def rmsnorm(x, w, rows, cols, eps):
    """cpu.go:200-220"""
    x, w = _f32(x), _f32(w)
    out = np.empty((rows, cols), dtype=np.float32)
    _lib.vxo_rmsnorm(_p(x), _p(w), _p(out), rows, cols, C.c_float(eps))
    return out


def rope(q, k, head_dim, num_heads, num_kv_heads, seq_len, start_pos, rope_dim, theta, neox):
    """cpu.go:226-303; returns rotated copies (q, k)."""
    q = _f32(q).copy()
    k2 = None if k is None else _f32(k).copy()
    _lib.vxo_rope(_p(q), None if k2 is None else _p(k2), head_dim, num_heads, num_kv_heads, seq_len,
                  start_pos, rope_dim, C.c_float(theta), int(bool(neox)))
    return q, k2


def rope_positions(q, k, head_dim, num_heads, num_kv_heads, positions, rope_dim, theta, neox):
    """Row r rotated as a one-row cpu.go:226-303 call with startPos=positions[r]."""
    q = _f32(q).copy()
    k2 = None if k is None else _f32(k).copy()
    pos = _i32(positions)
    _lib.vxo_rope_positions(_p(q), None if k2 is None else _p(k2), head_dim, num_heads, num_kv_heads,
                            pos.size, _p(pos), rope_dim, C.c_float(theta), int(bool(neox)))
    return q, k2


def rope_with_freqs(q, k, freqs, head_dim, num_heads, num_kv_heads, seq_len, start_pos, neox):
    """cpu.go:308-375; returns rotated copies (q, k)."""
    q = _f32(q).copy()
    k2 = None if k is None else _f32(k).copy()
    f = _f32(freqs)
    assert f.size >= head_dim // 2
    _lib.vxo_rope_with_freqs(_p(q), None if k2 is None else _p(k2), _p(f), head_dim, num_heads, num_kv_heads, seq_len,
                             start_pos, int(bool(neox)))
    return q, k2


def rope_shift(k, head_dim, num_kv_heads, num_tokens, shift, theta):
    """backend/cpu/backend.go:244-276; returns the rotated copy."""
    k2 = _f32(k).copy()
    _lib.vxo_rope_shift(_p(k2), head_dim, num_kv_heads, num_tokens, shift, C.c_float(theta))
    return k2


def silu(x):
    x = _f32(x)
    out = np.empty_like(x)
    _lib.vxo_silu(_p(x), _p(out), C.c_int64(x.size))
    return out


def silu_mul(gate, up):
    """cpu.go:390-400"""
    gate, up = _f32(gate), _f32(up)
    out = np.empty_like(gate)
    _lib.vxo_silu_mul(_p(gate), _p(up), _p(out), C.c_int64(gate.size))
    return out


def layernorm(x, weight, bias, rows, cols, eps):
    """cpu.go:404-436"""
    x, weight, bias = _f32(x), _f32(weight), _f32(bias)
    out = np.empty((rows, cols), dtype=np.float32)
    _lib.vxo_layernorm(_p(x), _p(weight), _p(bias), _p(out), rows, cols, C.c_float(eps))
    return out


def gelu(x):
    """cpu.go:440-454"""
    x = _f32(x)
    out = np.empty_like(x)
    _lib.vxo_gelu(_p(x), _p(out), C.c_int64(x.size))
    return out


def gelu_mul(gate, up):
    """cpu.go:457-473"""
    gate, up = _f32(gate), _f32(up)
    out = np.empty_like(gate)
    _lib.vxo_gelu_mul(_p(gate), _p(up), _p(out), C.c_int64(gate.size))
    return out


def add_bias(x, bias, rows, cols):
    """cpu.go:476-487"""
    x, bias = _f32(x), _f32(bias)
    out = np.empty((rows, cols), dtype=np.float32)
    _lib.vxo_add_bias(_p(x), _p(bias), _p(out), rows, cols)
    return out


def scale_buffer(buf, scale):
    """cpu.go:558-563; returns the scaled copy."""
    b = _f32(buf).copy()
    _lib.vxo_scale_buffer(_p(b), C.c_float(scale), C.c_int64(b.size))
    return b


def logit_softcap(logits, cap):
    """model.go:336-350; returns the capped copy."""
    out = _f32(logits).copy()
    _lib.vxo_logit_softcap(_p(out), C.c_int64(out.size), C.c_float(cap))
    return out


def medusa_forward(hidden, fc1, fc2):
    """heads.go:83-117 for one head: hidden [H], fc1 [H,H], fc2 [H,V] (input index first) -> (intermediate, logits)."""
    hidden, fc1, fc2 = _f32(hidden), _f32(fc1), _f32(fc2)
    h, v = fc1.shape[0], fc2.shape[1]
    assert fc1.shape == (h, h) and fc2.shape == (h, v) and hidden.shape == (h,)
    inter, logits = np.empty(h, dtype=np.float32), np.empty(v, dtype=np.float32)
    _lib.vxo_medusa_forward(_p(hidden), _p(fc1), _p(fc2), _p(inter), _p(logits), h, v)
    return inter, logits


def softmax(x, rows, cols):
    """cpu.go:490-518"""
    x = _f32(x)
    out = np.empty((rows, cols), dtype=np.float32)
    _lib.vxo_softmax(_p(x), _p(out), rows, cols)
    return out


def add(a, b):
    a, b = _f32(a), _f32(b)
    out = np.empty_like(a)
    _lib.vxo_add(_p(a), _p(b), _p(out), C.c_int64(a.size))
    return out


def mul(a, b):
    a, b = _f32(a), _f32(b)
    out = np.empty_like(a)
    _lib.vxo_mul(_p(a), _p(b), _p(out), C.c_int64(a.size))
    return out


def embedding(ids, table, vocab, dim, out=None):
    """cpu.go:543-555 (out-of-range ids leave the row as it was)."""
    ids, table = _i32(ids), _f32(table)
    if out is None:
        out = np.zeros((ids.size, dim), dtype=np.float32)
    _lib.vxo_embedding(_p(ids), ids.size, _p(table), _p(out), vocab, dim)
    return out


def argmax(x):
    """sampler.go:80-91"""
    x = _f32(x).reshape(-1)
    return int(_lib.vxo_argmax(_p(x), x.size))


# ---------------------------------------------------------------- attention
def sdpa(q, k, v, kv_len, num_q_heads, num_kv_heads, head_dim, scale, kv_head_stride):
    """cpu.go:568-632"""
    q, k, v = _f32(q), _f32(k), _f32(v)
    out = np.empty((num_q_heads, head_dim), dtype=np.float32)
    _lib.vxo_sdpa(_p(q), _p(k), _p(v), _p(out), kv_len, num_q_heads, num_kv_heads, head_dim,
                  C.c_float(scale), kv_head_stride)
    return out


def sdpa_prefill(q, k, v, seq_len, num_q_heads, num_kv_heads, head_dim, scale):
    """cpu.go:635-701"""
    q, k, v = _f32(q), _f32(k), _f32(v)
    out = np.empty((seq_len, num_q_heads, head_dim), dtype=np.float32)
    _lib.vxo_sdpa_prefill(_p(q), _p(k), _p(v), _p(out), seq_len, num_q_heads, num_kv_heads, head_dim,
                          C.c_float(scale))
    return out


def sdpa_softcap(q, k, v, kv_len, num_q_heads, num_kv_heads, head_dim, scale, softcap, kv_head_stride):
    """cpu.go:705-765"""
    q, k, v = _f32(q), _f32(k), _f32(v)
    out = np.empty((num_q_heads, head_dim), dtype=np.float32)
    _lib.vxo_sdpa_softcap(_p(q), _p(k), _p(v), _p(out), kv_len, num_q_heads, num_kv_heads, head_dim,
                          C.c_float(scale), C.c_float(softcap), kv_head_stride)
    return out


def sdpa_prefill_softcap(q, k, v, seq_len, num_q_heads, num_kv_heads, head_dim, scale, softcap):
    """cpu.go:770-841"""
    q, k, v = _f32(q), _f32(k), _f32(v)
    out = np.empty((seq_len, num_q_heads, head_dim), dtype=np.float32)
    _lib.vxo_sdpa_prefill_softcap(_p(q), _p(k), _p(v), _p(out), seq_len, num_q_heads, num_kv_heads, head_dim,
                                  C.c_float(scale), C.c_float(softcap))
    return out


def reshape_paged_kv(src, pool, block_idx, block_off, num_kv_heads, head_dim, block_size, is_value):
    """In-place scatter into pool (float32 or uint16-as-f16 numpy array).
    metal_bridge_darwin.m:8539-8642"""
    src = _f32(src)
    bi, bo = _i32(block_idx), _i32(block_off)
    assert pool.flags["C_CONTIGUOUS"]
    if pool.dtype == np.float32:
        fn = _lib.vxo_reshape_paged_kv_f32
    else:
        assert pool.dtype == np.uint16
        fn = _lib.vxo_reshape_paged_kv_f16
    fn(_p(src), _p(pool), _p(bi), _p(bo), bi.size, num_kv_heads, head_dim, block_size, int(bool(is_value)))


def _pool_kind(pool):
    assert pool.flags["C_CONTIGUOUS"]
    if pool.dtype == np.float32:
        return 0
    assert pool.dtype == np.uint16
    return 1


def sdpa_paged_decode(q, pool, block_table, num_blocks, block_size, num_q_heads, num_kv_heads, head_dim,
                      scale, tokens_in_last_block):
    """PagedKVOps.SDPAPagedDecode[F16], backend.go:426-438"""
    q, bt = _f32(q), _i32(block_table)
    out = np.empty((num_q_heads, head_dim), dtype=np.float32)
    _lib.vxo_sdpa_paged_decode(_p(q), _p(pool), _pool_kind(pool), _p(bt), _p(out), num_blocks, block_size,
                               num_q_heads, num_kv_heads, head_dim, C.c_float(scale), tokens_in_last_block)
    return out


def sdpa_paged_decode_batched(q, pool, block_tables, block_size, num_q_heads, num_kv_heads, head_dim,
                              scale, seq_lens):
    """PagedKVOps.SDPAPagedDecodeBatched, backend.go:440-454; block_tables [B, max_blocks]."""
    q, bts, sl = _f32(q), _i32(block_tables), _i32(seq_lens)
    batch, max_blocks = bts.shape
    out = np.empty((batch, num_q_heads, head_dim), dtype=np.float32)
    _lib.vxo_sdpa_paged_decode_batched(_p(q), _p(pool), _pool_kind(pool), _p(bts), _p(out), batch, max_blocks,
                                       block_size, num_q_heads, num_kv_heads, head_dim, C.c_float(scale), _p(sl))
    return out


def sdpa_paged_multiquery(q, pool, block_table, kv_lens, block_size, num_q_heads, num_kv_heads, head_dim,
                          scale, tree_mask=None, tree_base=0):
    """PagedKVOps.SDPAPagedDecodeMultiquery, backend.go:459-465 (+ tree-mask extension)."""
    q, bt = _f32(q), _i32(block_table)
    qlen = q.size // (num_q_heads * head_dim)
    out = np.empty((qlen, num_q_heads, head_dim), dtype=np.float32)
    kl = _i32(kv_lens if kv_lens is not None else np.zeros(qlen))
    tm = None if tree_mask is None else _u8(tree_mask)
    _lib.vxo_sdpa_paged_multiquery(_p(q), _p(pool), _pool_kind(pool), _p(bt), _p(out), _p(kl), block_size,
                                   num_q_heads, num_kv_heads, head_dim, C.c_float(scale), qlen,
                                   None if tm is None else _p(tm), tree_base)
    return out
