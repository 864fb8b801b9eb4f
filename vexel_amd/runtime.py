"""ModelRuntime: Python handle on libvexel_host.so, the C++ restatement of the Go runtime
pieces that drive the batched-decode path (inference/runtime: GPUBlockPool, BlockRuntime.
ExecuteWithPagedKV, ModelRuntime.DecodeWithPagedKVBatched / PrefillWithPagedKV). Method
names follow the Go methods in snake_case. Nothing is computed in Python."""
import ctypes as C
import os

import numpy as np

from . import lib as _l
from .backend import HipBackend, VexelError, VxQWeight

HOST_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libvexel_host.so")


class VhConfig(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("num_layers", "hidden", "num_heads", "num_kv_heads", "head_dim", "ffn",
                                        "vocab")] + \
               [("eps", C.c_float), ("rope_theta", C.c_float)] + \
               [(n, C.c_int) for n in ("block_size", "pool_blocks", "max_seqs", "max_blocks_per_seq", "max_batch",
                                        "kv_fp16")]


VhQWeight = VxQWeight  # vh_qweight is a typedef of vx_qweight
VH_F32 = 0             # vh_qweight.fmt of a float32 output head


class VhLoadOptions(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("block_size", "pool_blocks", "max_seqs", "max_blocks_per_seq", "max_batch",
                                        "kv_fp16")]


class VhLayerWeights(C.Structure):
    _fields_ = [("attn_norm", C.c_void_p), ("ffn_norm", C.c_void_p)] + \
               [(n, VhQWeight) for n in ("wq", "wk", "wv", "wo", "w1", "w2", "w3")]


class VhArch(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("norm_type", "mlp_type", "parallel_residual", "rope_dim", "rope_neox",
                                        "post_norms")] + [("attn_softcap", C.c_float), ("embedding_scale", C.c_float),
                                                         ("final_softcap", C.c_float)]


EXTRA_NAMES = ("attn_norm_bias", "ffn_norm_bias", "wq_bias", "wk_bias", "wv_bias", "wo_bias", "w1_bias", "w2_bias",
               "post_attn_norm", "post_ffn_norm")


class VhLayerExtras(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in EXTRA_NAMES]


NORM_TYPES = {"rms": 0, "layer": 1}
MLP_TYPES = {"swiglu": 0, "gelu": 1, "geglu": 2}

_host = None


def load_host():
    global _host
    if _host is None:
        _l.load()
        if not os.path.exists(HOST_LIB_PATH):
            raise RuntimeError("%s is missing: build it with `python -m vexel_amd.build`" % HOST_LIB_PATH)
        h = C.CDLL(HOST_LIB_PATH)
        h.vh_last_error.restype = C.c_char_p
        h.vh_kv_pool.restype = C.c_void_p
        h.vh_kv_pool.argtypes = [C.c_void_p, C.c_int]
        h.vh_step_buffers.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
        h.vh_step_buffers.restype = None
        h.vh_model_create.argtypes = [C.c_void_p, C.POINTER(VhConfig), C.POINTER(C.c_void_p)]
        h.vh_model_destroy.argtypes = [C.c_void_p]
        h.vh_model_destroy.restype = None
        h.vh_model_get_config.argtypes = [C.c_void_p, C.POINTER(VhConfig)]
        h.vh_model_get_config.restype = None
        h.vh_model_load_gguf.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(VhLoadOptions), C.POINTER(C.c_void_p)]
        h.vh_model_set_fused.argtypes = [C.c_void_p, C.c_int]
        h.vh_model_set_fused.restype = None
        h.vh_model_set_layer.argtypes = [C.c_void_p, C.c_int, C.POINTER(VhLayerWeights)]
        h.vh_model_set_head.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(VhQWeight)]
        h.vh_model_set_architecture.argtypes = [C.c_void_p, C.POINTER(VhArch)]
        h.vh_model_set_layer_extras.argtypes = [C.c_void_p, C.c_int, C.POINTER(VhLayerExtras)]
        h.vh_model_set_final_norm_bias.argtypes = [C.c_void_p, C.c_void_p]
        for name in ("vh_pool_create_sequence", "vh_pool_delete_sequence", "vh_pool_has_sequence", "vh_pool_seq_len"):
            getattr(h, name).argtypes = [C.c_void_p, C.c_int64]
        h.vh_pool_truncate_sequence.argtypes = [C.c_void_p, C.c_int64, C.c_int]
        h.vh_pool_share_blocks.argtypes = [C.c_void_p, C.c_int64, C.c_int64, C.c_int]
        h.vh_fragment_cache.argtypes = [C.c_void_p, C.c_char_p, C.c_int64]
        h.vh_fragment_insert.argtypes = [C.c_void_p, C.c_int64, C.c_char_p, C.c_int, C.POINTER(C.c_int)]
        h.vh_fragment_delete.argtypes = [C.c_void_p, C.c_char_p]
        h.vh_fragment_tokens.argtypes = [C.c_void_p, C.c_char_p]
        h.vh_fragment_count.argtypes = [C.c_void_p]
        h.vh_pool_block_stats.argtypes = [C.c_void_p] + [C.POINTER(C.c_int)] * 3
        h.vh_pool_block_stats.restype = None
        h.vh_pool_block_table.argtypes = [C.c_void_p, C.c_int64, C.c_void_p, C.c_int]
        h.vh_pool_adopt_blocks.argtypes = [C.c_void_p, C.c_int64, C.c_void_p, C.c_int, C.c_int]
        h.vh_pool_device_matches_host.argtypes = [C.c_void_p]
        h.vh_decode_batched.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]
        h.vh_prefill.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int64, C.c_int, C.c_int, C.c_void_p]
        h.vh_verify_tree.argtypes = [C.c_void_p, C.c_int] + [C.c_void_p] * 10
        h.vh_decode_graph.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int,
                                      C.c_void_p, C.POINTER(C.c_float)]
        _host = h
    return _host


class VhSchedConfig(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("max_batch_size", "max_tokens", "eos_token", "prefill_chunk")]


class Scheduler:
    """scheduler.Scheduler over a ModelRuntime: add_sequence / step / remove_sequence; the loop is the caller's."""

    def __init__(self, mr, max_batch_size, max_tokens=0, eos_token=2, prefill_chunk=0):
        self._h = load_host()
        h = self._h
        if not getattr(h, "_sched_bound", False):
            h.vh_sched_create.argtypes = [C.c_void_p, C.POINTER(VhSchedConfig), C.POINTER(C.c_void_p)]
            h.vh_sched_destroy.argtypes = [C.c_void_p]
            h.vh_sched_destroy.restype = None
            h.vh_sched_add_sequence.argtypes = [C.c_void_p, C.c_int64, C.c_void_p, C.c_int, C.c_int]
            h.vh_sched_set_sampling.argtypes = [C.c_void_p, C.c_int64, C.c_float, C.c_int, C.c_float, C.c_uint64]
            h.vh_sched_remove_sequence.argtypes = [C.c_void_p, C.c_int64]
            h.vh_sched_sequence_count.argtypes = [C.c_void_p]
            h.vh_sched_state.argtypes = [C.c_void_p, C.c_int64]
            h.vh_sched_position.argtypes = [C.c_void_p, C.c_int64]
            h.vh_sched_generated.argtypes = [C.c_void_p, C.c_int64, C.c_void_p, C.c_int]
            h.vh_sched_step.argtypes = [C.c_void_p, C.POINTER(C.c_int)]
            h.vh_argmax.argtypes = [C.c_void_p, C.c_int]
            h.vh_sample.argtypes = [C.c_void_p, C.c_int, C.c_float, C.c_int, C.c_float, C.c_float]
            h._sched_bound = True
        self.mr = mr
        cfg = VhSchedConfig(max_batch_size, max_tokens, eos_token, prefill_chunk)
        s = C.c_void_p()
        self._s = None
        self._ck(h.vh_sched_create(mr._m, C.byref(cfg), C.byref(s)))
        self._s = s

    def _ck(self, rc):
        if rc != 0:
            raise VexelError(rc, self._h.vh_last_error().decode())

    def close(self):
        if self._s:
            self._h.vh_sched_destroy(self._s)
            self._s = None

    def add_sequence(self, seq_id, prompt, max_tokens=0):
        p = np.ascontiguousarray(prompt, dtype=np.int32)
        self._ck(self._h.vh_sched_add_sequence(self._s, seq_id, p.ctypes.data, p.size, max_tokens))

    def set_sampling(self, seq_id, temperature, top_k, top_p, seed):
        self._ck(self._h.vh_sched_set_sampling(self._s, seq_id, temperature, top_k, top_p, seed))

    def remove_sequence(self, seq_id):
        self._ck(self._h.vh_sched_remove_sequence(self._s, seq_id))

    def sequence_count(self):
        return self._h.vh_sched_sequence_count(self._s)

    def state(self, seq_id):
        return self._h.vh_sched_state(self._s, seq_id)

    def position(self, seq_id):
        return self._h.vh_sched_position(self._s, seq_id)

    def generated(self, seq_id):
        n = self._h.vh_sched_generated(self._s, seq_id, None, 0)
        if n < 0:
            return None
        out = np.zeros(max(n, 1), dtype=np.int32)
        self._h.vh_sched_generated(self._s, seq_id, out.ctypes.data, n)
        return [int(x) for x in out[:n]]

    def step(self):
        n = C.c_int()
        self._ck(self._h.vh_sched_step(self._s, C.byref(n)))
        return n.value

    def sample(self, logits, temperature, top_k, top_p, r):
        a = np.ascontiguousarray(logits, dtype=np.float32)
        return self._h.vh_sample(a.ctypes.data, a.size, temperature, top_k, top_p, r)


class ModelRuntime:
    def __init__(self, be: HipBackend, num_layers, hidden, num_heads, num_kv_heads, head_dim, ffn, vocab,
                 eps=1e-5, rope_theta=10000.0, block_size=16, pool_blocks=256, max_seqs=64,
                 max_blocks_per_seq=None, max_batch=64, kv_fp16=True):
        self._h = load_host()
        self.be = be
        if max_blocks_per_seq is None:
            max_blocks_per_seq = pool_blocks
        self.cfg = VhConfig(num_layers, hidden, num_heads, num_kv_heads, head_dim, ffn, vocab, eps, rope_theta,
                            block_size, pool_blocks, max_seqs, max_blocks_per_seq, max_batch, int(bool(kv_fp16)))
        m = C.c_void_p()
        self._ck(self._h.vh_model_create(be._h, C.byref(self.cfg), C.byref(m)))
        self._m = m
        self._keep = []   # device buffers owned by this model

    @classmethod
    def from_gguf(cls, be: HipBackend, path, block_size=16, pool_blocks=256, max_seqs=64, max_blocks_per_seq=None,
                  max_batch=64, kv_fp16=True):
        """ModelRuntime.LoadWeightsGGUF + CopyWeightsToDevice (runtime/loader.go): a LLaMA-family checkpoint read
        by the C++ loader; the model owns the device copies of the weights."""
        self = cls.__new__(cls)
        self._h = load_host()
        self.be = be
        opt = VhLoadOptions(block_size, pool_blocks, max_seqs, max_blocks_per_seq or pool_blocks, max_batch,
                            int(bool(kv_fp16)))
        m = C.c_void_p()
        self._m = None
        self._keep = []
        self._ck(self._h.vh_model_load_gguf(be._h, os.fsencode(path), C.byref(opt), C.byref(m)))
        self._m = m
        self.cfg = VhConfig()
        self._h.vh_model_get_config(m, C.byref(self.cfg))
        return self

    def _ck(self, rc):
        if rc != 0:
            raise VexelError(rc, self._h.vh_last_error().decode())

    def close(self):
        if self._m:
            self._h.vh_model_destroy(self._m)
            self._m = None
            for p in self._keep:
                self.be.free(p)
            self._keep = []

    # ---- weights
    def _up(self, arr):
        p = self.be.upload(np.ascontiguousarray(arr), permanent=True)
        self._keep.append(p)
        return p

    def adopt_device_buffer(self, ptr):
        """The model frees `ptr` (a vx_alloc_permanent buffer) when it is closed."""
        self._keep.append(ptr)

    @staticmethod
    def qweight(fmt, dev_ptr, n, k):
        return VhQWeight(fmt, dev_ptr, n, k)

    def set_layer(self, layer, attn_norm, ffn_norm, weights):
        """weights: dict name -> (fmt, numpy uint8 rows | device pointer, n, k) for wq wk wv wo w1 w2 w3."""
        lw = VhLayerWeights()
        lw.attn_norm = attn_norm if isinstance(attn_norm, int) else self._up(np.asarray(attn_norm, dtype=np.float32))
        lw.ffn_norm = ffn_norm if isinstance(ffn_norm, int) else self._up(np.asarray(ffn_norm, dtype=np.float32))
        ptrs = {}
        # matrices that one launch multiplies together go into one device buffer, back to back, when they come
        # from the host in one format and width: the kernels then see a single row range
        for group in (("wq", "wk", "wv"), ("w1", "w3")):
            ws = [weights.get(n_) for n_ in group]
            if all(w is not None and not isinstance(w[1], int) for w in ws) and len({(w[0], w[3]) for w in ws}) == 1:
                rows = [np.ascontiguousarray(w[1]).reshape(w[2], -1) for w in ws]
                if len({r.shape[1] for r in rows}) == 1 and rows[0].shape[1] % 16 == 0:
                    base = self._up(np.concatenate(rows, axis=0))
                    off = 0
                    for n_, r in zip(group, rows):
                        ptrs[n_] = base + off
                        off += r.nbytes
        for name in ("wq", "wk", "wv", "wo", "w1", "w2", "w3"):
            if weights.get(name) is None:          # w3 of a GELU MLP
                continue
            fmt, data, n, k = weights[name]
            ptr = ptrs.get(name) or (data if isinstance(data, int) else self._up(data))
            setattr(lw, name, VhQWeight(fmt, ptr, n, k))
        self._ck(self._h.vh_model_set_layer(self._m, layer, C.byref(lw)))

    def set_architecture(self, norm_type="rms", mlp_type="swiglu", parallel_residual=False, rope_dim=0, rope_neox=False,
                         post_norms=False, attn_softcap=0.0, embedding_scale=0.0, final_softcap=0.0):
        """The switches of runtime/config.go:14-62,120-131; any non-default one selects block.go's general sequence."""
        a = VhArch(NORM_TYPES[norm_type], MLP_TYPES[mlp_type], int(bool(parallel_residual)), rope_dim,
                   int(bool(rope_neox)), int(bool(post_norms)), attn_softcap, embedding_scale, final_softcap)
        self._ck(self._h.vh_model_set_architecture(self._m, C.byref(a)))

    def set_layer_extras(self, layer, **tensors):
        """Biases and post-norm weights of a layer (block.go:266-283): float32 vectors by name, absent = None."""
        e = VhLayerExtras()
        for name, arr in tensors.items():
            if name not in EXTRA_NAMES:
                raise KeyError(name)
            if arr is not None:
                setattr(e, name, arr if isinstance(arr, int) else self._up(np.asarray(arr, dtype=np.float32)))
        self._ck(self._h.vh_model_set_layer_extras(self._m, layer, C.byref(e)))

    def set_final_norm_bias(self, bias):
        self._ck(self._h.vh_model_set_final_norm_bias(
            self._m, bias if isinstance(bias, int) else self._up(np.asarray(bias, dtype=np.float32))))

    def set_head(self, embedding_f32, final_norm, lm_head):
        """embedding_f32: numpy [vocab,hidden] float32 or device pointer; lm_head: (fmt, data, n, k)."""
        emb = embedding_f32 if isinstance(embedding_f32, int) else self._up(np.asarray(embedding_f32, dtype=np.float32))
        fn = final_norm if isinstance(final_norm, int) else self._up(np.asarray(final_norm, dtype=np.float32))
        fmt, data, n, k = lm_head
        ptr = data if isinstance(data, int) else self._up(data)
        qw = VhQWeight(fmt, ptr, n, k)
        self._ck(self._h.vh_model_set_head(self._m, emb, fn, C.byref(qw)))

    def set_fused(self, on):
        """Decode through the fused entry points where the weights allow it (default) or, when off,
        through one backend call per operation as runtime/block.go does; the two agree to float32
        summation order."""
        self._h.vh_model_set_fused(self._m, int(bool(on)))

    def kv_pool(self, layer):
        return self._h.vh_kv_pool(self._m, layer)

    def step_buffers(self):
        """(block-table matrix, table rows, kv lengths): device addresses of the last decode step's metadata."""
        p = [C.c_void_p(), C.c_void_p(), C.c_void_p()]
        self._h.vh_step_buffers(self._m, C.byref(p[0]), C.byref(p[1]), C.byref(p[2]))
        return tuple(x.value for x in p)

    # ---- GPUBlockPool
    def create_sequence(self, seq_id):
        self._ck(self._h.vh_pool_create_sequence(self._m, seq_id))

    def delete_sequence(self, seq_id):
        self._ck(self._h.vh_pool_delete_sequence(self._m, seq_id))

    def truncate_sequence(self, seq_id, new_len):
        self._ck(self._h.vh_pool_truncate_sequence(self._m, seq_id, new_len))

    def has_sequence(self, seq_id):
        return bool(self._h.vh_pool_has_sequence(self._m, seq_id))

    def share_blocks(self, src, dst, num_tokens):
        self._ck(self._h.vh_pool_share_blocks(self._m, src, dst, num_tokens))

    # ---- named fragments (kv/fragment.go, kv/paged_cache.go:285-343)
    def cache_fragment(self, name, seq_id):
        self._ck(self._h.vh_fragment_cache(self._m, name.encode(), seq_id))

    def insert_fragment(self, seq_id, name, insert_pos):
        """-> tokens inserted (0 when no fragment has that name)"""
        n = C.c_int(0)
        self._ck(self._h.vh_fragment_insert(self._m, seq_id, name.encode(), insert_pos, C.byref(n)))
        return n.value

    def delete_fragment(self, name):
        self._ck(self._h.vh_fragment_delete(self._m, name.encode()))

    def fragment_tokens(self, name):
        return self._h.vh_fragment_tokens(self._m, name.encode())

    def fragment_count(self):
        return self._h.vh_fragment_count(self._m)

    def block_stats(self):
        a, b, c = C.c_int(), C.c_int(), C.c_int()
        self._h.vh_pool_block_stats(self._m, C.byref(a), C.byref(b), C.byref(c))
        return a.value, b.value, c.value

    def seq_len(self, seq_id):
        return self._h.vh_pool_seq_len(self._m, seq_id)

    def block_table(self, seq_id):
        cap = self.cfg.max_blocks_per_seq + self.cfg.pool_blocks
        buf = np.zeros(cap, dtype=np.int32)
        n = self._h.vh_pool_block_table(self._m, seq_id, buf.ctypes.data, cap)
        return None if n < 0 else [int(x) for x in buf[:n]]

    def adopt_blocks(self, seq_id, blocks, seq_len):
        b = np.ascontiguousarray(blocks, dtype=np.int32)
        self._ck(self._h.vh_pool_adopt_blocks(self._m, seq_id, b.ctypes.data, b.size, seq_len))

    def device_matches_host(self):
        r = self._h.vh_pool_device_matches_host(self._m)
        if r < 0:
            raise VexelError(1, "device mirror read failed")
        return bool(r)

    # ---- drivers
    def decode_with_paged_kv_batched(self, tokens, seq_ids, positions, want_logits=True):
        """-> (logits [B,V] or None, argmax [B])"""
        t = np.ascontiguousarray(tokens, dtype=np.int32)
        s = np.ascontiguousarray(seq_ids, dtype=np.int64)
        p = np.ascontiguousarray(positions, dtype=np.int32)
        b = t.size
        logits = np.empty((b, self.cfg.vocab), dtype=np.float32) if want_logits else None
        am = np.empty(b, dtype=np.int32)
        self._ck(self._h.vh_decode_batched(self._m, t.ctypes.data, s.ctypes.data, p.ctypes.data, b,
                                           logits.ctypes.data if want_logits else None, am.ctypes.data))
        return logits, am

    def prefill_with_paged_kv(self, tokens, seq_id, start_pos, all_logits=False):
        t = np.ascontiguousarray(tokens, dtype=np.int32)
        rows = t.size if all_logits else 1
        logits = np.empty((rows, self.cfg.vocab), dtype=np.float32)
        self._ck(self._h.vh_prefill(self._m, t.ctypes.data, t.size, seq_id, start_pos, int(all_logits),
                                    logits.ctypes.data))
        return logits if all_logits else logits[0]

    def verify_tree(self, seq_ids, input_tokens, start_pos, trees, want_logits=True):
        """One verification pass over a candidate tree per sequence (vh_verify_tree). trees: one
        (node tokens, parent indices) pair per sequence, in CandidateTree.Linearize order.
        -> ([accepted node indices per sequence], [final token per sequence], [logits (1 + nodes, vocab) per
        sequence] or None)"""
        n = len(seq_ids)
        s = np.ascontiguousarray(seq_ids, dtype=np.int64)
        t = np.ascontiguousarray(input_tokens, dtype=np.int32)
        sp = np.ascontiguousarray(start_pos, dtype=np.int32)
        nn = np.array([len(tr[0]) for tr in trees], dtype=np.int32)
        toks = np.ascontiguousarray([x for tr in trees for x in tr[0]] or [0], dtype=np.int32)
        par = np.ascontiguousarray([x for tr in trees for x in tr[1]] or [0], dtype=np.int32)
        nacc = np.zeros(n, dtype=np.int32)
        acc = np.zeros(max(1, int(nn.sum())), dtype=np.int32)
        fin = np.zeros(n, dtype=np.int32)
        rows = n + int(nn.sum())
        logits = np.empty((rows, self.cfg.vocab), dtype=np.float32) if want_logits else None
        self._ck(self._h.vh_verify_tree(self._m, n, s.ctypes.data, t.ctypes.data, sp.ctypes.data, nn.ctypes.data,
                                        toks.ctypes.data, par.ctypes.data, nacc.ctypes.data, acc.ctypes.data,
                                        fin.ctypes.data, logits.ctypes.data if want_logits else None))
        accepted, per_seq, node0, row0 = [], [], 0, 0
        for i in range(n):
            accepted.append([int(x) for x in acc[node0:node0 + nacc[i]]])
            if want_logits:
                per_seq.append(logits[row0:row0 + 1 + nn[i]])
            node0 += int(nn[i])
            row0 += 1 + int(nn[i])
        return accepted, [int(x) for x in fin], (per_seq if want_logits else None)

    def decode_graph(self, first_tokens, seq_ids, positions, steps, use_graph=True, batch=None):
        """Greedy device-driven decode. first_tokens=None continues the batch loaded on the device.
        -> (tokens [steps,B], ms_per_step of the timed steps)"""
        if first_tokens is not None:
            t = np.ascontiguousarray(first_tokens, dtype=np.int32)
            s = np.ascontiguousarray(seq_ids, dtype=np.int64)
            p = np.ascontiguousarray(positions, dtype=np.int32)
            b = t.size
            args = (t.ctypes.data, s.ctypes.data, p.ctypes.data)
        else:
            b = batch
            args = (None, None, None)
        out = np.empty((steps, b), dtype=np.int32)
        ms = C.c_float()
        self._ck(self._h.vh_decode_graph(self._m, *args, b, steps, int(bool(use_graph)), out.ctypes.data,
                                         C.byref(ms)))
        return out, ms.value
