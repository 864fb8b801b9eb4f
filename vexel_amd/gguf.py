"""GGUF checkpoint reader: Python handle on the C++ reader in libvexel_host.so (vh_gguf_*), which restates
inference/pkg/gguf/gguf.go. Nothing is parsed in Python."""
import ctypes as C
import os

from .backend import VexelError
from .runtime import load_host


class VhGGUFTensor(C.Structure):
    _fields_ = [("name", C.c_char_p), ("n_dims", C.c_int), ("dims", C.c_uint64 * 4), ("type", C.c_uint32),
                ("offset", C.c_uint64), ("n_bytes", C.c_uint64), ("data", C.c_void_p)]


class VhGGUFConfig(C.Structure):
    _fields_ = [("architecture", C.c_char * 64)] + \
               [(n, C.c_int) for n in ("num_layers", "hidden", "num_heads", "num_kv_heads", "ffn", "context_length",
                                        "vocab", "rope_dim_count", "head_dim")] + \
               [("rope_theta", C.c_float), ("rms_eps", C.c_float), ("attn_softcap", C.c_float),
                ("final_softcap", C.c_float)]


def _bind(h):
    if getattr(h, "_gguf_bound", False):
        return h
    h.vh_gguf_open.argtypes = [C.c_char_p, C.POINTER(C.c_void_p)]
    h.vh_gguf_close.argtypes = [C.c_void_p]
    h.vh_gguf_close.restype = None
    h.vh_gguf_version.argtypes = [C.c_void_p]
    h.vh_gguf_version.restype = C.c_uint32
    h.vh_gguf_data_offset.argtypes = [C.c_void_p]
    h.vh_gguf_data_offset.restype = C.c_int64
    h.vh_gguf_num_tensors.argtypes = [C.c_void_p]
    h.vh_gguf_num_metadata.argtypes = [C.c_void_p]
    h.vh_gguf_tensor_at.argtypes = [C.c_void_p, C.c_int, C.POINTER(VhGGUFTensor)]
    h.vh_gguf_find_tensor.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(VhGGUFTensor)]
    h.vh_gguf_metadata_key.argtypes = [C.c_void_p, C.c_int]
    h.vh_gguf_metadata_key.restype = C.c_char_p
    h.vh_gguf_meta_type.argtypes = [C.c_void_p, C.c_char_p]
    h.vh_gguf_meta_u32.argtypes = [C.c_void_p, C.c_char_p]
    h.vh_gguf_meta_u32.restype = C.c_uint32
    h.vh_gguf_meta_u64.argtypes = [C.c_void_p, C.c_char_p]
    h.vh_gguf_meta_u64.restype = C.c_uint64
    h.vh_gguf_meta_f32.argtypes = [C.c_void_p, C.c_char_p]
    h.vh_gguf_meta_f32.restype = C.c_float
    h.vh_gguf_meta_str.argtypes = [C.c_void_p, C.c_char_p]
    h.vh_gguf_meta_str.restype = C.c_char_p
    h.vh_gguf_meta_array_len.argtypes = [C.c_void_p, C.c_char_p]
    h.vh_gguf_meta_array_len.restype = C.c_int64
    h.vh_gguf_get_config.argtypes = [C.c_void_p, C.POINTER(VhGGUFConfig)]
    h.vh_gguf_tensor_name.argtypes = [C.c_char_p, C.c_char_p, C.c_size_t]
    h._gguf_bound = True
    return h


class GGUFFile:
    """gguf.File: open(path) parses header, metadata and the tensor table; tensor bytes are read from the mapping."""

    def __init__(self, path):
        self._h = _bind(load_host())
        g = C.c_void_p()
        if self._h.vh_gguf_open(os.fsencode(path), C.byref(g)) != 0:
            raise VexelError(1, self._h.vh_last_error().decode())
        self._g = g

    def close(self):
        if self._g:
            self._h.vh_gguf_close(self._g)
            self._g = None

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    @property
    def version(self):
        return self._h.vh_gguf_version(self._g)

    @property
    def data_offset(self):
        return self._h.vh_gguf_data_offset(self._g)

    def _tensor(self, t):
        return dict(name=t.name.decode(), dims=[int(t.dims[i]) for i in range(t.n_dims)], type=int(t.type),
                    offset=int(t.offset), n_bytes=int(t.n_bytes),
                    data=C.string_at(t.data, t.n_bytes) if t.data else None)

    def tensors(self):
        out = []
        for i in range(self._h.vh_gguf_num_tensors(self._g)):
            t = VhGGUFTensor()
            self._h.vh_gguf_tensor_at(self._g, i, C.byref(t))
            out.append(self._tensor(t))
        return out

    def get_tensor(self, name):
        t = VhGGUFTensor()
        if self._h.vh_gguf_find_tensor(self._g, name.encode(), C.byref(t)) != 0:
            return None
        return self._tensor(t)

    def metadata_keys(self):
        return [self._h.vh_gguf_metadata_key(self._g, i).decode() for i in range(self._h.vh_gguf_num_metadata(self._g))]

    def meta_type(self, key):
        return self._h.vh_gguf_meta_type(self._g, key.encode())

    def meta_u32(self, key):
        return self._h.vh_gguf_meta_u32(self._g, key.encode())

    def meta_u64(self, key):
        return self._h.vh_gguf_meta_u64(self._g, key.encode())

    def meta_f32(self, key):
        return self._h.vh_gguf_meta_f32(self._g, key.encode())

    def meta_str(self, key):
        s = self._h.vh_gguf_meta_str(self._g, key.encode())
        return None if s is None else s.decode()

    def meta_array_len(self, key):
        return self._h.vh_gguf_meta_array_len(self._g, key.encode())

    def config(self):
        c = VhGGUFConfig()
        self._h.vh_gguf_get_config(self._g, C.byref(c))
        d = {n: getattr(c, n) for n, _ in VhGGUFConfig._fields_}
        d["architecture"] = c.architecture.decode()
        return d


def layer_tensor_name(hf_name):
    """gguf.GetLayerTensorName."""
    h = _bind(load_host())
    buf = C.create_string_buffer(256)
    if h.vh_gguf_tensor_name(hf_name.encode(), buf, 256) != 0:
        raise VexelError(1, h.vh_last_error().decode())
    return buf.value.decode()
