"""CPU-side checks of the drop-in boundary: the shared library loads, exports every symbol
include/vexel_hip.h declares, and the Python binding table names exactly those symbols.
No compute call is made (there is no GPU here)."""
import ctypes
import os
import re

from vexel_amd import lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "vexel_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return set(re.findall(r"\b(vx_[a-z0-9_]+)\s*\(", text))


def test_header_and_binding_agree():
    assert _declared() == set(lib.SIGNATURES)


def test_library_exports_every_declared_symbol():
    assert os.path.exists(lib.LIB_PATH), "build the library first: python -m vexel_amd.build"
    dll = ctypes.CDLL(lib.LIB_PATH)
    for name in sorted(_declared()):
        assert hasattr(dll, name), "missing export " + name
    lib.load()


def test_host_library_exports_every_declared_symbol():
    """include/vexel_host.h against libvexel_host.so (the host runtime above the C ABI)."""
    text = open(os.path.join(ROOT, "include", "vexel_host.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = set(re.findall(r"\b(vh_[a-z0-9_]+)\s*\(", text))
    assert len(names) > 40
    path = os.path.join(ROOT, "vexel_amd", "libvexel_host.so")
    assert os.path.exists(path), "build the library first: python -m vexel_amd.build"
    dll = ctypes.CDLL(path)
    for name in sorted(names):
        assert hasattr(dll, name), "missing export " + name


def test_error_text_is_available_without_a_gpu():
    l = lib.load()
    assert isinstance(l.vx_last_error(), bytes)
    # a call without a backend is refused before anything touches the device
    assert l.vx_matmul_q5_k(None, None, None, None, 1, 32, 32) == lib.VX_ERR_INVALID
    assert b"null backend" in l.vx_last_error()


def test_every_entry_point_cites_the_reference():
    text = open(os.path.join(ROOT, "include", "vexel_hip.h")).read()
    assert text.count("backend.go") >= 10 and "gpu_block_pool.go" in text


def test_geometry_queries_answer_without_a_gpu():
    """The capability queries are plain functions of the head geometry: which shapes the streaming decode attention
    takes (and leaves split for the fused tail), and how many rows of a candidate tree share one pass over the
    context (16 queries per K/V row: 16 / G rows, whole)."""
    dll = lib.load()
    split = dll.vx_sdpa_paged_decode_split_supported
    rows = dll.vx_sdpa_paged_tree_rows_per_entry
    # (pool is f16, block size, query heads, kv heads, head size)
    assert split(1, 16, 32, 32, 128) == 1 and split(1, 16, 32, 8, 128) == 1 and split(1, 16, 28, 4, 128) == 1
    assert split(1, 16, 32, 2, 128) == 1 and split(1, 16, 24, 2, 128) == 1      # 16 and 12 query heads per kv head
    assert split(1, 16, 36, 4, 128) == 0 and split(1, 16, 32, 2, 64) == 0        # 9 per kv head; 16 at heads of 64
    assert split(1, 16, 8, 4, 256) == 1 and split(1, 16, 12, 4, 256) == 0 and split(1, 16, 32, 32, 80) == 1
    assert split(0, 16, 32, 32, 128) == 0 and split(1, 32, 32, 32, 128) == 0    # float32 pool; 32-token blocks
    assert [rows(1, 16, g * 2, 2, 128) for g in range(1, 9)] == [16, 8, 5, 4, 3, 2, 2, 2]
    assert rows(1, 16, 18, 2, 128) == 0 and rows(1, 16, 8, 4, 256) == 0 and rows(0, 16, 8, 8, 128) == 0
    assert rows(1, 16, 8, 2, 64) == 4 and rows(1, 8, 8, 8, 128) == 0
