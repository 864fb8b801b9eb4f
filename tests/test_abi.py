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
