"""Builds libvexel_hip.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree."""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libvexel_hip.so")
HOST_LIB = os.path.join(HERE, "libvexel_host.so")
SYNTH_LIB = os.path.join(HERE, "libvexel_synth.so")
OBJ_DIR = os.path.join(HERE, "build")

SOURCES = ["backend.hip", "elementwise.hip", "attention.hip", "qgemm.hip", "qstream.hip", "qmatvec.hip", "pack.hip", "sampler.hip", "medusa.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["-O3", "--offload-arch=gfx950", "-fPIC", "-std=c++17", "-fvisibility=default",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         # float32 operations round one by one, as the reference's Go on amd64 does (cpu.go never fuses a multiply
         # with an add); where a fused multiply-add is meant the kernels call fmaf themselves
         "-ffp-contract=off",
         "-Wall", "-Wno-unused-function",
         "-I" + os.path.join(ROOT, "include"), "-I" + CSRC]


def _compile(src):
    obj = os.path.join(OBJ_DIR, src.replace(".hip", ".o"))
    cmd = [HIPCC] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose=True):
    """Compiles every source and links the shared library. Always rebuilds."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(_compile, SOURCES))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    if verbose:
        print("built", LIB)
    # benchmark support (synthetic weights / KV made on the device); not part of the C ABI
    cmd = [HIPCC] + FLAGS + ["-shared", os.path.join(CSRC, "synth.hip"), "-o", SYNTH_LIB]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("synth build failed:\n" + r.stderr)
    if verbose:
        print("built", SYNTH_LIB)
    # host runtime: plain C++ above the C ABI (links the HIP library, finds it next to itself)
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-I" + os.path.join(ROOT, "include"),
           os.path.join(HERE, "host", "runtime.cpp"), os.path.join(HERE, "host", "gguf.cpp"),
           os.path.join(HERE, "host", "scheduler.cpp"), "-o", HOST_LIB, "-L" + HERE, "-lvexel_hip",
           "-Wl,-rpath,$ORIGIN", "-pthread"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("host runtime build failed:\n" + r.stderr)
    if r.stderr.strip():
        sys.stderr.write(r.stderr)
    if verbose:
        print("built", HOST_LIB)
    return LIB


if __name__ == "__main__":
    build()
