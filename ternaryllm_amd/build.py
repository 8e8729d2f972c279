"""Builds libternary_spmm.so (host packers + gfx950 kernels) in-tree with hipcc."""
import os
import shutil
import subprocess

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG_DIR)
LIB_PATH = os.path.join(PKG_DIR, "libternary_spmm.so")
SOURCES = ["tl_pack.cpp", "tl_layout.cpp", "tl_kernels.hip", "tl_small_m.hip", "tl_rows.hip", "tl_decode.hip"]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the gfx950 library cannot be built on this machine")
    return exe


def build_library(verbose=True):
    """Compiles every translation unit for gfx950 and links the shared library. Always recompiles."""
    csrc = os.path.join(PKG_DIR, "csrc")
    cmd = [
        hipcc(), "-shared", "-fPIC", "-O3", "-std=c++17", "--offload-arch=gfx950",
        # packed-fp32 VALU forms are kept out of the generated code
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
        "-Wall", "-Wno-unused-command-line-argument",
        "-I", os.path.join(ROOT, "include"), "-I", csrc,
        "-x", "hip",
    ] + [os.path.join(csrc, s) for s in SOURCES] + ["-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB_PATH


if __name__ == "__main__":
    build_library()
