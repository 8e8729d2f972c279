"""CPU baselines for bench.py's `cpu_baseline` leg -- test / measurement infrastructure only.

Two providers with one interface:
  * "reference": the reference's own AVX2 / AVX-512 GEMM kernels
    (ternaryLLM_CPU/src/GEMM_CPU_FP32.cpp:2956 and :8365), compiled in place from the reference
    checkout into oracle/_ref/libref_cpu.so by oracle/Makefile, behind oracle/ref_cpu_shim.cpp;
  * "port": this repository's restatement of the same kernels (oracle/cpu_port.cpp).
The reference build uses AVX-512 in every function, so it is only offered on hosts with avx512f/bw/vl/dq.
"""
import ctypes
import os
import time

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))


def _cpu_flags():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("flags"):
                    return set(line.split(":", 1)[1].split())
    except OSError:
        pass
    return set()


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def _aligned(shape, dtype=np.float32, align=64):
    n = int(np.prod(shape))
    raw = np.zeros(n * np.dtype(dtype).itemsize + align, np.uint8)
    off = (-raw.ctypes.data) % align
    return raw[off:off + n * np.dtype(dtype).itemsize].view(dtype).reshape(shape)


class _Provider:
    kind = None

    def gemm(self, x_km, w_i8, M, N, K):
        raise NotImplementedError


class ReferenceProvider(_Provider):
    kind = "reference"

    def __init__(self):
        path = os.path.join(_HERE, "_ref", "libref_cpu.so")
        need = {"avx2", "fma", "avx512f", "avx512bw", "avx512vl", "avx512dq"}
        if not os.path.exists(path):
            raise RuntimeError("oracle/_ref/libref_cpu.so is not built")
        if not need <= _cpu_flags():
            raise RuntimeError("host lacks the AVX-512 subsets the reference build was compiled for")
        L = ctypes.CDLL(path)
        L.ref_group_build.restype = ctypes.c_void_p
        L.ref_group_build.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        L.ref_group_free.argtypes = [ctypes.c_void_p]
        for fn in (L.ref_gemm_32xg8_avx2, L.ref_gemm_32xg16_avx512):
            fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        self.L = L
        self.kernel_name = "GEMM_CPU_FP32_colMajor_TCSC_Merged_GroupMin_32xG16_AVX512_OpenMP"

    def build(self, w_i8, K, N):
        return self.L.ref_group_build(w_i8.ctypes.data, K, N, 16)

    def free(self, h):
        self.L.ref_group_free(h)

    def run(self, h, x_km, y_nm, M, N, K):
        self.L.ref_gemm_32xg16_avx512(x_km.ctypes.data, h, y_nm.ctypes.data, M, N, K)


class PortProvider(_Provider):
    kind = "port"

    def __init__(self):
        path = os.path.join(_HERE, "libcpu_port.so")
        if not os.path.exists(path):
            raise RuntimeError("oracle/libcpu_port.so is not built")
        L = ctypes.CDLL(path)
        L.port_group_build.restype = ctypes.c_void_p
        L.port_group_build.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        L.port_group_free.argtypes = [ctypes.c_void_p]
        L.port_gemm_32xg8_avx2.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        L.port_gemv_g64_avx2.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int]
        self.L = L
        self.kernel_name = "port of GEMM_CPU_FP32_colMajor_TCSC_Merged_GroupMin_32xG8_AVX2_OpenMP"

    def build(self, w_i8, K, N):
        return self.L.port_group_build(w_i8.ctypes.data, K, N, 8, 1)

    def free(self, h):
        self.L.port_group_free(h)

    def run(self, h, x_km, y_nm, M, N, K):
        self.L.port_gemm_32xg8_avx2(x_km.ctypes.data, h, y_nm.ctypes.data, M, N, K)

    def gemv(self, w_i8, x, N, K):
        h = self.L.port_group_build(w_i8.ctypes.data, K, N, 64, 0)
        y = np.zeros(N, np.float32)
        self.L.port_gemv_g64_avx2(np.ascontiguousarray(x, np.float32).ctypes.data, h, y.ctypes.data, N, K)
        self.L.port_group_free(h)
        return y


def provider(prefer_reference=True):
    if prefer_reference:
        try:
            return ReferenceProvider()
        except (RuntimeError, OSError):
            pass
    return PortProvider()


def threads():
    return int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))


def time_gemm(w, x, runs=10, prefer_reference=True, check=True):
    """Times Y = X @ W on the CPU with the reference's headline kernel.

    w: int [K, N] ternary, x: float [M, K] (M % 32 == 0, N % 16 == 0).  Converts to the kernel's
    layouts (X as [K][M], result [N][M], 64-byte aligned), checks the result against the float64
    product, then reports the mean of `runs` calls, like the reference's driver
    (ternaryLLM_CPU/src/main.cpp:1014,1069-1099)."""
    p = provider(prefer_reference)
    K, N = w.shape
    M = x.shape[0]
    assert M % 32 == 0 and N % 16 == 0 and K < 32768
    w8 = np.ascontiguousarray(w, dtype=np.int8)
    x_km = _aligned((K, M))
    x_km[:] = np.asarray(x, np.float32).T
    y_nm = _aligned((N, M))
    h = p.build(w8, K, N)
    p.run(h, x_km, y_nm, M, N, K)
    max_err = None
    if check:
        ref = (np.asarray(x, np.float64) @ w.astype(np.float64)).T
        scale = np.maximum(np.abs(ref), np.linalg.norm(x, axis=1)[None, :] * np.sqrt(np.count_nonzero(w) / w.size))
        max_err = float(np.max(np.abs(y_nm - ref) / scale))
        if max_err > 1e-4:
            p.free(h)
            raise RuntimeError(f"CPU baseline kernel disagrees with the exact product (max rel err {max_err})")
    t0 = time.perf_counter()
    for _ in range(runs):
        p.run(h, x_km, y_nm, M, N, K)
    dt = (time.perf_counter() - t0) / runs
    p.free(h)
    return {"seconds": dt, "kind": p.kind, "kernel": p.kernel_name, "threads": threads(), "max_rel_err": max_err,
            "cpu": cpu_model()}


def time_gemv(w, x, runs=20):
    """Times y = x @ W (one row) on the CPU with this repository's port of the reference's decode kernel
    GEMV_CPU_FP32_rowMajor_TCSC_Merged_GroupMin_G64_AVX2_OpenMP (ternaryLLM_CPU/src/GEMM_CPU_FP32.cpp:15008-15081;
    the reference's own file holds it behind aligned loads that fault under GCC, so the port is what runs).
    w: int [K, N] ternary (N % 64 == 0), x: float [K].  Checked against the float64 product first."""
    p = PortProvider()
    K, N = w.shape
    assert N % 64 == 0 and K < 32768
    w8 = np.ascontiguousarray(w, dtype=np.int8)
    xv = np.ascontiguousarray(x, np.float32)
    y = np.zeros(N, np.float32)
    h = p.L.port_group_build(w8.ctypes.data, K, N, 64, 0)
    p.L.port_gemv_g64_avx2(xv.ctypes.data, h, y.ctypes.data, N, K)
    ref = xv.astype(np.float64) @ w.astype(np.float64)
    max_err = float(np.max(np.abs(y - ref)) / max(1e-9, np.abs(ref).max()))
    if max_err > 1e-4:
        p.L.port_group_free(h)
        raise RuntimeError(f"CPU GEMV port disagrees with the exact product (max err / max {max_err})")
    t0 = time.perf_counter()
    for _ in range(runs):
        p.L.port_gemv_g64_avx2(xv.ctypes.data, h, y.ctypes.data, N, K)
    dt = (time.perf_counter() - t0) / runs
    p.L.port_group_free(h)
    return {"seconds": dt, "kind": "port", "kernel": "port of GEMV_CPU_FP32_rowMajor_TCSC_Merged_GroupMin_G64_AVX2_OpenMP",
            "threads": threads(), "max_err_over_max": max_err, "cpu": cpu_model()}
