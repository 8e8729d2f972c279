"""CPU baselines for bench.py's `cpu_baseline` leg -- test / measurement infrastructure only.

Two providers with one interface:
  * "reference": the reference's own AVX2 / AVX-512 GEMM kernels
    (ternaryLLM_CPU/src/GEMM_CPU_FP32.cpp:2956 and :8365), compiled in place from the reference
    checkout into oracle/_ref/libref_cpu.so by oracle/Makefile, behind oracle/ref_cpu_shim.cpp;
  * "port": this repository's restatement of the same kernels (oracle/cpu_port.cpp).
The reference build uses AVX-512 in every function, so it is only offered on hosts with avx512f/bw/vl/dq.

Timing follows the plan the reference's driver implies (ternaryLLM_CPU/src/main.cpp:1014,1069-1099: 10 runs)
with the threads held still: one OpenMP thread per PHYSICAL core of the process's CPU set, bound
(OMP_PROC_BIND=close, OMP_PLACES=cores).  The OpenMP runtime reads those variables once, when it starts, and
a process that has imported torch has started it long before: the timed kernels therefore run in a child
process (`python -m oracle.cpu_baseline ...`) whose environment is set before anything loads OpenMP.
"""
import ctypes
import json
import os
import subprocess
import sys
import tempfile
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
    """The `model name` of /proc/cpuinfo with what identifies the part where that name is generic (a virtual machine
    may report a bare family name): vendor, family, model and stepping numbers."""
    want = {"vendor_id": None, "model name": None, "cpu family": None, "model": None, "stepping": None}
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                key, _, value = line.partition(":")
                key = key.strip()
                if key in want and want[key] is None:
                    want[key] = value.strip()
                if all(v is not None for v in want.values()):
                    break
    except OSError:
        pass
    if want["model name"] is None:
        return "unknown"
    ids = ", ".join("%s %s" % (label, want[key]) for label, key in (("family", "cpu family"), ("model", "model"), ("stepping", "stepping"))
                    if want[key] is not None)
    return "%s (%s%s)" % (want["model name"], (want["vendor_id"] + ", ") if want["vendor_id"] else "", ids)


def physical_cores():
    """Distinct (package, core) pairs among the CPUs this process may run on; the logical CPU count of that set
    when /proc/cpuinfo does not say."""
    try:
        allowed = os.sched_getaffinity(0)
    except AttributeError:
        allowed = set(range(os.cpu_count() or 1))
    cores, cpu, pkg = set(), None, 0
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                key, _, val = line.partition(":")
                key = key.strip()
                if key == "processor":
                    cpu = int(val)
                elif key == "physical id":
                    pkg = int(val)
                elif key == "core id" and cpu in allowed:
                    cores.add((pkg, int(val)))
    except (OSError, ValueError):
        cores = set()
    return len(cores) if cores else len(allowed)


def threads():
    """Threads of a timed run: one per physical core, no more than OMP_NUM_THREADS when the host sets it."""
    n = physical_cores()
    cap = os.environ.get("OMP_NUM_THREADS")
    if cap and cap.isdigit() and int(cap) > 0:
        n = min(n, int(cap))
    return max(1, n)


def _aligned(shape, dtype=np.float32, align=64):
    n = int(np.prod(shape))
    raw = np.zeros(n * np.dtype(dtype).itemsize + align, np.uint8)
    off = (-raw.ctypes.data) % align
    return raw[off:off + n * np.dtype(dtype).itemsize].view(dtype).reshape(shape)


class ReferenceProvider:
    """The reference's own kernels; `which` is "avx2" (32 rows x 8 columns, the reference's headline choice
    "MergedMin_32G8_AVX2", main.cpp:1018,1088) or "avx512" (32 x 16, GEMM_CPU_FP32.cpp:8365)."""
    kind = "reference"

    def __init__(self, which="avx2"):
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
        self.group = 8 if which == "avx2" else 16
        self.fn = L.ref_gemm_32xg8_avx2 if which == "avx2" else L.ref_gemm_32xg16_avx512
        self.kernel_name = ("GEMM_CPU_FP32_colMajor_TCSC_Merged_GroupMin_32xG8_AVX2_OpenMP" if which == "avx2"
                            else "GEMM_CPU_FP32_colMajor_TCSC_Merged_GroupMin_32xG16_AVX512_OpenMP")

    def build(self, w_i8, K, N):
        return self.L.ref_group_build(w_i8.ctypes.data, K, N, self.group)

    def free(self, h):
        self.L.ref_group_free(h)

    def run(self, h, x_km, y_nm, M, N, K):
        self.fn(x_km.ctypes.data, h, y_nm.ctypes.data, M, N, K)


class PortProvider:
    kind = "port"
    group = 8

    def __init__(self):
        path = os.path.join(_HERE, "libcpu_port.so")
        if not os.path.exists(path):
            raise RuntimeError("oracle/libcpu_port.so is not built")
        L = ctypes.CDLL(path)
        L.port_group_build.restype = ctypes.c_void_p
        L.port_group_build.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        L.port_group_free.argtypes = [ctypes.c_void_p]
        L.port_gemm_32xg8_avx2.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        for fn in (L.port_gemv_g64_avx2, L.port_gemv_g64_avx512):
            fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int]
        self.L = L
        self.kernel_name = "port of GEMM_CPU_FP32_colMajor_TCSC_Merged_GroupMin_32xG8_AVX2_OpenMP"

    def build(self, w_i8, K, N):
        return self.L.port_group_build(w_i8.ctypes.data, K, N, 8, 1)

    def free(self, h):
        self.L.port_group_free(h)

    def run(self, h, x_km, y_nm, M, N, K):
        self.L.port_gemm_32xg8_avx2(x_km.ctypes.data, h, y_nm.ctypes.data, M, N, K)

    def gemv(self, w_i8, x, N, K, wide=False):
        h = self.L.port_group_build(w_i8.ctypes.data, K, N, 64, 0)
        y = np.zeros(N, np.float32)
        (self.L.port_gemv_g64_avx512 if wide else self.L.port_gemv_g64_avx2)(np.ascontiguousarray(x, np.float32).ctypes.data, h, y.ctypes.data, N, K)
        self.L.port_group_free(h)
        return y


def _stats(samples):
    s = sorted(samples)
    return {"min": s[0], "median": s[len(s) // 2], "mean": sum(s) / len(s), "max": s[-1]}


def _gemm_providers(prefer_reference):
    out = []
    if prefer_reference:
        for which in ("avx2", "avx512"):
            try:
                out.append(ReferenceProvider(which))
            except (RuntimeError, OSError):
                pass
    if not out:
        out.append(PortProvider())
    return out


def _time_gemm_here(w, x, runs, prefer_reference, check):
    """Runs in the process whose OpenMP environment is already what it should be."""
    K, N = w.shape
    M = x.shape[0]
    assert M % 32 == 0 and N % 16 == 0 and K < 32768
    w8 = np.ascontiguousarray(w, dtype=np.int8)
    x_km = _aligned((K, M))
    x_km[:] = np.asarray(x, np.float32).T
    y_nm = _aligned((N, M))
    results = []
    for p in _gemm_providers(prefer_reference):
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
        samples = []
        for _ in range(runs):
            t0 = time.perf_counter()
            p.run(h, x_km, y_nm, M, N, K)
            samples.append(time.perf_counter() - t0)
        p.free(h)
        st = _stats(samples)
        results.append({"seconds": st["mean"], "seconds_min": st["min"], "seconds_median": st["median"], "seconds_max": st["max"],
                        "runs": runs, "kind": p.kind, "kernel": p.kernel_name, "group": p.group, "max_rel_err": max_err})
    return results


def _time_gemv_here(w, x, runs):
    p = PortProvider()
    K, N = w.shape
    assert N % 64 == 0 and K < 32768
    w8 = np.ascontiguousarray(w, dtype=np.int8)
    xv = np.ascontiguousarray(x, np.float32)
    ref = xv.astype(np.float64) @ w.astype(np.float64)
    h = p.L.port_group_build(w8.ctypes.data, K, N, 64, 0)
    results = []
    kernels = [("port of GEMV_CPU_FP32_rowMajor_TCSC_Merged_GroupMin_G64_AVX2_OpenMP", p.L.port_gemv_g64_avx2)]
    if "avx512f" in _cpu_flags():
        kernels.append(("port of GEMV_CPU_FP32_rowMajor_TCSC_Merged_GroupMin_G64_AVX512_OpenMP", p.L.port_gemv_g64_avx512))
    for name, fn in kernels:
        y = np.zeros(N, np.float32)
        fn(xv.ctypes.data, h, y.ctypes.data, N, K)
        max_err = float(np.max(np.abs(y - ref)) / max(1e-9, np.abs(ref).max()))
        if max_err > 1e-4:
            p.L.port_group_free(h)
            raise RuntimeError(f"CPU GEMV port disagrees with the exact product (max err / max {max_err})")
        for _ in range(10):  # (the team's threads up and spinning, the operands in the caches they will stay in)
            fn(xv.ctypes.data, h, y.ctypes.data, N, K)
        samples = []
        for _ in range(runs):
            t0 = time.perf_counter()
            fn(xv.ctypes.data, h, y.ctypes.data, N, K)
            samples.append(time.perf_counter() - t0)
        st = _stats(samples)
        results.append({"seconds": st["mean"], "seconds_min": st["min"], "seconds_median": st["median"], "seconds_max": st["max"],
                        "runs": runs, "kind": "port", "kernel": name, "max_err_over_max": max_err})
    p.L.port_group_free(h)
    return results


def _in_child(mode, w, x, runs, prefer_reference=True, check=True):
    """Writes the operands where a child process finds them, runs `python -m oracle.cpu_baseline` there with the
    OpenMP variables set, and returns what it printed."""
    n = threads()
    env = dict(os.environ, OMP_NUM_THREADS=str(n), OMP_PROC_BIND="close", OMP_PLACES="cores", OMP_DYNAMIC="false")
    with tempfile.TemporaryDirectory(prefix="tl_cpu_baseline_") as tmp:
        path = os.path.join(tmp, "operands.npz")
        np.savez(path, w=np.ascontiguousarray(w, dtype=np.int8), x=np.asarray(x, np.float32))
        cmd = [sys.executable, "-m", "oracle.cpu_baseline", mode, path, str(runs), "1" if prefer_reference else "0", "1" if check else "0"]
        done = subprocess.run(cmd, cwd=os.path.dirname(_HERE), env=env, capture_output=True, text=True, timeout=600)
    if done.returncode != 0:
        raise RuntimeError("CPU baseline child failed: " + (done.stderr.strip().splitlines() or ["?"])[-1])
    results = json.loads(done.stdout.strip().splitlines()[-1])
    for r in results:
        r.update({"threads": n, "cpu": cpu_model(), "binding": "OMP_PROC_BIND=close OMP_PLACES=cores, one thread per physical core"})
    return results


def time_gemm_all(w, x, runs=10, prefer_reference=True, check=True):
    """Times Y = X @ W on the CPU with the reference's GEMM kernels, every one this host can run: the AVX2
    32 x 8 kernel (the reference's own headline choice) first, its AVX-512 32 x 16 sibling second; this
    repository's port of the first where the reference build is absent.

    w: int [K, N] ternary, x: float [M, K] (M % 32 == 0, N % 16 == 0).  Operands are converted to the kernels'
    layouts (X as [K][M], result [N][M], 64-byte aligned), the result is checked against the float64 product,
    then each kernel is called `runs` times; `seconds` is the mean (the reference driver's statistic), minimum,
    median and maximum beside it."""
    return _in_child("gemm", w, x, runs, prefer_reference, check)


def time_gemm(w, x, runs=10, prefer_reference=True, check=True):
    """The first entry of time_gemm_all: the reference's headline kernel."""
    return time_gemm_all(w, x, runs, prefer_reference, check)[0]


def time_gemv_all(w, x, runs=20):
    """Times y = x @ W (one row) on the CPU with this repository's ports of the reference's decode kernels
    GEMV_CPU_FP32_rowMajor_TCSC_Merged_GroupMin_G64_AVX2_OpenMP (ternaryLLM_CPU/src/GEMM_CPU_FP32.cpp:15008-15081)
    and ..._G64_AVX512_OpenMP (:15684-15729); the reference's own file holds them behind aligned loads that fault
    under GCC, so the ports are what runs.  w: int [K, N] ternary (N % 64 == 0), x: float [K].  Checked against
    the float64 product first."""
    return _in_child("gemv", w, np.asarray(x, np.float32)[None, :], runs)


def time_gemv(w, x, runs=20):
    return time_gemv_all(w, x, runs)[0]


if __name__ == "__main__":
    mode, path, runs = sys.argv[1], sys.argv[2], int(sys.argv[3])
    with np.load(path) as z:
        w_, x_ = z["w"].astype(np.int32), z["x"]
    if mode == "gemm":
        res = _time_gemm_here(w_, x_, runs, sys.argv[4] == "1", sys.argv[5] == "1")
    else:
        res = _time_gemv_here(w_, x_[0], runs)
    print(json.dumps(res))
