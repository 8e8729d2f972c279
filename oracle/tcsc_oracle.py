"""ctypes front end of the C oracle (tcsc_oracle.c) -- test infrastructure only.

Every wrapper takes and returns numpy arrays.  The C library is built by
``make -C oracle liboracle.so`` (``__graft_entry__.build()`` does it); loading fails
loudly when it is missing.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build(force=False):
    """Compile liboracle.so (and the CPU baselines) with the Makefile next to this file."""
    target = os.path.join(_HERE, "liboracle.so")
    if force or not os.path.exists(target):
        subprocess.check_call(["make", "-C", _HERE, "liboracle.so", "libcpu_port.so"])
    return target


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            raise RuntimeError("oracle/liboracle.so is not built: run `make -C oracle`")
        _LIB = ctypes.CDLL(path)
        _LIB.orc_tiled_mcsc_len.restype = ctypes.c_int64
    return _LIB


def _p(a, ct):
    return a.ctypes.data_as(ctypes.POINTER(ct))


def _w32(w):
    w = np.ascontiguousarray(w, dtype=np.int32)
    assert w.ndim == 2
    return w


def count_nnz(w):
    return int((w == 1).sum()), int((w == -1).sum())


def csc(w):
    """(neg_row, neg_off, pos_row, pos_off) as the reference's convert_to_ter_csc returns them."""
    w = _w32(w)
    K, N = w.shape
    cp, cn = count_nnz(w)
    neg_row = np.zeros(cn, np.int32)
    pos_row = np.zeros(cp, np.int32)
    neg_off = np.zeros(N + 1, np.int32)
    pos_off = np.zeros(N + 1, np.int32)
    rc = lib().orc_csc(_p(w, ctypes.c_int32), N, K, cp, cn, _p(neg_row, ctypes.c_int32), _p(neg_off, ctypes.c_int32),
                       _p(pos_row, ctypes.c_int32), _p(pos_off, ctypes.c_int32))
    assert rc == 0, rc
    return neg_row, neg_off, pos_row, pos_off


def tiled_csc(w, tile_k):
    w = _w32(w)
    K, N = w.shape
    T = -(-K // tile_k)
    cp, cn = count_nnz(w)
    neg_row = np.zeros(cn, np.int32)
    pos_row = np.zeros(cp, np.int32)
    neg_off = np.zeros(N * T * 2, np.int32)
    pos_off = np.zeros(N * T * 2, np.int32)
    rc = lib().orc_tiled_csc(_p(w, ctypes.c_int32), N, K, cp, cn, tile_k, _p(neg_row, ctypes.c_int32),
                             _p(neg_off, ctypes.c_int32), _p(pos_row, ctypes.c_int32), _p(pos_off, ctypes.c_int32))
    assert rc == 0, rc
    return neg_row, neg_off, pos_row, pos_off


def tiled_mcsc(w, tile_k, padding=False, padding_size=4):
    """(merged_row, merged_off, col_tile_idx) as the reference's convert_to_ter_tiled_mcsc returns them."""
    w = _w32(w)
    K, N = w.shape
    T = -(-K // tile_k)
    cp, cn = count_nnz(w)
    _, neg_off, _, pos_off = tiled_csc(w, tile_k)
    n = lib().orc_tiled_mcsc_len(_p(neg_off, ctypes.c_int32), _p(pos_off, ctypes.c_int32), N, T, cp, cn,
                                 int(bool(padding)), int(padding_size))
    merged_row = np.zeros(n, np.int32)
    merged_off = np.zeros(N * T * 4, np.int32)
    tile_idx = np.zeros(N * T, np.int32)
    rc = lib().orc_tiled_mcsc(_p(w, ctypes.c_int32), N, K, cp, cn, tile_k, int(bool(padding)), int(padding_size),
                              _p(merged_row, ctypes.c_int32), ctypes.c_int64(n), _p(merged_off, ctypes.c_int32),
                              _p(tile_idx, ctypes.c_int32))
    assert rc == 0, rc
    return merged_row, merged_off, tile_idx


def dense_product(x, w):
    """Exact ternary product in float64: x [M, K] (any float dtype) times w [K, N] in {-1, 0, 1}."""
    x = np.ascontiguousarray(x, dtype=np.float64)
    w = _w32(w)
    M, K = x.shape
    assert w.shape[0] == K
    N = w.shape[1]
    y = np.zeros((M, N), np.float64)
    lib().orc_dense_product(_p(x, ctypes.c_double), _p(w, ctypes.c_int32), _p(y, ctypes.c_double), M, N, K)
    return y


def mcsc_product(x, merged_row, merged_off, N, tile_k, uniformed=False):
    """What the reference kernels add up when they walk merged arrays (ter_spmm_kernel.cuh:197-300)."""
    x = np.ascontiguousarray(x, dtype=np.float64)
    M, K = x.shape
    merged_row = np.ascontiguousarray(merged_row, dtype=np.int32)
    merged_off = np.ascontiguousarray(merged_off, dtype=np.int32)
    y = np.zeros((M, N), np.float64)
    lib().orc_mcsc_product(_p(x, ctypes.c_double), _p(merged_row, ctypes.c_int32), _p(merged_off, ctypes.c_int32),
                           _p(y, ctypes.c_double), M, N, K, tile_k, int(bool(uniformed)))
    return y


def fast_product(x, w):
    """float64 matmul through numpy/BLAS: the same exact product, for sizes where the C triple loop is slow.
    Tests check it against dense_product on small inputs before relying on it."""
    return np.asarray(x, dtype=np.float64) @ np.asarray(w, dtype=np.float64)
