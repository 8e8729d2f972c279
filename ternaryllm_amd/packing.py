"""Host-side packing: reference-compatible converters and the device weight blob.

The three converters keep the reference's names, argument order and output order
(ternaryLLM_GPU/csrc/ter_spmm_wrapper.cu:39-45, :92-99, :156-165); they return int32 numpy
arrays where the reference returns Python lists of ints -- the reference's only caller wraps
them in ``np.array`` straight away (TernaryLLM/TernaryLinear.py:110-112).
"""
import ctypes

import numpy as np

from . import _lib


def count_nnz(w):
    w = _lib.as_i32_matrix(w)
    p, n = ctypes.c_int64(), ctypes.c_int64()
    _lib.check(_lib.lib().tl_count_nnz(_lib.i32p(w), w.shape[1], w.shape[0], ctypes.byref(p), ctypes.byref(n)))
    return p.value, n.value


def _check_dims(w, columns, inners):
    if w.shape != (inners, columns):
        raise ValueError(f"weight has shape {w.shape}, expected (inners={inners}, columns={columns})")


def convert_to_ter_csc(w, columns, inners, w_cnt_pos_nnz, w_cnt_neg_nnz):
    """-> [neg_row_idx, neg_col_off, pos_row_idx, pos_col_off]  (ter_spmm_wrapper.cu:39-78)."""
    w = _lib.as_i32_matrix(w)
    _check_dims(w, columns, inners)
    neg_row = np.zeros(w_cnt_neg_nnz, np.int32)
    pos_row = np.zeros(w_cnt_pos_nnz, np.int32)
    neg_off = np.zeros(columns + 1, np.int32)
    pos_off = np.zeros(columns + 1, np.int32)
    _lib.check(_lib.lib().tl_convert_to_ter_csc(_lib.i32p(w), columns, inners, w_cnt_pos_nnz, w_cnt_neg_nnz,
                                                 _lib.i32p(neg_row), _lib.i32p(neg_off), _lib.i32p(pos_row),
                                                 _lib.i32p(pos_off)))
    return [neg_row, neg_off, pos_row, pos_off]


def convert_to_ter_tiled_csc(w, columns, inners, w_cnt_pos_nnz, w_cnt_neg_nnz, TILE_K):
    """-> [neg_row_idx_local, neg_off_tiled, pos_row_idx_local, pos_off_tiled]  (ter_spmm_wrapper.cu:92-152)."""
    w = _lib.as_i32_matrix(w)
    _check_dims(w, columns, inners)
    if TILE_K <= 0:
        raise ValueError("TILE_K must be positive")
    T = -(-inners // TILE_K)
    neg_row = np.zeros(w_cnt_neg_nnz, np.int32)
    pos_row = np.zeros(w_cnt_pos_nnz, np.int32)
    neg_off = np.zeros(columns * T * 2, np.int32)
    pos_off = np.zeros(columns * T * 2, np.int32)
    _lib.check(_lib.lib().tl_convert_to_ter_tiled_csc(_lib.i32p(w), columns, inners, w_cnt_pos_nnz, w_cnt_neg_nnz, TILE_K,
                                                       _lib.i32p(neg_row), _lib.i32p(neg_off), _lib.i32p(pos_row),
                                                       _lib.i32p(pos_off)))
    return [neg_row, neg_off, pos_row, pos_off]


def convert_to_ter_tiled_mcsc(w, columns, inners, w_cnt_pos_nnz, w_cnt_neg_nnz, TILE_K, padding, padding_size):
    """-> [merged_row_idx, merged_off (4 per tile), col_tile_idx]  (ter_spmm_wrapper.cu:156-315)."""
    w = _lib.as_i32_matrix(w)
    _check_dims(w, columns, inners)
    if TILE_K <= 0:
        raise ValueError("TILE_K must be positive")
    T = -(-inners // TILE_K)
    n = ctypes.c_int64()
    L = _lib.lib()
    _lib.check(L.tl_tiled_mcsc_size(_lib.i32p(w), columns, inners, w_cnt_pos_nnz, w_cnt_neg_nnz, TILE_K, int(bool(padding)),
                                    int(padding_size), ctypes.byref(n)))
    merged_row = np.zeros(n.value, np.int32)
    merged_off = np.zeros(columns * T * 4, np.int32)
    tile_idx = np.zeros(columns * T, np.int32)
    _lib.check(L.tl_convert_to_ter_tiled_mcsc(_lib.i32p(w), columns, inners, w_cnt_pos_nnz, w_cnt_neg_nnz, TILE_K,
                                              int(bool(padding)), int(padding_size), _lib.i32p(merged_row), n.value,
                                              _lib.i32p(merged_off), _lib.i32p(tile_idx)))
    return [merged_row, merged_off, tile_idx]


def tiled_mcsc_to_dense(merged_row, merged_off, columns, inners, TILE_K):
    """The ternary matrix that merged arrays encode (what the reference kernels would multiply by)."""
    merged_row = np.ascontiguousarray(merged_row)
    if merged_row.dtype not in (np.int16, np.int32):
        raise ValueError("merged_row must be int16 or int32")
    merged_off = np.ascontiguousarray(merged_off, dtype=np.int32)
    if TILE_K <= 0 or merged_off.size != columns * (-(-inners // TILE_K)) * 4:
        raise ValueError("merged_off must hold columns * ceil(inners / TILE_K) * 4 entries")
    w = np.zeros((inners, columns), np.int32)
    _lib.check(_lib.lib().tl_tiled_mcsc_to_dense(merged_row.ctypes.data, merged_row.dtype.itemsize, merged_row.size,
                                                  _lib.i32p(merged_off), columns, inners, TILE_K, _lib.i32p(w)))
    return w


class PackedWeight:
    """Device weight blob ("wave-tiled CSC") as host bytes plus its parsed header."""

    def __init__(self, blob):
        self.blob = np.ascontiguousarray(blob, dtype=np.uint8)
        if self.blob.size < 256:
            raise ValueError("blob shorter than its header")
        self.header = _lib.LayoutHeader.from_buffer_copy(self.blob[:256].tobytes())
        if self.header.magic != _lib.TL_LAYOUT_MAGIC:
            raise ValueError("not a packed ternary weight (bad magic)")
        if self.header.total_bytes > self.blob.size:
            raise ValueError("blob is truncated")
        self.blob = self.blob[: self.header.total_bytes]

    @property
    def inners(self):
        return self.header.inners

    @property
    def columns(self):
        return self.header.columns

    @property
    def nnz(self):
        return self.header.nnz_pos + self.header.nnz_neg

    @classmethod
    def from_dense(cls, w, tile_rows=0):
        """w: int32 [K, N] with values in {-1, 0, 1} (numpy or CPU torch)."""
        w = _lib.as_i32_matrix(w)
        K, N = w.shape
        size = ctypes.c_int64(0)
        L = _lib.lib()
        _lib.check(L.tl_layout_from_dense(_lib.i32p(w), N, K, tile_rows, None, ctypes.byref(size)))
        blob = np.zeros(size.value, np.uint8)
        _lib.check(L.tl_layout_from_dense(_lib.i32p(w), N, K, tile_rows, blob.ctypes.data, ctypes.byref(size)))
        return cls(blob)

    @classmethod
    def from_tiled_csc(cls, neg_row, neg_off_tiled, pos_row, pos_off_tiled, columns, inners, TILE_K, tile_rows=0):
        """From the four arrays convert_to_ter_tiled_csc returns (same order)."""
        arrs = [np.ascontiguousarray(a, dtype=np.int32) for a in (neg_row, neg_off_tiled, pos_row, pos_off_tiled)]
        T = -(-inners // TILE_K)
        if arrs[1].size != columns * T * 2 or arrs[3].size != columns * T * 2:
            raise ValueError("offset arrays must hold columns * ceil(inners / TILE_K) * 2 entries")
        if arrs[0].size < arrs[1][-1] or arrs[2].size < arrs[3][-1]:
            raise ValueError("row arrays are shorter than the offsets say")
        size = ctypes.c_int64(0)
        L = _lib.lib()
        _lib.check(L.tl_layout_size(_lib.i32p(arrs[1]), _lib.i32p(arrs[3]), columns, inners, TILE_K, tile_rows, ctypes.byref(size)))
        blob = np.zeros(size.value, np.uint8)
        _lib.check(L.tl_layout_build(_lib.i32p(arrs[0]), _lib.i32p(arrs[1]), _lib.i32p(arrs[2]), _lib.i32p(arrs[3]), columns,
                                     inners, TILE_K, tile_rows, blob.ctypes.data, size.value))
        return cls(blob)

    @classmethod
    def from_mcsc(cls, merged_row, merged_off, columns, inners, TILE_K, uniformed=False, tile_rows=0):
        """From the merged arrays convert_to_ter_tiled_mcsc returns (int16 or int32 indices): the blob
        multiplies by exactly what the reference kernels' walk of those arrays adds up, rows named
        several times included; `uniformed` leaves the same-sign part of every tile out, as the
        reference's kernels do under that flag (ter_spmm_kernel.cuh:59,249)."""
        merged_row = np.ascontiguousarray(merged_row)
        if merged_row.dtype not in (np.int16, np.int32):
            raise ValueError("merged_row must be int16 or int32")
        merged_off = np.ascontiguousarray(merged_off, dtype=np.int32)
        if TILE_K <= 0 or merged_off.size != columns * (-(-inners // TILE_K)) * 4:
            raise ValueError("merged_off must hold columns * ceil(inners / TILE_K) * 4 entries")
        size = ctypes.c_int64(0)
        L = _lib.lib()
        args = (merged_row.ctypes.data, merged_row.dtype.itemsize, merged_row.size, _lib.i32p(merged_off), columns, inners,
                TILE_K, int(bool(uniformed)), tile_rows)
        _lib.check(L.tl_layout_from_mcsc(*args, None, ctypes.byref(size)))
        blob = np.zeros(size.value, np.uint8)
        _lib.check(L.tl_layout_from_mcsc(*args, blob.ctypes.data, ctypes.byref(size)))
        return cls(blob)

    def validate(self):
        _lib.check(_lib.lib().tl_layout_validate(self.blob.ctypes.data, self.blob.size))

    def to_dense(self):
        w = np.zeros((self.inners, self.columns), np.int32)
        _lib.check(_lib.lib().tl_layout_to_dense(self.blob.ctypes.data, self.blob.size, _lib.i32p(w)))
        return w

    def algorithmic_bytes(self, M, x_bytes, y_bytes, scale_bytes=0):
        """Bytes one product must move at least once: the stream as stored (index bytes with their
        padding and the embedded descriptors), the chunk table, X, Y and the optional scale."""
        h = self.header
        table = (h.n_tiles * h.n_blocks + 1) * 4
        return int(h.stream_bytes + table + M * h.inners * x_bytes + M * h.columns * y_bytes + h.columns * scale_bytes)
