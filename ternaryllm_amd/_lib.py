"""ctypes binding of libternary_spmm.so (the C ABI declared in include/ternary_spmm.h).

The library is the only compute path: importing this module fails loudly when the shared
object is missing, and no function here has a Python or CPU fallback.
"""
import ctypes
import os

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_DIR, "libternary_spmm.so")

TL_F32, TL_F16 = 0, 1
TL_X_ROW_MAJOR, TL_X_K_MAJOR = 0, 1
TL_ACT_SILU_GATE = 1
TL_PRODUCER_NONE, TL_PRODUCER_SILU_GATE, TL_PRODUCER_ADD_RMSNORM, TL_PRODUCER_RMSNORM, TL_PRODUCER_RMSNORM_SUMS = 0, 1, 2, 3, 4
TL_LAYOUT_MAGIC = 0x35474C54
TL_ERR_UNSUPPORTED = -5

ERROR_NAMES = {
    -1: "TL_ERR_ARG", -2: "TL_ERR_SHAPE", -3: "TL_ERR_DTYPE", -4: "TL_ERR_ALIGN", -5: "TL_ERR_UNSUPPORTED",
    -6: "TL_ERR_LAUNCH", -7: "TL_ERR_VALUE", -8: "TL_ERR_SIZE", -9: "TL_ERR_FORMAT",
}
# bad arguments / shapes / dtypes / values are the caller's mistake; launch failures are runtime errors
_VALUE_ERRORS = {-1, -2, -3, -4, -7, -8, -9}


class Chain(ctypes.Structure):
    """Mirror of tl_chain (the residual / RMSNorm steps a 9-16-row product may take over)."""
    _fields_ = [("residual", ctypes.c_void_p), ("residual_ld", ctypes.c_int64), ("next_norm_weight", ctypes.c_void_p),
                ("image_out", ctypes.c_void_p), ("image_ld", ctypes.c_int64), ("squares_out", ctypes.c_void_p),
                ("squares_in", ctypes.c_void_p), ("squares_blocks", ctypes.c_int32), ("eps", ctypes.c_float)]


class LayoutHeader(ctypes.Structure):
    """Mirror of tl_layout_header (256 bytes)."""
    _fields_ = [
        ("magic", ctypes.c_uint32), ("version", ctypes.c_uint32), ("inners", ctypes.c_uint32),
        ("columns", ctypes.c_uint32), ("tile_rows", ctypes.c_uint32), ("n_tiles", ctypes.c_uint32),
        ("n_blocks", ctypes.c_uint32), ("max_chunk_dwords", ctypes.c_uint32),
        ("nnz_pos", ctypes.c_uint64), ("nnz_neg", ctypes.c_uint64),
        ("off_chunkstart", ctypes.c_uint64), ("off_stream", ctypes.c_uint64),
        ("stream_bytes", ctypes.c_uint64), ("total_bytes", ctypes.c_uint64),
        ("max_run_dwords", ctypes.c_uint32), ("mean_run_dwords_x16", ctypes.c_uint32),
        ("checksum", ctypes.c_uint64), ("reserved", ctypes.c_uint32 * 40),
    ]


assert ctypes.sizeof(LayoutHeader) == 256

_I32P = ctypes.POINTER(ctypes.c_int32)
_I64P = ctypes.POINTER(ctypes.c_int64)
_HDRP = ctypes.POINTER(LayoutHeader)
_VP = ctypes.c_void_p
_INT = ctypes.c_int
_I64 = ctypes.c_int64

# name -> (restype, argtypes); every symbol the header declares
SIGNATURES = {
    "tl_last_error": (ctypes.c_char_p, []),
    "tl_version": (_INT, []),
    "tl_reload_options": (_INT, []),
    "tl_count_nnz": (_INT, [_I32P, _INT, _INT, _I64P, _I64P]),
    "tl_convert_to_ter_csc": (_INT, [_I32P, _INT, _INT, _INT, _INT, _I32P, _I32P, _I32P, _I32P]),
    "tl_convert_to_ter_tiled_csc": (_INT, [_I32P, _INT, _INT, _INT, _INT, _INT, _I32P, _I32P, _I32P, _I32P]),
    "tl_tiled_mcsc_size": (_INT, [_I32P, _INT, _INT, _INT, _INT, _INT, _INT, _INT, _I64P]),
    "tl_convert_to_ter_tiled_mcsc": (_INT, [_I32P, _INT, _INT, _INT, _INT, _INT, _INT, _INT, _I32P, _I64, _I32P, _I32P]),
    "tl_tiled_mcsc_to_dense": (_INT, [_VP, _INT, _I64, _I32P, _INT, _INT, _INT, _I32P]),
    "tl_layout_size": (_INT, [_I32P, _I32P, _INT, _INT, _INT, _INT, _I64P]),
    "tl_layout_build": (_INT, [_I32P, _I32P, _I32P, _I32P, _INT, _INT, _INT, _INT, _VP, _I64]),
    "tl_layout_from_dense": (_INT, [_I32P, _INT, _INT, _INT, _VP, _I64P]),
    "tl_layout_from_mcsc": (_INT, [_VP, _INT, _I64, _I32P, _INT, _INT, _INT, _INT, _INT, _VP, _I64P]),
    "tl_layout_validate": (_INT, [_VP, _I64]),
    "tl_layout_to_dense": (_INT, [_VP, _I64, _I32P]),
    "tl_spmm_workspace": (_INT, [_HDRP, _I64, _INT, _INT, _I64P]),
    "tl_spmm": (_INT, [_HDRP, _VP, _VP, _INT, _INT, _I64, _I64, _VP, _INT, _I64, _VP, _INT, _VP, _I64, _VP]),
    "tl_spmm_noalloc": (_INT, [_HDRP, _VP, _VP, _INT, _INT, _I64, _I64, _VP, _INT, _I64, _VP, _INT, _VP]),
    "tl_spmv_fused": (_INT, [_HDRP, _VP, _INT, _VP, _VP, _VP, ctypes.c_float, _VP, _INT, _VP, _INT, _VP, _INT, _VP]),
    "tl_spmv_fused_gated": (_INT, [_HDRP, _VP, _INT, _VP, _VP, _VP, ctypes.c_float, _VP, _INT, _VP, _INT, _VP, _INT, _VP]),
    "tl_spmm_gated": (_INT, [_HDRP, _VP, _VP, _INT, _INT, _I64, _I64, _VP, _INT, _I64, _INT, _VP, _INT, _VP, _I64, _VP]),
    "tl_spmm_chain": (_INT, [_HDRP, _VP, _VP, _INT, _INT, _I64, _I64, _VP, _INT, _I64, _INT, _VP, _INT, ctypes.POINTER(Chain), _VP, _I64, _VP]),
    "tl_mlp_gate_up": (_INT, [_HDRP, _VP, _HDRP, _VP, _VP, _INT, _INT, _I64, _I64, _VP, _INT, _I64, _VP, _VP, _INT, _INT,
                              _VP, _I64, _VP]),
    "tl_spmm_time": (_INT, [_HDRP, _VP, _VP, _INT, _INT, _I64, _I64, _VP, _INT, _I64, _VP, _INT, _VP, _I64, _VP, _INT,
                            ctypes.POINTER(ctypes.c_float)]),
    "tl_read_probe_workgroups": (_INT, []),
    "tl_stream_read_probe": (_INT, [_VP, _I64, _VP, _VP]),
    "tl_rope_cache_update": (_INT, [_VP, _INT, _I64, _INT, _INT, _VP, _VP, _VP, _VP, _VP, _VP, _I64, _VP]),
    "tl_decode_attention": (_INT, [_VP, _VP, _VP, _INT, _I64, _INT, _INT, _I64, _VP, _VP, _I64, _VP]),
    "tl_decode_attention_split": (_INT, [_VP, _VP, _VP, _INT, _I64, _INT, _INT, _I64, _VP, _VP, _I64, _INT, _VP, _I64, _VP]),
    "tl_greedy_advance": (_INT, [_VP, _INT, _I64, _INT, _VP, _VP, _I64, _VP, _VP]),
    "tl_decode_attention_fold": (_INT, [_VP, _VP, _VP, _VP, _VP, _VP, _INT, _I64, _INT, _INT, _I64, _VP, _VP, _I64, _INT, _VP, _I64, _VP, _VP]),
    "tl_decode_attention_rope": (_INT, [_VP, _VP, _VP, _VP, _VP, _INT, _I64, _INT, _INT, _I64, _VP, _VP, _I64, _INT, _VP, _I64, _VP]),
    "tl_spmv_attn_combine": (_INT, [_HDRP, _VP, _VP, _INT, _INT, _INT, _VP, _INT, _VP, _INT, _VP]),
    "tl_spmv_attn_combine_add": (_INT, [_HDRP, _VP, _VP, _INT, _INT, _INT, _VP, _VP, _INT, _VP, _INT, _VP]),
    "tl_spmv_attn_combine_add_norm": (_INT, [_HDRP, _VP, _VP, _INT, _INT, _INT, _VP, _VP, _INT, _VP, _INT, _VP, _VP, _VP, _VP]),
    "tl_spmv_add": (_INT, [_HDRP, _VP, _VP, _INT, _VP, _VP, _INT, _VP, _INT, _VP]),
    "tl_spmv_add_norm": (_INT, [_HDRP, _VP, _VP, _INT, _VP, _VP, _INT, _VP, _INT, _VP, _VP, _VP, _VP]),
    "tl_add_rmsnorm": (_INT, [_VP, _VP, _VP, _INT, _I64, _INT, ctypes.c_float, _VP, _VP, _I64, _VP]),
    "tl_silu_mul": (_INT, [_VP, _INT, _I64, _INT, _VP, _I64, _VP]),
    "tl_silu_mul_pairs": (_INT, [_VP, _INT, _I64, _INT, _VP, _I64, _VP]),
}

_lib = None


def lib():
    """The loaded shared library; raises RuntimeError when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m ternaryllm_amd.build` (needs hipcc). "
                "There is no fallback path.")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(rc):
    """Turns a negative status into ValueError (caller mistakes) or RuntimeError (launch failures)."""
    if rc == 0:
        return
    msg = lib().tl_last_error().decode("utf-8", "replace")
    text = f"{ERROR_NAMES.get(rc, rc)}: {msg}"
    if rc in _VALUE_ERRORS:
        raise ValueError(text)
    raise RuntimeError(text)


def i32p(a):
    return a.ctypes.data_as(_I32P)


def as_i32_matrix(w):
    """Host, C-contiguous int32 [K, N] view of a weight given as numpy array or CPU torch tensor."""
    if hasattr(w, "detach"):
        if w.device.type != "cpu":
            raise RuntimeError("the packers take a CPU tensor")  # the reference asserts the same (wrapper.cu:47)
        w = w.detach().numpy()
    w = np.asarray(w)
    if w.ndim != 2:
        raise ValueError(f"weight must be 2-D, got shape {w.shape}")
    if w.dtype != np.int32:
        raise ValueError(f"weight must be int32 (the reference reads data_ptr<int32_t>), got {w.dtype}")
    return np.ascontiguousarray(w)
