"""Drop-in for the reference's extension module ``ter_spmm``
(ternaryLLM_GPU/csrc/ter_spmm_wrapper.cu:350-355): the same four callables, the same
positional arguments, backed by libternary_spmm.so.

``ter_spmm`` receives the *merged* tiled-CSC arrays, as in the reference.  They are decoded
once per weight into the ternary matrix they encode (including what the reference packer's
alignment rule drops, ter_spmm_wrapper.cu:277-291), repacked into the device format and
cached; the product itself then runs through the same kernels as TernaryLinear.
"""
import torch

from . import _lib, ops, packing
from .packing import convert_to_ter_csc, convert_to_ter_tiled_csc, convert_to_ter_tiled_mcsc  # noqa: F401

_cache = {}
_CACHE_LIMIT = 256


def _weight_from_merged(row_idx, col_off, columns, inners):
    key = (row_idx.data_ptr(), col_off.data_ptr(), row_idx._version, col_off._version, row_idx.numel(), columns, inners,
           str(row_idx.device))
    hit = _cache.get(key)
    if hit is not None:
        return hit
    if col_off.numel() % (4 * columns) != 0:
        raise ValueError("col_offsets must hold 4 entries per (column, tile)")
    tiles = col_off.numel() // (4 * columns)
    tile_k = -(-inners // tiles)
    dense = packing.tiled_mcsc_to_dense(row_idx.cpu().numpy(), col_off.cpu().numpy(), columns, inners, tile_k)
    weight = ops.DeviceWeight(packing.PackedWeight.from_dense(dense), row_idx.device)
    if len(_cache) >= _CACHE_LIMIT:
        _cache.clear()
    _cache[key] = weight
    return weight


def ter_spmm(X, w_tiled_merged_row_indice, w_tiled_merged_col_offset, w_col_tile_indices,
             batch_size, rows, columns, inners, uniformed, padded):
    """-> new tensor [batch_size, rows, columns]  (ter_spmm_wrapper.cu:318-348).

    X is [batch, rows, inners] (what the reference's modules pass) or [batch, inners, rows]
    (what the reference kernel reads, ter_spmm_kernel.cuh:173); the two are told apart by
    shape.  float32 as in the reference, float16 in addition.  `uniformed`, `padded` and
    `w_col_tile_indices` only select code paths in the reference and do not change the result
    the arrays encode; they are accepted and ignored."""
    del w_col_tile_indices, uniformed, padded
    for t, name in ((X, "X"), (w_tiled_merged_row_indice, "row indices"), (w_tiled_merged_col_offset, "col offsets")):
        if t.device.type != "cuda":
            raise RuntimeError(f"{name} must be a CUDA tensor")  # TORCH_INTERNAL_ASSERT in the reference (:326-328)
    if w_tiled_merged_row_indice.dtype not in (torch.int16, torch.int32) or w_tiled_merged_col_offset.dtype != torch.int32:
        raise ValueError("row indices must be int16/int32 and col offsets int32")
    if batch_size == 0:  # 2-D input in the reference's module: empty result, nothing launched
        return torch.empty((0, rows, columns), dtype=X.dtype, device=X.device)
    weight = _weight_from_merged(w_tiled_merged_row_indice, w_tiled_merged_col_offset, columns, inners)
    if X.numel() != batch_size * rows * inners:
        raise ValueError("X does not hold batch_size * rows * inners elements")
    x3 = X.reshape(batch_size, *X.shape[-2:]) if X.dim() >= 2 else X.reshape(batch_size, rows, inners)
    if x3.shape[-1] == inners and x3.shape[-2] == rows:
        return ops.spmm(weight, x3.reshape(batch_size * rows, inners)).reshape(batch_size, rows, columns)
    if x3.shape[-2] == inners and x3.shape[-1] == rows:
        out = torch.empty((batch_size, rows, columns), dtype=X.dtype, device=X.device)
        for b in range(batch_size):
            ops.spmm(weight, x3[b], x_layout=_lib.TL_X_K_MAJOR, out=out[b])
        return out
    raise ValueError(f"X of shape {tuple(X.shape)} is neither [batch, rows, inners] nor [batch, inners, rows]")
