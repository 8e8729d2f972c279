"""Drop-in for the reference's extension module ``ter_spmm``
(ternaryLLM_GPU/csrc/ter_spmm_wrapper.cu:350-355): the same four callables, the same
positional arguments, backed by libternary_spmm.so.

``ter_spmm`` receives the *merged* tiled-CSC arrays, as in the reference.  The device format
is built from them once per weight (``prepare``; the first ``ter_spmm`` call on arrays that
were not prepared does it) and multiplies by exactly what the reference kernels' walk of
those arrays adds up (ter_spmm_kernel.cuh:197-300): what the packer's alignment rule drops
(ter_spmm_wrapper.cu:277-291) stays dropped, a row that padded arrays name twice is added
twice.  The prepared weight lives on the row-index tensor itself, so it is freed with it and
can never be taken for another weight's.
"""
import torch

from . import _lib, ops, packing
from .packing import convert_to_ter_csc, convert_to_ter_tiled_csc, convert_to_ter_tiled_mcsc  # noqa: F401

_ATTR = "_tl_prepared"


def _dispatch_tile_k(inners):
    """Tile height the reference kernels are instantiated with for this K (DISPATCH_K, utils.cuh:59-80)."""
    return 64 if inners <= 512 else 256 if inners <= 2048 else 512


def _tile_k(col_off, columns, inners):
    """The packer's TILE_K is not an argument of ter_spmm: it must be the one the reference's kernel
    dispatch assumes for this K.  Taken from the K -> tile table of the reference's Python side
    (TernaryLinear.py:9-16), then from its kernel dispatch, whichever agrees with the number of tiles
    the offsets hold; arrays packed with another height are told apart only by that number."""
    if col_off.numel() == 0 or col_off.numel() % (4 * columns) != 0:
        raise ValueError("col_offsets must hold 4 entries per (column, tile)")
    tiles = col_off.numel() // (4 * columns)
    from .linear import merged_tile_size
    for tk in (merged_tile_size(inners), _dispatch_tile_k(inners), -(-inners // tiles)):
        if -(-inners // tk) == tiles:
            return tk
    raise ValueError(f"col_offsets hold {tiles} tiles per column: no tile height fits K={inners}")


def prepare(w_tiled_merged_row_indice, w_tiled_merged_col_offset, columns, inners, uniformed=False):
    """Builds the device weight for these merged arrays and attaches it to the row-index tensor.
    Doing this once at set-up (after the arrays are on the GPU) keeps ter_spmm a pure launch, as
    ter_spmm_wrapper.cu:318-348 is; otherwise the first ter_spmm call pays for it (a copy to the
    host, the host-side build, a copy back).  Returns the ops.DeviceWeight."""
    rows, offs = w_tiled_merged_row_indice, w_tiled_merged_col_offset
    if rows.dtype not in (torch.int16, torch.int32) or offs.dtype != torch.int32:
        raise ValueError("row indices must be int16/int32 and col offsets int32")
    tile_k = _tile_k(offs, columns, inners)
    packed = packing.PackedWeight.from_mcsc(rows.detach().cpu().numpy(), offs.detach().cpu().numpy(), columns, inners,
                                            tile_k, uniformed)
    weight = ops.DeviceWeight(packed, rows.device)
    # what the entry is valid for: these two tensor objects, unmodified since, these sizes and this flag
    setattr(rows, _ATTR, (weight, offs, rows._version, offs._version, columns, inners, bool(uniformed)))
    return weight


def _prepared(rows, offs, columns, inners, uniformed):
    hit = getattr(rows, _ATTR, None)
    if hit is not None:
        weight, offs0, v_rows, v_offs, n0, k0, u0 = hit
        if (offs0 is offs and v_rows == rows._version and v_offs == offs._version and (n0, k0, u0) == (columns, inners, bool(uniformed))
                and weight.device == rows.device):
            return weight
    return prepare(rows, offs, columns, inners, uniformed)


def ter_spmm(X, w_tiled_merged_row_indice, w_tiled_merged_col_offset, w_col_tile_indices,
             batch_size, rows, columns, inners, uniformed, padded, *, x_layout=None):
    """-> new tensor [batch_size, rows, columns]  (ter_spmm_wrapper.cu:318-348).

    X is [batch, rows, inners] (what the reference's modules pass) or [batch, inners, rows]
    (what the reference kernel reads, ter_spmm_kernel.cuh:173); the two are told apart by
    shape.  When rows == inners the shape does not tell: X is then read as [batch, rows, inners]
    unless x_layout says otherwise.  x_layout (not in the reference's signature): None (by shape),
    "row_major" / 0 for [batch, rows, inners], "k_major" / 1 for [batch, inners, rows]; a layout
    that the shape contradicts raises ValueError.  float32 as in the reference, float16 in addition.
    `uniformed`: the same-sign part of every tile is left out, as in the reference's kernels.
    `padded`: accepted; every pair of the arrays is walked.  (Under this flag the reference's M > 1
    kernel leaves out what remains of a tile's pair part after whole groups of 8 entries, 16 for
    K > 2048 -- it expects pair parts padded to that size, ter_spmm_kernel.cuh:214-246 -- while its
    M = 1 kernel walks them all; a result that depends on the row count is taken for a defect, not
    for the format.)
    `w_col_tile_indices` is not read (nor by the reference's kernels, ter_spmm_kernel.cuh:159-160)."""
    del w_col_tile_indices, padded
    for t, name in ((X, "X"), (w_tiled_merged_row_indice, "row indices"), (w_tiled_merged_col_offset, "col offsets")):
        if t.device.type != "cuda":
            raise RuntimeError(f"{name} must be a CUDA tensor")  # TORCH_INTERNAL_ASSERT in the reference (:326-328)
    if batch_size == 0:  # 2-D input in the reference's module: empty result, nothing launched
        return torch.empty((0, rows, columns), dtype=X.dtype, device=X.device)
    weight = _prepared(w_tiled_merged_row_indice, w_tiled_merged_col_offset, columns, inners, uniformed)
    if X.numel() != batch_size * rows * inners:
        raise ValueError("X does not hold batch_size * rows * inners elements")
    x3 = X.reshape(batch_size, *X.shape[-2:]) if X.dim() >= 2 else X.reshape(batch_size, rows, inners)
    layouts = {None: None, "row_major": _lib.TL_X_ROW_MAJOR, "k_major": _lib.TL_X_K_MAJOR,
               _lib.TL_X_ROW_MAJOR: _lib.TL_X_ROW_MAJOR, _lib.TL_X_K_MAJOR: _lib.TL_X_K_MAJOR}
    if x_layout not in layouts:
        raise ValueError(f"x_layout={x_layout!r}: expected None, 'row_major' (0) or 'k_major' (1)")
    asked = layouts[x_layout]
    if asked != _lib.TL_X_K_MAJOR and x3.shape[-1] == inners and x3.shape[-2] == rows:
        return ops.spmm(weight, x3.reshape(batch_size * rows, inners)).reshape(batch_size, rows, columns)
    if asked != _lib.TL_X_ROW_MAJOR and x3.shape[-2] == inners and x3.shape[-1] == rows:
        return ops.spmm_kmajor_batch(weight, x3)
    if asked is not None:
        raise ValueError(f"X of shape {tuple(X.shape)} is not x_layout={x_layout!r} for rows={rows}, inners={inners}")
    raise ValueError(f"X of shape {tuple(X.shape)} is neither [batch, rows, inners] nor [batch, inners, rows]")
