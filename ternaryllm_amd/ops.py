"""Tensor-level entry points over the C ABI: device weights and the ternary product.

torch is used for device memory and streams only; every product runs in libternary_spmm.so.
"""
import ctypes

import numpy as np
import torch

from . import _lib
from .packing import PackedWeight

_DTYPE_CODE = {torch.float32: _lib.TL_F32, torch.float16: _lib.TL_F16}


def _code(dtype, what):
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise ValueError(f"{what} must be float32 or float16, got {dtype}") from None


def _stream_ptr(device):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


class DeviceWeight:
    """A packed ternary weight resident on one GPU: the blob as a uint8 tensor plus the host header."""

    def __init__(self, packed, device):
        if not isinstance(packed, PackedWeight):
            raise TypeError("packed must be a PackedWeight")
        self.header = packed.header
        self.blob = torch.from_numpy(packed.blob).to(device)
        if self.blob.device.type != "cuda":
            raise RuntimeError("the ternary product runs on a GPU only: move the weight to a cuda device")
        if self.blob.data_ptr() % 256:
            raise RuntimeError("device allocator returned a blob that is not 256-byte aligned")
        self.algorithmic_bytes = packed.algorithmic_bytes

    @classmethod
    def from_blob_tensor(cls, blob_tensor):
        """Rebuilds the handle from a uint8 tensor that already holds a blob (e.g. a module buffer)."""
        self = cls.__new__(cls)
        head = blob_tensor[:256].cpu().numpy().tobytes()
        self.header = _lib.LayoutHeader.from_buffer_copy(head)
        if self.header.magic != _lib.TL_LAYOUT_MAGIC:
            raise ValueError("tensor does not hold a packed ternary weight")
        self.blob = blob_tensor
        return self

    @property
    def inners(self):
        return self.header.inners

    @property
    def columns(self):
        return self.header.columns

    @property
    def device(self):
        return self.blob.device


def _x_geometry(x, K, x_layout):
    if x.dim() != 2:
        raise ValueError("x must be 2-D here; fold batch dimensions first")
    if x_layout == _lib.TL_X_ROW_MAJOR:
        if x.shape[1] != K:
            raise ValueError(f"x has {x.shape[1]} columns, the weight has K={K}")
        M = x.shape[0]
    else:
        if x.shape[0] != K:
            raise ValueError(f"x has {x.shape[0]} rows, the weight has K={K}")
        M = x.shape[1]
    if x.stride(1) != 1:
        x = x.contiguous()
    return x, M, x.stride(0) if x.shape[0] > 1 else max(x.shape[1], 1)


_workspaces = {}


def release_workspaces():
    """Drops every cached scratch buffer (one per (device, stream) that has run a product needing one; torch
    reuses the memory in stream order).  Not while a captured HIP graph that contains such a product is still
    to be replayed: the graph holds the buffer's address."""
    _workspaces.clear()
    _attn_workspaces.clear()


def _workspace(header, M, x_code, x_layout, device):
    """Scratch for one call: one buffer per (device, stream), kept and only replaced by a larger one
    (work on one stream is ordered, so consecutive calls may share it); release_workspaces() drops them."""
    need = ctypes.c_int64(0)
    _lib.check(_lib.lib().tl_spmm_workspace(ctypes.byref(header), M, x_code, x_layout, ctypes.byref(need)))
    if need.value == 0:
        return None, 0
    key = (device.index, torch.cuda.current_stream(device).cuda_stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < need.value:
        ws = torch.empty(max(need.value, 1 << 20), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws, ws.numel()


def _scale_args(scale, N, device):
    if scale is None:
        return None, _lib.TL_F32
    if scale.device != device or scale.numel() != N or not scale.is_contiguous():
        raise ValueError("scale must be a contiguous tensor of N elements on the weight's device")
    return scale, _code(scale.dtype, "scale")


def spmm(weight, x, scale=None, out_dtype=None, x_layout=_lib.TL_X_ROW_MAJOR, out=None):
    """y[M, N] = (x @ W) * scale with fp32 accumulation.

    weight: DeviceWeight; x: cuda tensor [M, K] (row-major layout) or [K, M] (K-major layout),
    float32 or float16; scale: optional [N] tensor; returns a new [M, N] tensor of out_dtype
    (default: x.dtype)."""
    if x.device != weight.device:
        raise RuntimeError(f"x is on {x.device}, the weight on {weight.device}")
    x_code = _code(x.dtype, "x")
    x, M, ldx = _x_geometry(x, weight.inners, x_layout)
    N = weight.columns
    out_dtype = out_dtype or x.dtype
    y_code = _code(out_dtype, "out_dtype")
    if M == 0:
        return torch.empty((0, N), dtype=out_dtype, device=x.device)
    y = out if out is not None else torch.empty((M, N), dtype=out_dtype, device=x.device)
    if y.shape != (M, N) or y.dtype != out_dtype or y.stride(1) != 1:
        raise ValueError("out must be an [M, N] tensor of out_dtype with unit column stride")
    scale, s_code = _scale_args(scale, N, x.device)
    ws, ws_bytes = _workspace(weight.header, M, x_code, x_layout, x.device)
    with torch.cuda.device(x.device):
        rc = _lib.lib().tl_spmm(ctypes.byref(weight.header), weight.blob.data_ptr(), x.data_ptr(), x_code, x_layout, ldx, M,
                                y.data_ptr(), y_code, y.stride(0), scale.data_ptr() if scale is not None else None, s_code,
                                ws.data_ptr() if ws is not None else None, ws_bytes, _stream_ptr(x.device))
    _lib.check(rc)
    return y


def spmm_kmajor_batch(weight, x3, scale=None):
    """[batch, K, rows] -> [batch, rows, N]: the batch's K-major matrices laid side by side as one [K, batch * rows]
    matrix (one copy when batch > 1), then ONE product over all of them instead of one per batch entry."""
    batch, K, rows = x3.shape
    side_by_side = x3[0] if batch == 1 else x3.permute(1, 0, 2).reshape(K, batch * rows)
    return spmm(weight, side_by_side, scale, x_layout=_lib.TL_X_K_MAJOR).view(batch, rows, weight.columns)


def spmm_gated(weight, x, scale=None, x_layout=_lib.TL_X_ROW_MAJOR, kmajor=False):
    """h[M, N / 2] with h[:, j] = silu(y[:, 2j]) * y[:, 2j + 1], y = (x @ W) * scale, for a gate | up weight whose
    columns are (gate, up) pairs.  One launch (tl_spmm_gated) where the shape's kernel has the epilogue -- one
    aligned row, 9 to 16 fp16 rows and a wide N, or more than 48 rows -- else the product followed by
    silu_mul(pairs=True); the result is the same bit for bit.  With kmajor the transpose [N / 2, M] is returned, a
    view of a K-major image."""
    if x.device != weight.device:
        raise RuntimeError(f"x is on {x.device}, the weight on {weight.device}")
    if weight.columns % 2:
        raise ValueError("gate and up columns come in pairs: N must be even")
    x_code = _code(x.dtype, "x")
    xg, M, ldx = _x_geometry(x, weight.inners, x_layout)
    half = weight.columns // 2
    if not (kmajor and (M == 1 or M > 16)):  # the library says TL_ERR_UNSUPPORTED where the shape's kernel has no such epilogue
        if kmajor:
            out, ld = _kmajor_image(M, half, x)
        else:
            out, ld = torch.empty((M, half), dtype=x.dtype, device=x.device), half
        sc, s_code = _scale_args(scale, weight.columns, x.device)
        ws, ws_bytes = _workspace(weight.header, M, x_code, x_layout, x.device)
        with torch.cuda.device(x.device):
            rc = _lib.lib().tl_spmm_gated(ctypes.byref(weight.header), weight.blob.data_ptr(), xg.data_ptr(), x_code, x_layout, ldx, M,
                                          out.data_ptr(), x_code, ld, _lib.TL_X_K_MAJOR if kmajor else _lib.TL_X_ROW_MAJOR,
                                          sc.data_ptr() if sc is not None else None, s_code,
                                          ws.data_ptr() if ws is not None else None, ws_bytes, _stream_ptr(x.device))
        if rc != _lib.TL_ERR_UNSUPPORTED:
            _lib.check(rc)
            return out[:, :M] if kmajor else out
    return silu_mul(spmm(weight, x, scale, x_layout=x_layout), kmajor=kmajor, pairs=True)


def spmm_chain(weight, x, scale=None, x_layout=_lib.TL_X_ROW_MAJOR, residual=None, next_norm_weight=None, squares_in=None,
               eps=0.0, gated=False, kmajor=False):
    """A product of 9 to 16 fp16 rows that takes over the residual add and the RMSNorm around it (tl_spmm_chain), for a
    decoder layer without elementwise kernels.
      residual [M, N]: the result is residual + (x @ W) * scale;
      next_norm_weight [N]: the call also returns the K-major image of result * next_norm_weight (a [N, M] view: the
        activations of the next product, x_layout=1) and squares [N / 16, 16] float32, per block of 16 columns the sum
        of result^2 -- what that product needs as squares_in;
      squares_in: x is such an image; the sums are scaled by rsqrt(mean square + eps) of each row;
      gated / kmajor: as in spmm_gated (where the kernel for the width has no gated epilogue the gate is a second launch).
    Returns y, or (y, image, squares) with next_norm_weight.  Raises RuntimeError (TL_ERR_UNSUPPORTED) where the kernel
    for the shape has no such step."""
    if x.device != weight.device:
        raise RuntimeError(f"x is on {x.device}, the weight on {weight.device}")
    x_code = _code(x.dtype, "x")
    xg, M, ldx = _x_geometry(x, weight.inners, x_layout)
    N = weight.columns
    if kmajor and not gated:
        raise ValueError("a K-major result is written by the gated epilogue only (next_norm_weight gives the image of a plain product)")
    width = N // 2 if gated else N
    if kmajor:
        y, ldy = _kmajor_image(M, width, x)
    else:
        y, ldy = torch.empty((M, width), dtype=x.dtype, device=x.device), width
    chain = _lib.Chain()
    if residual is not None:
        if residual.shape != (M, N) or residual.dtype != x.dtype or residual.stride(1) != 1 or residual.device != x.device:
            raise ValueError("residual must be an [M, N] tensor of x's dtype with unit column stride")
        chain.residual, chain.residual_ld = residual.data_ptr(), residual.stride(0)
    image = squares = None
    if next_norm_weight is not None:
        if next_norm_weight.numel() != N or next_norm_weight.dtype != x.dtype or not next_norm_weight.is_contiguous():
            raise ValueError("next_norm_weight must be a contiguous [N] tensor of x's dtype")
        image, ild = _kmajor_image(M, N, x)
        squares = torch.empty(((N + 15) // 16, 16), dtype=torch.float32, device=x.device)
        chain.next_norm_weight, chain.image_out, chain.image_ld, chain.squares_out = next_norm_weight.data_ptr(), image.data_ptr(), ild, squares.data_ptr()
    if squares_in is not None:
        if squares_in.dtype != torch.float32 or squares_in.dim() != 2 or squares_in.shape[1] != 16 or not squares_in.is_contiguous():
            raise ValueError("squares_in must be a contiguous float32 [blocks, 16] tensor")
        chain.squares_in, chain.squares_blocks = squares_in.data_ptr(), squares_in.shape[0]
    chain.eps = float(eps)
    sc, s_code = _scale_args(scale, N, x.device)
    ws, ws_bytes = _workspace(weight.header, M, x_code, x_layout, x.device)
    y_layout = -1 if not gated else (_lib.TL_X_K_MAJOR if kmajor else _lib.TL_X_ROW_MAJOR)
    with torch.cuda.device(x.device):
        rc = _lib.lib().tl_spmm_chain(ctypes.byref(weight.header), weight.blob.data_ptr(), xg.data_ptr(), x_code, x_layout, ldx, M,
                                      y.data_ptr(), x_code, ldy, y_layout, sc.data_ptr() if sc is not None else None, s_code,
                                      ctypes.byref(chain), ws.data_ptr() if ws is not None else None, ws_bytes, _stream_ptr(x.device))
    if rc == _lib.TL_ERR_UNSUPPORTED and gated:
        # no gated epilogue in the kernel for this width: the gate takes a launch of its own
        plain = spmm_chain(weight, x, scale, x_layout, squares_in=squares_in, eps=eps)
        return silu_mul(plain, kmajor=kmajor, pairs=True)
    _lib.check(rc)
    if kmajor:
        y = y[:, :M]
    return (y, image[:, :M], squares) if next_norm_weight is not None else y


def mlp_gate_up(gate, up, x, gate_scale=None, up_scale=None, out_dtype=None):
    """h[M, N] = silu((x @ Wg) * sg) * ((x @ Wu) * su) in one pass over x (M > 48), else two products."""
    if gate.columns != up.columns or gate.inners != up.inners:
        raise ValueError("gate and up weights must have the same shape")
    x_code = _code(x.dtype, "x")
    x, M, ldx = _x_geometry(x, gate.inners, _lib.TL_X_ROW_MAJOR)
    N = gate.columns
    out_dtype = out_dtype or x.dtype
    if M <= 48 or gate.header.tile_rows != up.header.tile_rows:
        g = spmm(gate, x, gate_scale, torch.float32)
        u = spmm(up, x, up_scale, torch.float32)
        return (torch.nn.functional.silu(g) * u).to(out_dtype)
    h = torch.empty((M, N), dtype=out_dtype, device=x.device)
    gs, s_code = _scale_args(gate_scale, N, x.device)
    us, s_code2 = _scale_args(up_scale, N, x.device)
    if (gs is None) != (us is None) or (gs is not None and s_code != s_code2):
        raise ValueError("pass both scales, of one dtype, or neither")
    ws, ws_bytes = _workspace(gate.header, M, x_code, _lib.TL_X_ROW_MAJOR, x.device)
    with torch.cuda.device(x.device):
        rc = _lib.lib().tl_mlp_gate_up(ctypes.byref(gate.header), gate.blob.data_ptr(), ctypes.byref(up.header),
                                       up.blob.data_ptr(), x.data_ptr(), x_code, _lib.TL_X_ROW_MAJOR, ldx, M, h.data_ptr(),
                                       _code(out_dtype, "out_dtype"), h.stride(0), gs.data_ptr() if gs is not None else None,
                                       us.data_ptr() if us is not None else None, s_code, _lib.TL_ACT_SILU_GATE,
                                       ws.data_ptr() if ws is not None else None, ws_bytes, _stream_ptr(x.device))
    _lib.check(rc)
    return h


def spmv_fused(weight, producer, inp, inp2=None, norm_weight=None, eps=0.0, scale=None, out_dtype=None, want_sum=False, gated=False):
    """y[1, N] = (x @ W) * scale for one activation row x that the call produces itself (tl_spmv_fused):
    producer "silu_gate": x = silu(inp[:K]) * inp[K:] for a gate | up row inp of 2K values;
    producer "add_rmsnorm": s = inp + inp2 (inp2 may be None), x = rmsnorm(s) * norm_weight; with want_sum the
    call also returns s (a new tensor);
    producer "rmsnorm": x = rmsnorm(inp) * norm_weight with the normalisation factor applied to the column sums (the
    row multiplied is inp * norm_weight in inp's dtype; no part of the kernel waits for the mean);
    producer "rmsnorm_sums": the same product for a row that spmv_add(..., next_norm_weight=) left behind: inp is its
    image (row * norm weight), inp2 its float32 sums of squares, one per 16 values; norm_weight stays None.
    Returns y, or (y, s).  Raises RuntimeError (TL_ERR_UNSUPPORTED) where the
    fused kernel does not apply (K or the tile height not whole 16-byte pieces); callers then use the separate operators.
    gated: the weight's columns are (gate, up) pairs and y is [1, N / 2] with y[j] = silu(y'[2j]) * y'[2j + 1]
    (tl_spmv_fused_gated)."""
    K, N = weight.inners, weight.columns
    if gated and N % 2:
        raise ValueError("gate and up columns come in pairs: N must be even")
    code = {"silu_gate": _lib.TL_PRODUCER_SILU_GATE, "add_rmsnorm": _lib.TL_PRODUCER_ADD_RMSNORM, "rmsnorm": _lib.TL_PRODUCER_RMSNORM,
            "rmsnorm_sums": _lib.TL_PRODUCER_RMSNORM_SUMS}[producer]
    if producer == "rmsnorm_sums":
        if norm_weight is not None or want_sum:
            raise ValueError("the image already holds the norm weight, and the sum is the row that came with it")
        if inp2 is None or inp2.dtype != torch.float32 or inp2.numel() != (K + 15) // 16 or not inp2.is_contiguous() or inp2.device != weight.device:
            raise ValueError("inp2 must hold one float32 sum of squares per 16 values of the row")
    if producer == "rmsnorm" and (inp2 is not None or want_sum):
        raise ValueError("the rmsnorm producer has no second summand: the residual add belongs to the product before it (spmv_add)")
    x_code = _code(inp.dtype, "inp")
    need = 2 * K if producer == "silu_gate" else K
    tensors = [inp] + [t for t in (inp2 if producer != "rmsnorm_sums" else None, norm_weight) if t is not None]
    for t in tensors:
        if t.numel() != (need if t is inp else K) or not t.is_contiguous() or t.dtype != inp.dtype or t.device != weight.device:
            raise ValueError("inputs must be contiguous rows of the weight's K (2K for a gate | up row), one dtype, on the weight's device")
    if producer in ("add_rmsnorm", "rmsnorm") and norm_weight is None:
        raise ValueError(f"{producer} needs norm_weight")
    out_dtype = out_dtype or inp.dtype
    y = torch.empty((1, N // 2 if gated else N), dtype=out_dtype, device=inp.device)
    s_out = torch.empty(K, dtype=inp.dtype, device=inp.device).view(inp.shape) if (want_sum and producer == "add_rmsnorm") else None
    scale, s_code = _scale_args(scale, N, inp.device)
    call = _lib.lib().tl_spmv_fused_gated if gated else _lib.lib().tl_spmv_fused
    with torch.cuda.device(inp.device):
        rc = call(ctypes.byref(weight.header), weight.blob.data_ptr(), code, inp.data_ptr(),
                                      inp2.data_ptr() if inp2 is not None else None,
                                      norm_weight.data_ptr() if norm_weight is not None else None, float(eps),
                                      s_out.data_ptr() if s_out is not None else None, x_code, y.data_ptr(), _code(out_dtype, "out_dtype"),
                                      scale.data_ptr() if scale is not None else None, s_code, _stream_ptr(inp.device))
    _lib.check(rc)
    return (y, s_out) if want_sum else y


def spmv_add(weight, x, residual, scale=None, next_norm_weight=None):
    """residual + (x @ W) * scale for one contiguous row x [1, K] or [K] and a residual row of N values (tl_spmv_add):
    the residual add of a decoder layer in the epilogue of the product in front of it, rounded as the separate add of
    the stored product would round.  Returns a new [1, N] tensor of residual's dtype.
    next_norm_weight [N]: the weight of the RMSNorm the new row goes into (tl_spmv_add_norm).  Returns (y, image,
    squares) then: image = y * next_norm_weight in y's dtype and squares [ceil(N / 16)] float32, the sums of y^2 over
    runs of 16 values -- the inputs of spmv_fused(..., "rmsnorm_sums", image, squares).  Raises RuntimeError
    (TL_ERR_UNSUPPORTED) where the weight's shape leaves the product to a kernel without that epilogue."""
    K, N = weight.inners, weight.columns
    if x.numel() != K or residual.numel() != N or not x.is_contiguous() or not residual.is_contiguous():
        raise ValueError("x must be a contiguous row of K values and residual one of N")
    if x.device != weight.device or residual.device != weight.device:
        raise RuntimeError("x and residual must be on the weight's device")
    y = torch.empty((1, N), dtype=residual.dtype, device=x.device)
    scale, s_code = _scale_args(scale, N, x.device)
    if next_norm_weight is not None:
        if next_norm_weight.numel() != N or next_norm_weight.dtype != residual.dtype or not next_norm_weight.is_contiguous() or \
                next_norm_weight.device != weight.device:
            raise ValueError("next_norm_weight must be a contiguous row of N values of the residual's dtype on the weight's device")
        image = torch.empty((1, N), dtype=residual.dtype, device=x.device)
        squares = torch.empty((N + 15) // 16, dtype=torch.float32, device=x.device)
        with torch.cuda.device(x.device):
            rc = _lib.lib().tl_spmv_add_norm(ctypes.byref(weight.header), weight.blob.data_ptr(), x.data_ptr(), _code(x.dtype, "x"),
                                             residual.data_ptr(), y.data_ptr(), _code(residual.dtype, "residual"),
                                             scale.data_ptr() if scale is not None else None, s_code, next_norm_weight.data_ptr(),
                                             image.data_ptr(), squares.data_ptr(), _stream_ptr(x.device))
        _lib.check(rc)
        return y, image, squares
    with torch.cuda.device(x.device):
        rc = _lib.lib().tl_spmv_add(ctypes.byref(weight.header), weight.blob.data_ptr(), x.data_ptr(), _code(x.dtype, "x"), residual.data_ptr(),
                                    y.data_ptr(), _code(residual.dtype, "residual"), scale.data_ptr() if scale is not None else None, s_code,
                                    _stream_ptr(x.device))
    _lib.check(rc)
    return y


def spmv_attn_combine(weight, pieces, head_dim, x_dtype, scale=None, out_dtype=None, residual=None, next_norm_weight=None):
    """y[1, N] = (a @ W) * scale where a is the attention output (rounded to x_dtype) that `pieces` -- what
    decode_attention_pieces returned for batch 1 -- add up to: the output projection with the fold of the
    pieces inside (tl_spmv_attn_combine).  residual: a row of N values of the output dtype that the result is
    added to, as in spmv_add; with next_norm_weight [N] as well, returns (y, image, squares) as spmv_add does
    (tl_spmv_attn_combine_add_norm).  Raises RuntimeError (TL_ERR_UNSUPPORTED) where the fused kernel does not apply."""
    K, N = weight.inners, weight.columns
    if pieces.dtype != torch.float32 or pieces.dim() != 3 or not pieces.is_contiguous() or pieces.device != weight.device:
        raise ValueError("pieces must be a contiguous float32 [heads, splits, head_dim + 4] tensor on the weight's device")
    heads, splits, width = pieces.shape
    if width != head_dim + 4 or heads * head_dim != K:
        raise ValueError(f"pieces of shape {tuple(pieces.shape)} do not make a row of K={K} with head_dim={head_dim}")
    out_dtype = out_dtype or x_dtype
    if residual is not None and (residual.numel() != N or residual.dtype != out_dtype or not residual.is_contiguous() or residual.device != weight.device):
        raise ValueError("residual must be a contiguous row of N values of the output dtype on the weight's device")
    y = torch.empty((1, N), dtype=out_dtype, device=pieces.device)
    scale, s_code = _scale_args(scale, N, pieces.device)
    if next_norm_weight is not None:
        if residual is None:
            raise ValueError("next_norm_weight goes with a residual row")
        if next_norm_weight.numel() != N or next_norm_weight.dtype != out_dtype or not next_norm_weight.is_contiguous() or \
                next_norm_weight.device != weight.device:
            raise ValueError("next_norm_weight must be a contiguous row of N values of the output dtype on the weight's device")
        image = torch.empty((1, N), dtype=out_dtype, device=pieces.device)
        squares = torch.empty((N + 15) // 16, dtype=torch.float32, device=pieces.device)
        with torch.cuda.device(pieces.device):
            rc = _lib.lib().tl_spmv_attn_combine_add_norm(ctypes.byref(weight.header), weight.blob.data_ptr(), pieces.data_ptr(), splits, head_dim,
                                                          _code(x_dtype, "x_dtype"), residual.data_ptr(), y.data_ptr(), _code(out_dtype, "out_dtype"),
                                                          scale.data_ptr() if scale is not None else None, s_code, next_norm_weight.data_ptr(),
                                                          image.data_ptr(), squares.data_ptr(), _stream_ptr(pieces.device))
        _lib.check(rc)
        return y, image, squares
    with torch.cuda.device(pieces.device):
        if residual is None:
            rc = _lib.lib().tl_spmv_attn_combine(ctypes.byref(weight.header), weight.blob.data_ptr(), pieces.data_ptr(), splits, head_dim,
                                                 _code(x_dtype, "x_dtype"), y.data_ptr(), _code(out_dtype, "out_dtype"),
                                                 scale.data_ptr() if scale is not None else None, s_code, _stream_ptr(pieces.device))
        else:
            rc = _lib.lib().tl_spmv_attn_combine_add(ctypes.byref(weight.header), weight.blob.data_ptr(), pieces.data_ptr(), splits, head_dim,
                                                     _code(x_dtype, "x_dtype"), residual.data_ptr(), y.data_ptr(), _code(out_dtype, "out_dtype"),
                                                     scale.data_ptr() if scale is not None else None, s_code, _stream_ptr(pieces.device))
    _lib.check(rc)
    return y


def spmm_time(weight, x, iters, scale=None, out_dtype=None, x_layout=_lib.TL_X_ROW_MAJOR):
    """Mean milliseconds per tl_spmm call over `iters` back-to-back calls, timed with HIP events
    recorded on the stream the kernels run on.  Returns (ms, y)."""
    x_code = _code(x.dtype, "x")
    x, M, ldx = _x_geometry(x, weight.inners, x_layout)
    N = weight.columns
    out_dtype = out_dtype or x.dtype
    y = torch.empty((M, N), dtype=out_dtype, device=x.device)
    scale, s_code = _scale_args(scale, N, x.device)
    ws, ws_bytes = _workspace(weight.header, M, x_code, x_layout, x.device)
    ms = ctypes.c_float(0)
    with torch.cuda.device(x.device):
        rc = _lib.lib().tl_spmm_time(ctypes.byref(weight.header), weight.blob.data_ptr(), x.data_ptr(), x_code,
                                     x_layout, ldx, M, y.data_ptr(), _code(out_dtype, "out_dtype"), y.stride(0),
                                     scale.data_ptr() if scale is not None else None, s_code,
                                     ws.data_ptr() if ws is not None else None, ws_bytes, _stream_ptr(x.device), iters,
                                     ctypes.byref(ms))
    _lib.check(rc)
    return ms.value, y


def stream_read_probe(buf, out=None):
    """One launch that only reads the bytes of `buf` (a contiguous cuda tensor of a multiple of 16 bytes), folded into
    one dword per workgroup of `out` (made when not given): the floor of a launch that streams that much memory."""
    n = _lib.lib().tl_read_probe_workgroups()
    if out is None:
        out = torch.empty(n, dtype=torch.int32, device=buf.device)
    if out.numel() < n or out.dtype != torch.int32 or not buf.is_contiguous():
        raise ValueError("out must hold one int32 per probe workgroup, buf must be contiguous")
    with torch.cuda.device(buf.device):
        _lib.check(_lib.lib().tl_stream_read_probe(buf.data_ptr(), buf.numel() * buf.element_size(), out.data_ptr(), _stream_ptr(buf.device)))
    return out


def rope_cache_update(qkv, cos_table, sin_table, pos, q_out, k_cache, v_cache):
    """Rotates q and k of one token per batch row and writes k, v into row `pos` of the caches.
    qkv: [B, 3 * heads * head_dim] (q | k | v); cos/sin tables: [max_seq, head_dim]; pos: int64 device
    tensor with one element; q_out: [B, heads, head_dim]; caches: [B, heads, max_seq, head_dim]."""
    B, heads, max_seq, hd = k_cache.shape
    for t in (qkv, cos_table, sin_table, q_out, k_cache, v_cache):
        if not t.is_contiguous() or t.dtype != qkv.dtype or t.device != qkv.device:
            raise ValueError("tensors must be contiguous, of one dtype, on one device")
    if qkv.numel() != B * 3 * heads * hd or q_out.numel() != B * heads * hd or v_cache.shape != k_cache.shape:
        raise ValueError("shapes of qkv, q_out and the caches do not agree")
    if cos_table.shape != (max_seq, hd) or sin_table.shape != (max_seq, hd):
        raise ValueError("rotary tables must be [max_seq, head_dim]")
    if pos.dtype != torch.int64 or pos.numel() != 1 or pos.device != qkv.device:
        raise ValueError("pos must be a one-element int64 tensor on the same device")
    with torch.cuda.device(qkv.device):
        rc = _lib.lib().tl_rope_cache_update(qkv.data_ptr(), _code(qkv.dtype, "qkv"), B, heads, hd, cos_table.data_ptr(),
                                             sin_table.data_ptr(), pos.data_ptr(), q_out.data_ptr(), k_cache.data_ptr(),
                                             v_cache.data_ptr(), max_seq, _stream_ptr(qkv.device))
    _lib.check(rc)
    return q_out


def _kmajor_image(rows, width, like):
    """An uninitialised K-major image [width][ld] for `rows` activation rows, ld = rows rounded up to 16: the
    layout spmm multiplies 5 to 48 rows from without a re-layout pass.  Returns (buffer, ld)."""
    ld = (rows + 15) // 16 * 16
    return torch.empty((width, ld), dtype=like.dtype, device=like.device), ld


_attn_workspaces = {}
_attn_arrivals = {}
_ATTN_MAX_SPLITS = 8


def _attention_splits(B, heads, device):
    """Workgroups per (batch row, head): as many as keep half the compute units busy (more pieces cost the
    fold more than they save the pass over the cache), at most 8."""
    units = torch.cuda.get_device_properties(device).multi_processor_count
    return max(1, min(_ATTN_MAX_SPLITS, units // max(1, 2 * B * heads)))


def _check_fresh(fresh, k_cache):
    """fresh = (qkv, cos_table, sin_table) of rope_cache_update, for the attention calls that do its work too."""
    B, heads, max_seq, hd = k_cache.shape
    qkv, cos_table, sin_table = fresh
    for t in (qkv, cos_table, sin_table):
        if not t.is_contiguous() or t.dtype != k_cache.dtype or t.device != k_cache.device:
            raise ValueError("tensors must be contiguous, of one dtype, on one device")
    if qkv.numel() != B * 3 * heads * hd:
        raise ValueError("qkv must hold q | k | v of one token per batch row")
    if cos_table.shape != (max_seq, hd) or sin_table.shape != (max_seq, hd):
        raise ValueError("rotary tables must be [max_seq, head_dim]")
    return qkv, cos_table, sin_table


def _attention_call(q, fresh, k_cache, v_cache, pos, out_ptr, ld, splits, ws_ptr, ws_bytes, arrivals_ptr=None):
    B, heads, max_seq, hd = k_cache.shape
    L = _lib.lib()
    with torch.cuda.device(k_cache.device):
        if arrivals_ptr is not None:
            qkv, cos_table, sin_table = fresh if fresh is not None else (None, None, None)
            rc = L.tl_decode_attention_fold(q.data_ptr() if fresh is None else None, qkv.data_ptr() if qkv is not None else None,
                                            cos_table.data_ptr() if qkv is not None else None, sin_table.data_ptr() if qkv is not None else None,
                                            k_cache.data_ptr(), v_cache.data_ptr(), _code(k_cache.dtype, "cache"), B, heads, hd, max_seq,
                                            pos.data_ptr(), out_ptr, ld, splits, ws_ptr, ws_bytes, arrivals_ptr, _stream_ptr(k_cache.device))
        elif fresh is None:
            rc = L.tl_decode_attention_split(q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), _code(q.dtype, "q"), B, heads, hd,
                                             max_seq, pos.data_ptr(), out_ptr, ld, splits, ws_ptr, ws_bytes, _stream_ptr(q.device))
        else:
            qkv, cos_table, sin_table = fresh
            rc = L.tl_decode_attention_rope(qkv.data_ptr(), cos_table.data_ptr(), sin_table.data_ptr(), k_cache.data_ptr(),
                                            v_cache.data_ptr(), _code(qkv.dtype, "qkv"), B, heads, hd, max_seq, pos.data_ptr(), out_ptr, ld,
                                            splits, ws_ptr, ws_bytes, _stream_ptr(qkv.device))
    _lib.check(rc)


def decode_attention(q, k_cache, v_cache, pos, out=None, kmajor=False, splits=None, fresh=None, fold_inside=True):
    """Attention of one query per (batch row, head) over cache rows [0, pos].  q: [B, heads, head_dim];
    caches: [B, heads, max_seq, head_dim]; pos: one-element int64 device tensor.  Returns [B, heads * head_dim],
    or with kmajor its transpose [heads * head_dim, B] as a view of a K-major image (for spmm's x_layout=1).
    splits: workgroups that share the cache rows of a (batch row, head) (1 to 8; default: by the size of
    the step, see _attention_splits).  Their pieces are folded by the last of them to finish (tl_decode_attention_fold),
    or with fold_inside=False by a second launch (tl_decode_attention_split, tl_decode_attention_rope).
    fresh=(qkv, cos_table, sin_table) with q=None: the same kernel also does what rope_cache_update does --
    rotates q and k of the token and writes its k, v into cache row `pos` -- in the one launch."""
    B, heads, max_seq, hd = k_cache.shape
    if (q is None) == (fresh is None):
        raise ValueError("give q, or fresh=(qkv, cos_table, sin_table) with q=None")
    if fresh is not None:
        fresh = _check_fresh(fresh, k_cache)
        q = fresh[0]   # stands for dtype, device and the element count below
    ld = 0
    if kmajor:
        if out is not None:
            raise ValueError("out= and kmajor exclude each other")
        image, ld = _kmajor_image(B, heads * hd, q)
        out = image
    elif out is None:
        out = torch.empty((B, heads * hd), dtype=q.dtype, device=q.device)
    for t in (q, k_cache, v_cache, out):
        if not t.is_contiguous() or t.dtype != q.dtype or t.device != q.device:
            raise ValueError("tensors must be contiguous, of one dtype, on one device")
    if q.numel() != B * heads * hd * (3 if fresh is not None else 1) or out.numel() != max(B, ld) * heads * hd or v_cache.shape != k_cache.shape:
        raise ValueError("shapes of q, out and the caches do not agree")
    if pos.dtype != torch.int64 or pos.numel() != 1 or pos.device != q.device:
        raise ValueError("pos must be a one-element int64 tensor on the same device")
    if splits is None:
        splits = _attention_splits(B, heads, q.device)
    ws_ptr, ws_bytes, arrivals_ptr = None, 0, None
    if splits > 1:
        # scratch for the pieces: one buffer per (device, stream), like the products' (work on a stream is ordered)
        key = (q.device.index, torch.cuda.current_stream(q.device).cuda_stream)
        need = B * heads * _ATTN_MAX_SPLITS * (hd + 4) * 4
        ws = _attn_workspaces.get(key)
        if ws is None or ws.numel() < need:
            ws = torch.empty(need, dtype=torch.uint8, device=q.device)
            _attn_workspaces[key] = ws
        ws_ptr, ws_bytes = ws.data_ptr(), ws.numel()
        if fold_inside:
            # one counter per (batch row, head): zero between calls (the kernel leaves them so)
            counters = _attn_arrivals.get(key)
            if counters is None or counters.numel() < B * heads:
                counters = torch.zeros(B * heads, dtype=torch.int32, device=q.device)
                _attn_arrivals[key] = counters
            arrivals_ptr = counters.data_ptr()
    _attention_call(None if fresh is not None else q, fresh, k_cache, v_cache, pos, out.data_ptr(), ld, splits, ws_ptr, ws_bytes, arrivals_ptr)
    return out[:, :B] if kmajor else out


def decode_attention_pieces(q, k_cache, v_cache, pos, splits=None, fresh=None):
    """The attention of decode_attention left unfolded: float32 [B * heads, splits, head_dim + 4], per piece
    head_dim unnormalised sums, the piece's maximum and its sum of exponentials (two unused floats behind them).
    spmv_attn_combine folds them inside the output projection (batch 1).  fresh: as in decode_attention."""
    B, heads, max_seq, hd = k_cache.shape
    if (q is None) == (fresh is None):
        raise ValueError("give q, or fresh=(qkv, cos_table, sin_table) with q=None")
    if fresh is not None:
        fresh = _check_fresh(fresh, k_cache)
        q = fresh[0]
    for t in (q, k_cache, v_cache):
        if not t.is_contiguous() or t.dtype != q.dtype or t.device != q.device:
            raise ValueError("tensors must be contiguous, of one dtype, on one device")
    if q.numel() != B * heads * hd * (3 if fresh is not None else 1) or v_cache.shape != k_cache.shape:
        raise ValueError("shapes of q and the caches do not agree")
    if pos.dtype != torch.int64 or pos.numel() != 1 or pos.device != q.device:
        raise ValueError("pos must be a one-element int64 tensor on the same device")
    if splits is None:
        splits = _attention_splits(B, heads, q.device)
    pieces = torch.empty((B * heads, splits, hd + 4), dtype=torch.float32, device=q.device)
    _attention_call(None if fresh is not None else q, fresh, k_cache, v_cache, pos, None, 0, splits, pieces.data_ptr(), pieces.numel() * 4)
    return pieces


def greedy_advance(logits, token, pos=None, max_pos=0, mask=None):
    """token[b] = argmax(logits[b]) (torch.argmax's result), and, with pos, pos = min(pos + 1, max_pos) and
    mask.view(-1)[pos] = True: the end of a greedy decode step in one launch (tl_greedy_advance).  logits: contiguous
    [B, vocab]; token: int64 [B]; pos: one-element int64 tensor; mask: bool tensor with one element per cache slot."""
    if logits.dim() != 2 or not logits.is_contiguous() or token.dtype != torch.int64 or token.numel() != logits.shape[0] or not token.is_contiguous():
        raise ValueError("logits must be contiguous [B, vocab] and token an int64 tensor of B elements")
    if pos is not None and (pos.dtype != torch.int64 or pos.numel() != 1):
        raise ValueError("pos must be a one-element int64 tensor")
    if mask is not None and (pos is None or mask.dtype != torch.bool or not mask.is_contiguous() or mask.numel() <= max_pos):
        raise ValueError("mask must be a contiguous bool tensor with more than max_pos elements, given together with pos")
    for t in (token, pos, mask):
        if t is not None and t.device != logits.device:
            raise ValueError("tensors must be on one device")
    with torch.cuda.device(logits.device):
        rc = _lib.lib().tl_greedy_advance(logits.data_ptr(), _code(logits.dtype, "logits"), logits.shape[0], logits.shape[1], token.data_ptr(),
                                          pos.data_ptr() if pos is not None else None, int(max_pos),
                                          mask.data_ptr() if mask is not None else None, _stream_ptr(logits.device))
    _lib.check(rc)
    return token


def add_rmsnorm(x, y, weight, eps, kmajor=False):
    """(x + y, rmsnorm(x + y) * weight) for [rows, width] tensors of one dtype; y may be None (then the
    first result is x itself).  With kmajor the second result is its transpose [width, rows], a view of a
    K-major image (for spmm's x_layout=1)."""
    if x.dim() != 2 or not x.is_contiguous() or weight.numel() != x.shape[1] or not weight.is_contiguous():
        raise ValueError("x must be a contiguous [rows, width] tensor and weight [width]")
    if y is not None and (y.shape != x.shape or y.dtype != x.dtype or not y.is_contiguous()):
        raise ValueError("y must match x")
    if weight.dtype != x.dtype:
        raise ValueError("weight must have x's dtype")
    h, ld = _kmajor_image(x.shape[0], x.shape[1], x) if kmajor else (torch.empty_like(x), 0)
    x_out = torch.empty_like(x) if y is not None else x
    with torch.cuda.device(x.device):
        rc = _lib.lib().tl_add_rmsnorm(x.data_ptr(), y.data_ptr() if y is not None else None, weight.data_ptr(), _code(x.dtype, "x"),
                                       x.shape[0], x.shape[1], float(eps), x_out.data_ptr() if y is not None else None, h.data_ptr(),
                                       ld, _stream_ptr(x.device))
    _lib.check(rc)
    return x_out, (h[:, :x.shape[0]] if kmajor else h)


def silu_mul(gate_up, kmajor=False, pairs=False):
    """silu(gate_up[:, :w]) * gate_up[:, w:] for a contiguous [rows, 2 * w] tensor; with kmajor the transpose
    [w, rows] of that, a view of a K-major image (for spmm's x_layout=1).  pairs: gate and up of output j are
    columns 2j and 2j + 1 instead of j and w + j."""
    if gate_up.dim() != 2 or not gate_up.is_contiguous() or gate_up.shape[1] % 2:
        raise ValueError("gate_up must be a contiguous [rows, 2 * width] tensor")
    rows, w = gate_up.shape[0], gate_up.shape[1] // 2
    out, ld = _kmajor_image(rows, w, gate_up) if kmajor else (torch.empty((rows, w), dtype=gate_up.dtype, device=gate_up.device), 0)
    with torch.cuda.device(gate_up.device):
        call = _lib.lib().tl_silu_mul_pairs if pairs else _lib.lib().tl_silu_mul
        rc = call(gate_up.data_ptr(), _code(gate_up.dtype, "gate_up"), rows, w, out.data_ptr(), ld, _stream_ptr(gate_up.device))
    _lib.check(rc)
    return out[:, :rows] if kmajor else out
