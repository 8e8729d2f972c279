"""TernaryLinear: the reference's module (ternaryLLM_GPU/TernaryLLM/TernaryLinear.py:115-182) on
top of the gfx950 library.  Constructor arguments, buffer names and the forward contract are
the reference's; additions are keyword-only."""
import numpy as np
import torch
from torch import nn

from . import ops, packing

# K -> tile height of the merged format, TernaryLinear.py:9-16.  The reference raises KeyError for
# any other K (e.g. 11008); here other sizes take the largest listed height that divides K, else 256.
MapKSizeToTileSize = {8192: 512, 4096: 512, 3072: 512, 2048: 256, 1024: 256, 512: 64}


def merged_tile_size(k):
    if k in MapKSizeToTileSize:
        return MapKSizeToTileSize[k]
    for t in (512, 256, 64):
        if k % t == 0:
            return t
    return 256


def ternarize_weights(w):
    raise NotImplementedError("ternarize_weights not implement")  # as in the reference, TernaryLinear.py:19-20


def ternarize_threshold(w, sparsity=None):
    """Ternarises a float weight [K, N] column by column: an entry becomes sign(w) where |w| exceeds the
    column's threshold, else 0, and each column gets the scale that minimises the squared error for that
    support, mean |w| over the kept entries.  The threshold is 0.7 * mean |w| of the column (the classic
    ternary-weight rule) or, with `sparsity` given, the column's `sparsity` quantile of |w|, so that about
    that fraction of each column is zero.  Returns (int32 [K, N] in {-1, 0, 1}, float32 scale [N]).
    The reference has no counterpart (its ternarize_weights raises); random weights stay the default."""
    w = torch.as_tensor(w, dtype=torch.float32)
    mag = w.abs()
    if sparsity is None:
        thr = 0.7 * mag.mean(dim=0, keepdim=True)
    else:
        if not 0.0 <= sparsity < 1.0:
            raise ValueError("sparsity must be in [0, 1)")
        thr = torch.quantile(mag, sparsity, dim=0, keepdim=True)
    keep = mag > thr
    t = (torch.sign(w) * keep).to(torch.int32)
    kept = keep.sum(dim=0).clamp(min=1)
    scale = (mag * keep).sum(dim=0) / kept
    return t, scale


def random_ternary_weights(size, sparsity=0.8, uniform=False, block_size=512, generator=None):
    """Random ternary [K, N] int32 matrix, distributed as the reference's generator
    (TernaryLinear.py:23-85).  i.i.d. mode: r ~ U[0,1); r < s -> 0, s <= r < (s+1)/2 -> -1, else +1.
    uniform mode: the flattened [N, K] matrix is cut into blocks of `block_size`; every block gets the
    same even number of non-zeros (plus 2 for the first few to reach the total), half +1 half -1, at
    random positions.  `generator` (a CPU torch.Generator) makes the draw reproducible."""
    K, N = int(size[0]), int(size[1])
    if not uniform:
        r = torch.rand((K, N), generator=generator)
        w = torch.zeros((K, N), dtype=torch.int32)
        w[(r >= sparsity) & (r < (sparsity + 1) / 2)] = -1
        w[r >= (sparsity + 1) / 2] = 1
        return w
    total = K * N
    n_blocks = total // block_size
    if n_blocks == 0:
        raise ValueError("block_size exceeds the matrix")
    nnz = int(total * (1 - sparsity))
    nnz -= nnz % 2
    per_block = (nnz // n_blocks) // 2 * 2
    counts = torch.full((n_blocks,), per_block, dtype=torch.int64)
    extra = (nnz - per_block * n_blocks) // 2
    if extra > 0:
        reps = torch.arange(extra) % n_blocks
        counts += 2 * torch.bincount(reps, minlength=n_blocks)
    if int(counts.max()) > block_size:
        raise ValueError("sparsity too low for this block size")
    # rank of a random key inside each block = a random permutation of its positions
    keys = torch.rand((n_blocks, block_size), generator=generator)
    rank = keys.argsort(dim=1).argsort(dim=1)
    half = (counts // 2).unsqueeze(1)
    blocks = torch.zeros((n_blocks, block_size), dtype=torch.int32)
    blocks[rank < half] = 1
    blocks[(rank >= half) & (rank < 2 * half)] = -1
    flat = torch.zeros(total, dtype=torch.int32)
    flat[: n_blocks * block_size] = blocks.reshape(-1)
    return flat.view(N, K).T.contiguous()


def convert_ternary_weights(w, padding=False, padding_size=4, dtype=torch.int32, device="cpu"):
    """Merged tiled-CSC arrays of a ternary weight: (row_indices, col_offsets, col_tile_indices),
    as the reference's helper of the same name (TernaryLinear.py:87-113)."""
    w_ = w.detach().to("cpu", torch.int32).contiguous()
    cnt_pos, cnt_neg = packing.count_nnz(w_)
    k, n = w_.shape
    merged = packing.convert_to_ter_tiled_mcsc(w_, n, k, cnt_pos, cnt_neg, merged_tile_size(k), padding, padding_size)
    row_indices = torch.from_numpy(merged[0]).to(device).contiguous().to(dtype)
    col_offsets = torch.from_numpy(merged[1]).to(device).contiguous()
    col_tile_indices = torch.from_numpy(merged[2]).to(device).contiguous().to(dtype)
    return row_indices, col_offsets, col_tile_indices


class TernaryLinear(nn.Module):
    """y = x @ W (* scale) for a ternary W, W generated at random as in the reference.

    Reference arguments: in_features (K), out_features (N), sparsity, uniform, uniform_blk_size,
    padding, padding_size, bias, device, dtype.  As in the reference the bias is allocated but never
    added (TernaryLinear.py:137-140, :152-182).
    Keyword-only additions: `weight` (use this int32 [K, N] ternary matrix instead of a random one),
    `scale` (per-output-channel factor, [N]), `generator` (seed for the random weight),
    `reference_buffers` (also build the reference's merged arrays; they are not used by forward).
    """
    __constants__ = ["in_features", "out_features"]

    def __init__(self, in_features, out_features, sparsity=0.8, uniform=False, uniform_blk_size=512, padding=False,
                 padding_size=4, bias=True, device=None, dtype=torch.int32, *, weight=None, scale=None, generator=None,
                 reference_buffers=True):
        super().__init__()
        if bias:
            self.bias = nn.Parameter(torch.zeros(out_features, device=device), requires_grad=False)
        else:
            self.register_parameter("bias", None)
        if weight is None:
            weight = random_ternary_weights((in_features, out_features), sparsity, uniform, uniform_blk_size, generator)
        else:
            weight = torch.as_tensor(weight).to("cpu", torch.int32).contiguous()
            if tuple(weight.shape) != (in_features, out_features):
                raise ValueError(f"weight must be [{in_features}, {out_features}]")
        self._dense = weight  # kept on the CPU, as the reference's `ternary_weight` attribute
        if reference_buffers:
            rows, offs, tiles = convert_ternary_weights(weight, padding=padding, padding_size=padding_size, device=device,
                                                        dtype=torch.int16)
        else:
            rows, offs, tiles = (torch.zeros(0, dtype=torch.int16, device=device), torch.zeros(0, dtype=torch.int32, device=device),
                                 torch.zeros(0, dtype=torch.int16, device=device))
        self.register_buffer("w_row_indices", rows, False)
        self.register_buffer("w_col_offsets", offs, False)
        self.register_buffer("w_col_tile_indices", tiles, False)
        packed = packing.PackedWeight.from_dense(weight)
        self._header = packed.header
        self._packed_nnz = packed.nnz
        self.register_buffer("w_packed", torch.from_numpy(packed.blob.copy()).to(device), True)
        if scale is not None:
            scale = torch.as_tensor(scale).reshape(-1)
            if scale.numel() != out_features:
                raise ValueError("scale must have out_features elements")
            self.register_buffer("w_scale", scale.to(device).contiguous(), True)
        else:
            self.w_scale = None
        self.in_features = in_features
        self.out_features = out_features
        self.uniform = uniform
        self.padding = padding
        self._handle = None

    @classmethod
    def from_float(cls, weight, sparsity=None, device=None, scale_dtype=torch.float32):
        """A module that approximates x @ weight for a float weight [K, N] (note: nn.Linear stores the
        transpose): ternarised by ternarize_threshold, with its per-column scale."""
        t, scale = ternarize_threshold(weight, sparsity)
        self = cls.from_packed(packing.PackedWeight.from_dense(t), scale.to(scale_dtype), device=device)
        self._dense = t
        return self

    @classmethod
    def from_packed(cls, packed, scale=None, device=None):
        """A module around an existing PackedWeight: no random draw, no dense copy kept, no bias and
        none of the reference's merged arrays (`ternary_weight` decodes the blob on demand)."""
        self = cls.__new__(cls)
        nn.Module.__init__(self)
        self.register_parameter("bias", None)
        empty16 = torch.zeros(0, dtype=torch.int16, device=device)
        self.register_buffer("w_row_indices", empty16, False)
        self.register_buffer("w_col_offsets", torch.zeros(0, dtype=torch.int32, device=device), False)
        self.register_buffer("w_col_tile_indices", empty16.clone(), False)
        self._dense = None
        self._header = packed.header
        self._packed_nnz = packed.nnz
        self.register_buffer("w_packed", torch.from_numpy(packed.blob).to(device), True)
        if scale is not None:
            scale = torch.as_tensor(scale).reshape(-1)
            if scale.numel() != packed.columns:
                raise ValueError("scale must have out_features elements")
            self.register_buffer("w_scale", scale.to(device).contiguous(), True)
        else:
            self.w_scale = None
        self.in_features = packed.inners
        self.out_features = packed.columns
        self.uniform = False
        self.padding = False
        self._handle = None
        return self

    @property
    def ternary_weight(self):
        """The dense int32 [K, N] weight on the CPU (decoded from the packed blob after a state_dict load)."""
        if self._dense is None:
            pw = packing.PackedWeight(self.w_packed.detach().cpu().numpy())
            self._dense = torch.from_numpy(pw.to_dense())
        return self._dense

    def _load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
        # a packed weight has its own length: take the incoming blob's size before the generic copy
        blob = state_dict.get(prefix + "w_packed")
        if blob is not None:
            pw = packing.PackedWeight(blob.detach().cpu().numpy())
            if (pw.inners, pw.columns) != (self.in_features, self.out_features):
                raise ValueError(f"packed weight is {pw.inners}x{pw.columns}, module is {self.in_features}x{self.out_features}")
            pw.validate()
            self.w_packed = torch.empty(blob.shape, dtype=torch.uint8, device=self.w_packed.device)
            self._header = pw.header
            self._packed_nnz = pw.nnz
            self._dense = None
            self._handle = None
        super()._load_from_state_dict(state_dict, prefix, *args, **kwargs)

    def device_weight(self):
        """The DeviceWeight view of `w_packed` on its current device."""
        h = self._handle
        if h is None or h.blob.data_ptr() != self.w_packed.data_ptr():
            h = ops.DeviceWeight.__new__(ops.DeviceWeight)
            h.header = self._header
            h.blob = self.w_packed
            if h.blob.device.type != "cuda":
                raise RuntimeError("TernaryLinear runs on a GPU only: call .to('cuda') first")
            self._handle = h
        return h

    def forward(self, input):
        """input: (batch, rows, K), (rows, K) or (K,) -- also (batch, K, rows) as the reference kernel
        reads it; returns (batch, rows, N) / (rows, N) / (N,) in the input dtype."""
        if input.dim() > 3:
            raise AssertionError("Input has dim larger than 3")  # the reference asserts (TernaryLinear.py:161)
        w = self.device_weight()
        K, N = self.in_features, self.out_features
        if input.shape[-1] == K:
            lead = input.shape[:-1]
            y = ops.spmm(w, input.reshape(-1, K), self.w_scale)
            return y.reshape(*lead, N)
        if input.dim() >= 2 and input.shape[-2] == K:  # K-major activations
            if input.dim() == 2:
                return ops.spmm(w, input, self.w_scale, x_layout=1)
            return ops.spmm_kmajor_batch(w, input, self.w_scale)
        raise ValueError(f"input of shape {tuple(input.shape)} does not match in_features={K}")

    def extra_repr(self):
        return f"in_features={self.in_features}, out_features={self.out_features}, nnz={self._packed_nnz}"


__all__ = ["TernaryLinear", "random_ternary_weights", "convert_ternary_weights", "MapKSizeToTileSize",
           "ternarize_weights", "ternarize_threshold"]
