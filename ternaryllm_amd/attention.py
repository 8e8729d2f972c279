"""LlamaTernaryAttention: four ternary projections around dense softmax attention, with the
constructor and the forward contract of the reference's module
(ternaryLLM_GPU/TernaryLLM/TernaryAttn.py:15-127).  The reference borrows rotary embedding,
repeat_kv and the KV cache from the `transformers` package; here the rotary embedding is a
textbook rotate-half RoPE, repeat_kv an expand, and the cache may be a `transformers` Cache
(anything with its `update(key, value, layer_idx, cache_kwargs)`) or a plain (k, v) tuple."""
import math

import torch
from torch import nn

from . import ops
from .linear import TernaryLinear
from .packing import PackedWeight


def side_by_side_key(device, projections):
    """What a weight built from several projections depends on: the device, each projection's packed buffer and
    scale (address and version, so that an assignment, an in-place edit or a state_dict load all count)."""
    key = [device]
    for p in projections:
        key += [p.w_packed.data_ptr(), p.w_packed._version]
        key += [None, None] if p.w_scale is None else [p.w_scale.data_ptr(), p.w_scale._version]
    return tuple(key)


def rope_tables(positions, head_dim, theta, dtype, device):
    """cos/sin of shape [len(positions), head_dim] for the rotate-half form of RoPE."""
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, device=device, dtype=torch.float32) / head_dim))
    ang = positions.to(torch.float32)[:, None] * inv[None, :]
    ang = torch.cat([ang, ang], dim=-1)
    return ang.cos().to(dtype), ang.sin().to(dtype)


def apply_rope(x, cos, sin):
    """x: [batch, heads, seq, head_dim]; cos/sin: [seq, head_dim] or [batch, seq, head_dim]."""
    half = x.shape[-1] // 2
    rot = torch.cat([-x[..., half:], x[..., :half]], dim=-1)
    if cos.dim() == 2:
        cos, sin = cos[None], sin[None]
    return x * cos[:, None] + rot * sin[:, None]


class LlamaTernaryAttention(nn.Module):
    def __init__(self, config, layer_idx=None, *, generator=None, reference_buffers=True, fused_qkv=True):
        """fused_qkv: multiply the hidden states by ONE packed weight that holds the columns of q_proj, k_proj and
        v_proj side by side (built from the three at the first forward on a device, and again when one of them
        changes; a fourth blob as large as the three together): one pass over the activations, one re-layout and one
        fix-up launch instead of three of each.  q_proj, k_proj and v_proj stay what the reference has there."""
        super().__init__()
        self.config = config
        self.fused_qkv = fused_qkv
        self._qkv = None  # (DeviceWeight, scale or None, key) of the side-by-side weight
        self.layer_idx = layer_idx
        self.hidden_size = config.hidden_size
        self.num_heads = config.num_attention_heads
        self.head_dim = getattr(config, "head_dim", None) or self.hidden_size // self.num_heads
        self.num_key_value_heads = config.num_key_value_heads
        self.num_key_value_groups = self.num_heads // self.num_key_value_heads
        self.max_position_embeddings = getattr(config, "max_position_embeddings", None)
        self.rope_theta = config.rope_theta
        self.attention_dropout = config.attention_dropout
        # The reference sets this and never reads it: it applies whatever mask the caller passes and none
        # when there is no mask (TernaryAttn.py:38,103-105).  Here a forward without a mask is causal
        # while this is True; set it to False for the reference's literal behaviour.
        self.is_causal = True

        def make(k, n):
            return TernaryLinear(k, n, sparsity=config.sparsity, uniform=config.uniform_sparsity,
                                 uniform_blk_size=config.uniform_sparsity_block_size, padding=config.padding,
                                 padding_size=config.padding_size, bias=config.attention_bias, generator=generator,
                                 reference_buffers=reference_buffers)

        self.q_proj = make(self.hidden_size, self.num_heads * self.head_dim)
        self.k_proj = make(self.hidden_size, self.num_key_value_heads * self.head_dim)
        self.v_proj = make(self.hidden_size, self.num_key_value_heads * self.head_dim)
        self.o_proj = make(self.num_heads * self.head_dim, self.hidden_size)

    def _qkv_weight(self, device):
        """q | k | v side by side as one packed weight on `device`."""
        projections = (self.q_proj, self.k_proj, self.v_proj)
        key = side_by_side_key(device, projections)
        if self._qkv is None or self._qkv[2] != key:
            both = torch.cat([p.ternary_weight for p in projections], dim=1).contiguous()
            scale = None
            given = [p.w_scale for p in projections if p.w_scale is not None]
            if given:  # a projection without a scale counts as one of ones, in the type of the first that has one
                scale = torch.cat([(p.w_scale if p.w_scale is not None else torch.ones(p.out_features, device=device)).to(device, given[0].dtype)
                                   for p in projections]).contiguous()
            self._qkv = (ops.DeviceWeight(PackedWeight.from_dense(both.numpy()), device), scale, key)
        return self._qkv[:2]

    def _rotary(self, position_ids, position_embeddings, q_len, past_len, dtype, device):
        if position_embeddings is not None:   # computed by the model, as newer `transformers` do
            cos, sin = position_embeddings
            return cos.to(dtype), sin.to(dtype)
        if position_ids is None:
            position_ids = torch.arange(past_len, past_len + q_len, device=device)
        if position_ids.dim() == 1:
            return rope_tables(position_ids, self.head_dim, self.rope_theta, dtype, device)
        cos, sin = rope_tables(position_ids.reshape(-1), self.head_dim, self.rope_theta, dtype, device)
        return cos.view(*position_ids.shape, -1), sin.view(*position_ids.shape, -1)

    def forward(self, hidden_states, attention_mask=None, position_ids=None, past_key_value=None, output_attentions=False,
                use_cache=False, cache_position=None, position_embeddings=None, *, position_offset=None, **kwargs):
        """The reference's signature and 3-tuple result (TernaryAttn.py:59-70,127):
        (attn_output [batch, seq, hidden], attn_weights or None, past_key_value).

        attention_mask: additive, broadcastable to [batch, heads, q_len, kv_len]; longer masks are cut to
        the key length as in the reference (:103-105).  position_embeddings: (cos, sin) of
        [batch or 1, q_len, head_dim], else they are computed from position_ids ([q_len] or
        [batch, q_len]), else from cache_position, else from the cache's length.  past_key_value: a `transformers` Cache (updated in
        place with `layer_idx`; newer versions pass it as `past_key_values`) or a (k, v) tuple of
        [batch, kv_heads, past, head_dim]; with a tuple, or with use_cache and no cache, the third
        result is the new (k, v) tuple.  position_offset: position of the first token when neither
        position_ids nor position_embeddings are given (default: the tuple cache's length)."""
        if past_key_value is None:
            past_key_value = kwargs.pop("past_key_values", None)
        bsz, q_len, _ = hidden_states.shape
        if self.fused_qkv and hidden_states.is_cuda:
            weight, scale = self._qkv_weight(hidden_states.device)
            nq, nkv = self.q_proj.out_features, self.k_proj.out_features
            qkv = ops.spmm(weight, hidden_states.reshape(bsz * q_len, -1), scale).view(bsz, q_len, nq + 2 * nkv)
            q, k, v = (t.reshape(bsz, q_len, -1, self.head_dim).transpose(1, 2) for t in qkv.split((nq, nkv, nkv), dim=-1))
        else:
            q = self.q_proj(hidden_states).view(bsz, q_len, -1, self.head_dim).transpose(1, 2)
            k = self.k_proj(hidden_states).view(bsz, q_len, -1, self.head_dim).transpose(1, 2)
            v = self.v_proj(hidden_states).view(bsz, q_len, -1, self.head_dim).transpose(1, 2)
        is_tuple = isinstance(past_key_value, (tuple, list))
        past_len = position_offset
        if past_len is None:
            if is_tuple:
                past_len = past_key_value[0].shape[2]
            elif cache_position is not None and torch.is_tensor(cache_position) and cache_position.numel() > 0:
                past_len = int(cache_position.reshape(-1)[0])   # the position of the first new token
            elif past_key_value is not None and hasattr(past_key_value, "get_seq_length"):
                past_len = int(past_key_value.get_seq_length(self.layer_idx))
            else:
                past_len = 0
        cos, sin = self._rotary(position_ids, position_embeddings, q_len, past_len, q.dtype, q.device)
        q, k = apply_rope(q, cos, sin), apply_rope(k, cos, sin)
        if is_tuple:
            k = torch.cat([past_key_value[0], k], dim=2)
            v = torch.cat([past_key_value[1], v], dim=2)
            past_key_value = (k, v)
        elif past_key_value is not None:
            k, v = past_key_value.update(k, v, self.layer_idx, {"sin": sin, "cos": cos, "cache_position": cache_position})
        elif use_cache:
            past_key_value = (k, v)
        kv_len = k.shape[2]
        if self.num_key_value_groups > 1:
            k = k.repeat_interleave(self.num_key_value_groups, dim=1)
            v = v.repeat_interleave(self.num_key_value_groups, dim=1)
        if attention_mask is not None:
            mask = attention_mask[..., :kv_len]
            if mask.dtype != torch.bool:
                mask = mask.to(q.dtype)
        elif self.is_causal and q_len > 1:
            # query i sits at key position kv_len - q_len + i
            mask = torch.ones((q_len, kv_len), dtype=torch.bool, device=q.device).tril(kv_len - q_len)
        else:
            mask = None
        dropout = self.attention_dropout if self.training else 0.0
        if output_attentions:
            # the reference's eager form (TernaryAttn.py:101-110): scores, fp32 softmax, weights returned
            scores = torch.matmul(q, k.transpose(2, 3)) / math.sqrt(self.head_dim)
            if mask is not None:
                scores = scores.masked_fill(~mask, float("-inf")) if mask.dtype == torch.bool else scores + mask
            attn_weights = torch.softmax(scores, dim=-1, dtype=torch.float32).to(q.dtype)
            attn = torch.matmul(nn.functional.dropout(attn_weights, p=dropout, training=self.training), v)
        else:
            attn_weights = None
            attn = nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=mask, dropout_p=dropout)
        attn = attn.transpose(1, 2).reshape(bsz, q_len, -1)
        return self.o_proj(attn), attn_weights, past_key_value


class TwoResultAttention(nn.Module):
    """Adapter for `transformers` releases whose decoder layer unpacks two results from `self_attn`
    (attn_output, attn_weights) and hands the cache over as `past_key_values`: wraps a LlamaTernaryAttention,
    which keeps the three results of the release the reference was written against (4.45)."""

    def __init__(self, attention):
        super().__init__()
        self.attention = attention

    def forward(self, *args, **kwargs):
        out = self.attention(*args, **kwargs)
        return out[0], out[1]


def collect_attn_linear_layers(model):
    """(name, module) of the nn.Linear attention projections under `model` (TernaryAttn.py:134-140)."""
    return [(name, m) for name, m in model.named_modules()
            if isinstance(m, nn.Linear) and any(tag in name for tag in ("q_proj", "k_proj", "v_proj", "o_proj"))]


def replace_linear_layers(layers, attn, sparsity=0.8, *, generator=None, reference_buffers=False):
    """Puts a random TernaryLinear of the same shape in the place of each listed projection of the
    attention module `attn` and moves it to the GPU (TernaryAttn.py:142-147; `layers` as returned by
    collect_attn_linear_layers(attn))."""
    for name, module in layers:
        ternary = TernaryLinear(module.in_features, module.out_features, sparsity, False, generator=generator,
                                reference_buffers=reference_buffers).to("cuda")
        parent_name, _, leaf = name.rpartition(".")
        setattr(attn.get_submodule(parent_name) if parent_name else attn, leaf, ternary)
    torch.cuda.empty_cache()


__all__ = ["LlamaTernaryAttention", "TwoResultAttention", "rope_tables", "apply_rope", "collect_attn_linear_layers",
           "replace_linear_layers"]
