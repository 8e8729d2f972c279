"""LlamaTernaryAttention: four ternary projections around dense causal attention
(ternaryLLM_GPU/TernaryLLM/TernaryAttn.py:15-127).  The reference borrows rotary embedding,
repeat_kv and the KV cache from the `transformers` package; here they are a textbook RoPE, an
expand, and a plain (k, v) tuple, and the softmax attention is torch's
scaled_dot_product_attention."""
import torch
from torch import nn

from .linear import TernaryLinear


def rope_tables(positions, head_dim, theta, dtype, device):
    """cos/sin of shape [len(positions), head_dim] for the rotate-half form of RoPE."""
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, device=device, dtype=torch.float32) / head_dim))
    ang = positions.to(torch.float32)[:, None] * inv[None, :]
    ang = torch.cat([ang, ang], dim=-1)
    return ang.cos().to(dtype), ang.sin().to(dtype)


def apply_rope(x, cos, sin):
    """x: [batch, heads, seq, head_dim]."""
    half = x.shape[-1] // 2
    rot = torch.cat([-x[..., half:], x[..., :half]], dim=-1)
    return x * cos[None, None] + rot * sin[None, None]


class LlamaTernaryAttention(nn.Module):
    def __init__(self, config, layer_idx=None, *, generator=None, reference_buffers=True):
        super().__init__()
        self.config = config
        self.layer_idx = layer_idx
        self.hidden_size = config.hidden_size
        self.num_heads = config.num_attention_heads
        self.head_dim = self.hidden_size // self.num_heads
        self.num_key_value_heads = config.num_key_value_heads
        self.num_key_value_groups = self.num_heads // self.num_key_value_heads
        self.rope_theta = config.rope_theta
        self.attention_dropout = config.attention_dropout

        def make(k, n):
            return TernaryLinear(k, n, sparsity=config.sparsity, uniform=config.uniform_sparsity,
                                 uniform_blk_size=config.uniform_sparsity_block_size, padding=config.padding,
                                 padding_size=config.padding_size, bias=config.attention_bias, generator=generator,
                                 reference_buffers=reference_buffers)

        self.q_proj = make(self.hidden_size, self.num_heads * self.head_dim)
        self.k_proj = make(self.hidden_size, self.num_key_value_heads * self.head_dim)
        self.v_proj = make(self.hidden_size, self.num_key_value_heads * self.head_dim)
        self.o_proj = make(self.num_heads * self.head_dim, self.hidden_size)

    def forward(self, hidden_states, past_key_value=None, position_offset=0, use_cache=False):
        """hidden_states: [batch, seq, hidden]; past_key_value: optional (k, v) of
        [batch, kv_heads, past, head_dim].  Returns (output, present) with present = (k, v) or None."""
        bsz, q_len, _ = hidden_states.shape
        q = self.q_proj(hidden_states).view(bsz, q_len, self.num_heads, self.head_dim).transpose(1, 2)
        k = self.k_proj(hidden_states).view(bsz, q_len, self.num_key_value_heads, self.head_dim).transpose(1, 2)
        v = self.v_proj(hidden_states).view(bsz, q_len, self.num_key_value_heads, self.head_dim).transpose(1, 2)
        pos = torch.arange(position_offset, position_offset + q_len, device=hidden_states.device)
        cos, sin = rope_tables(pos, self.head_dim, self.rope_theta, q.dtype, q.device)
        q, k = apply_rope(q, cos, sin), apply_rope(k, cos, sin)
        if past_key_value is not None:
            k = torch.cat([past_key_value[0], k], dim=2)
            v = torch.cat([past_key_value[1], v], dim=2)
        present = (k, v) if use_cache else None
        if self.num_key_value_groups > 1:
            k = k.repeat_interleave(self.num_key_value_groups, dim=1)
            v = v.repeat_interleave(self.num_key_value_groups, dim=1)
        causal = past_key_value is None and q_len > 1
        if past_key_value is not None and q_len > 1:
            raise ValueError("a multi-token step on top of a cache is not supported")
        attn = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=causal)
        attn = attn.transpose(1, 2).reshape(bsz, q_len, self.num_heads * self.head_dim)
        return self.o_proj(attn), present


__all__ = ["LlamaTernaryAttention", "rope_tables", "apply_rope"]
