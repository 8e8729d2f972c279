"""LlamaTernaryMLP: down(act(gate(x)) * up(x)) with three TernaryLinear
(ternaryLLM_GPU/TernaryLLM/TernaryMLP.py:11-35).  For more than 48 token rows the gate and up
products and the SiLU-gate run as one fused kernel pass over x."""
import torch
from torch import nn

from . import ops
from .linear import TernaryLinear


class LlamaTernaryMLP(nn.Module):
    def __init__(self, config, *, generator=None, scales=None, reference_buffers=True):
        """config: object with hidden_size, intermediate_size, sparsity, uniform_sparsity,
        uniform_sparsity_block_size, padding, padding_size, mlp_bias, hidden_act.
        scales: optional dict with 'gate', 'up', 'down' per-output-channel tensors."""
        super().__init__()
        self.config = config
        self.hidden_size = config.hidden_size
        self.intermediate_size = config.intermediate_size
        if config.hidden_act != "silu":
            raise ValueError("only the SiLU gate of Llama is supported")
        scales = scales or {}

        def make(k, n, name):
            return TernaryLinear(k, n, sparsity=config.sparsity, uniform=config.uniform_sparsity,
                                 uniform_blk_size=config.uniform_sparsity_block_size, padding=config.padding,
                                 padding_size=config.padding_size, bias=config.mlp_bias, generator=generator,
                                 scale=scales.get(name), reference_buffers=reference_buffers)

        self.gate_proj = make(self.hidden_size, self.intermediate_size, "gate")
        self.up_proj = make(self.hidden_size, self.intermediate_size, "up")
        self.down_proj = make(self.intermediate_size, self.hidden_size, "down")
        self.act_fn = torch.nn.functional.silu

    def forward(self, x):
        lead = x.shape[:-1]
        x2 = x.reshape(-1, self.hidden_size)
        h = ops.mlp_gate_up(self.gate_proj.device_weight(), self.up_proj.device_weight(), x2, self.gate_proj.w_scale,
                            self.up_proj.w_scale)
        return self.down_proj(h).reshape(*lead, self.hidden_size)


__all__ = ["LlamaTernaryMLP"]
