"""LlamaTernaryMLP: down(act(gate(x)) * up(x)) with three TernaryLinear
(ternaryLLM_GPU/TernaryLLM/TernaryMLP.py:11-35).  The gate and up products and the SiLU gate run as one
kernel pass over x: two weights walked side by side, or (paired=True) one weight whose columns are
(gate, up) pairs with the gate in the product's epilogue."""
import torch
from torch import nn

from . import ops
from .attention import side_by_side_key
from .linear import TernaryLinear
from .packing import PackedWeight


def activation_function(name):
    """The activation the reference looks up in transformers' ACT2FN (TernaryMLP.py:30): that table when the package
    is there, else the handful of torch functions Llama-style configurations name."""
    try:
        from transformers.activations import ACT2FN
        return ACT2FN[name]
    except (ImportError, KeyError):
        table = {"silu": torch.nn.functional.silu, "swish": torch.nn.functional.silu, "gelu": torch.nn.functional.gelu,
                 "relu": torch.nn.functional.relu, "gelu_new": lambda t: torch.nn.functional.gelu(t, approximate="tanh"),
                 "gelu_pytorch_tanh": lambda t: torch.nn.functional.gelu(t, approximate="tanh"), "tanh": torch.tanh,
                 "sigmoid": torch.sigmoid}
        if name not in table:
            raise ValueError(f"activation {name!r} unknown")
        return table[name]


class LlamaTernaryMLP(nn.Module):
    def __init__(self, config, *, generator=None, scales=None, reference_buffers=True, paired=False):
        """config: object with hidden_size, intermediate_size, sparsity, uniform_sparsity,
        uniform_sparsity_block_size, padding, padding_size, mlp_bias, hidden_act.
        scales: optional dict with 'gate', 'up', 'down' per-output-channel tensors.
        paired: multiply by one packed weight of 2 x intermediate_size columns, (gate, up) pairs side by side, built
        from the two projections at the first forward on a device (a third blob as large as the two together; the
        product is one plain launch over twice the columns, a few percent faster than the two-weight kernel)."""
        super().__init__()
        self.config = config
        self.paired = paired
        self._pairs = None  # (DeviceWeight, scale or None, what it was built from) of the paired weight
        self.hidden_size = config.hidden_size
        self.intermediate_size = config.intermediate_size
        # the fused kernels gate with SiLU; any other activation of the reference's table (TernaryMLP.py:30,
        # transformers' ACT2FN) runs as two products and the torch operator
        self.hidden_act = getattr(config, "hidden_act", "silu")
        scales = scales or {}

        def make(k, n, name):
            return TernaryLinear(k, n, sparsity=config.sparsity, uniform=config.uniform_sparsity,
                                 uniform_blk_size=config.uniform_sparsity_block_size, padding=config.padding,
                                 padding_size=config.padding_size, bias=config.mlp_bias, generator=generator,
                                 scale=scales.get(name), reference_buffers=reference_buffers)

        self.gate_proj = make(self.hidden_size, self.intermediate_size, "gate")
        self.up_proj = make(self.hidden_size, self.intermediate_size, "up")
        self.down_proj = make(self.intermediate_size, self.hidden_size, "down")
        self.act_fn = activation_function(self.hidden_act)

    def _paired_weight(self, device):
        """The (gate, up) pair weight on `device`: column 2j the gate, column 2j + 1 the up projection of output j."""
        # built again when the device, either projection's packed buffer or either scale changes (a move, an
        # assignment, an edit in place, a state_dict load)
        key = side_by_side_key(device, (self.gate_proj, self.up_proj))
        if self._pairs is None or self._pairs[2] != key:
            g, u = self.gate_proj.ternary_weight, self.up_proj.ternary_weight
            both = torch.empty((g.shape[0], 2 * g.shape[1]), dtype=torch.int32)
            both[:, 0::2], both[:, 1::2] = g, u
            scale = None
            given = [t for t in (self.gate_proj.w_scale, self.up_proj.w_scale) if t is not None]
            if given:  # a projection without a scale counts as one of ones, in the other's type
                ones = torch.ones(g.shape[1], dtype=given[0].dtype, device=device)
                sg = self.gate_proj.w_scale if self.gate_proj.w_scale is not None else ones
                su = self.up_proj.w_scale if self.up_proj.w_scale is not None else ones
                scale = torch.stack([sg.to(device), su.to(device).to(sg.dtype)], 1).reshape(-1).contiguous()
            self._pairs = (ops.DeviceWeight(PackedWeight.from_dense(both.numpy()), device), scale, key)
        return self._pairs[:2]

    def forward(self, x):
        lead = x.shape[:-1]
        x2 = x.reshape(-1, self.hidden_size)
        if self.hidden_act not in ("silu", "swish"):
            h = self.act_fn(self.gate_proj(x2)) * self.up_proj(x2)
            return self.down_proj(h).reshape(*lead, self.hidden_size)
        if self.paired:
            weight, scale = self._paired_weight(x2.device)
            h = ops.spmm_gated(weight, x2, scale)
        else:
            h = ops.mlp_gate_up(self.gate_proj.device_weight(), self.up_proj.device_weight(), x2, self.gate_proj.w_scale,
                                self.up_proj.w_scale)
        return self.down_proj(h).reshape(*lead, self.hidden_size)


__all__ = ["LlamaTernaryMLP"]
