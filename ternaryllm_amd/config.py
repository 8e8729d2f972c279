"""TernaryConfig: the reference's configuration class (ternaryLLM_GPU/TernaryLLM/configuration_ternary.py:3-47) --
a `transformers` LlamaConfig with the ternary knobs on top, so that it can be handed to a `transformers` model,
saved and loaded with one.  Arguments go by keyword (the reference forwards 23 positional arguments, which only the
release it was written against takes in that order).  Without the `transformers` package a plain dataclass with
the same fields and defaults stands in: the modules here only read attributes."""
from dataclasses import dataclass

try:  # the package is optional: nothing on the product path needs it
    from transformers.models.llama.configuration_llama import LlamaConfig
except Exception:  # noqa: BLE001 - absent, or a release that does not import here
    LlamaConfig = None

def _rope_theta_of(config, default=10000.0):
    params = getattr(config, "rope_parameters", None) or {}
    return float(params.get("rope_theta", default)) if isinstance(params, dict) else default


if LlamaConfig is None:
    @dataclass
    class TernaryConfig:
        vocab_size: int = 32000
        hidden_size: int = 4096
        intermediate_size: int = 11008
        num_hidden_layers: int = 32
        num_attention_heads: int = 32
        num_key_value_heads: int = None
        hidden_act: str = "silu"
        max_position_embeddings: int = 2048
        rms_norm_eps: float = 1e-6
        rope_theta: float = 10000.0
        attention_bias: bool = False
        attention_dropout: float = 0.0
        mlp_bias: bool = False
        head_dim: int = None
        # ternary knobs, names as in the reference
        ternary_attn_linear: bool = True
        ternary_mlp: bool = True
        sparsity: float = 0.8
        uniform_sparsity: bool = False
        uniform_sparsity_block_size: int = 512
        padding: bool = False
        padding_size: int = 4

        def __post_init__(self):
            if self.num_key_value_heads is None:
                self.num_key_value_heads = self.num_attention_heads
            if self.head_dim is None:
                self.head_dim = self.hidden_size // self.num_attention_heads

elif hasattr(LlamaConfig, "__dataclass_fields__"):
    # releases whose configurations declare their fields (5.x): the knobs are further fields, and the rotary base,
    # which those releases keep inside `rope_parameters`, stays readable under the name the reference's modules use
    from huggingface_hub.dataclasses import strict

    @strict
    class TernaryConfig(LlamaConfig):
        ternary_attn_linear: bool = True
        ternary_mlp: bool = True
        sparsity: float = 0.8
        uniform_sparsity: bool = False
        uniform_sparsity_block_size: int = 512
        padding: bool = False
        padding_size: int = 4

        @property
        def rope_theta(self):
            return _rope_theta_of(self)

        @rope_theta.setter
        def rope_theta(self, value):
            params = dict(getattr(self, "rope_parameters", None) or {"rope_type": "default"})
            params["rope_theta"] = float(value)
            self.rope_parameters = params

else:
    class TernaryConfig(LlamaConfig):
        """(releases with hand-written constructors, 4.x: every Llama argument by keyword)"""

        def __init__(self, ternary_attn_linear=True, ternary_mlp=True, sparsity=0.8, uniform_sparsity=False,
                     uniform_sparsity_block_size=512, padding=False, padding_size=4, **kwargs):
            super().__init__(**kwargs)
            self.ternary_attn_linear = ternary_attn_linear
            self.ternary_mlp = ternary_mlp
            self.sparsity = sparsity
            self.uniform_sparsity = uniform_sparsity
            self.uniform_sparsity_block_size = uniform_sparsity_block_size
            self.padding = padding
            self.padding_size = padding_size
            if getattr(self, "head_dim", None) is None:
                self.head_dim = self.hidden_size // self.num_attention_heads


__all__ = ["TernaryConfig"]
