"""TernaryConfig: the ternary knobs of the reference's configuration class
(ternaryLLM_GPU/TernaryLLM/configuration_ternary.py:28-47) on a plain Llama-shaped config.
It does not derive from transformers.LlamaConfig: the modules here only read attributes."""
from dataclasses import dataclass


@dataclass
class TernaryConfig:
    hidden_size: int = 4096
    intermediate_size: int = 11008
    num_hidden_layers: int = 32
    num_attention_heads: int = 32
    num_key_value_heads: int = 32
    vocab_size: int = 32000
    max_position_embeddings: int = 4096
    rms_norm_eps: float = 1e-5
    rope_theta: float = 10000.0
    hidden_act: str = "silu"
    attention_bias: bool = False
    attention_dropout: float = 0.0
    mlp_bias: bool = False
    # ternary knobs, names as in the reference
    ternary_attn_linear: bool = True
    ternary_mlp: bool = True
    sparsity: float = 0.8
    uniform_sparsity: bool = False
    uniform_sparsity_block_size: int = 512
    padding: bool = False
    padding_size: int = 4

    @property
    def head_dim(self):
        return self.hidden_size // self.num_attention_heads
