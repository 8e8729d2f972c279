"""MI355X-native ternary sparse GEMM behind the ternaryLLM extension API.

The exports mirror ternaryLLM_GPU/TernaryLLM/__init__.py.  Everything that computes goes
through libternary_spmm.so (built in-tree by ternaryllm_amd.build); there is no fallback."""
from .config import TernaryConfig
from .linear import TernaryLinear, random_ternary_weights, convert_ternary_weights, MapKSizeToTileSize
from .mlp import LlamaTernaryMLP
from .attention import LlamaTernaryAttention
from .llama import TernaryLlamaDecoder
from .surgery import (collect_linear_layers, replace_linear_layers, prepare_ternary_model, add_padding_to_token,
                      collect_attn_linear_layers)

__all__ = ["TernaryLinear", "LlamaTernaryMLP", "LlamaTernaryAttention", "TernaryConfig", "TernaryLlamaDecoder", "collect_linear_layers", "replace_linear_layers",
           "prepare_ternary_model", "add_padding_to_token", "collect_attn_linear_layers",
           "random_ternary_weights", "convert_ternary_weights", "MapKSizeToTileSize"]
