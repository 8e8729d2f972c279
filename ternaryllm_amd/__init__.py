"""MI355X-native ternary sparse GEMM behind the ternaryLLM extension API.

The exports mirror ternaryLLM_GPU/TernaryLLM/__init__.py.  Everything that computes goes
through libternary_spmm.so (built in-tree by ternaryllm_amd.build); there is no fallback."""
from .config import TernaryConfig
from .linear import TernaryLinear, random_ternary_weights, convert_ternary_weights, MapKSizeToTileSize
from .mlp import LlamaTernaryMLP
from .attention import LlamaTernaryAttention
from .llama import TernaryLlamaDecoder

__all__ = ["TernaryLinear", "LlamaTernaryMLP", "LlamaTernaryAttention", "TernaryConfig", "TernaryLlamaDecoder",
           "random_ternary_weights", "convert_ternary_weights", "MapKSizeToTileSize"]
