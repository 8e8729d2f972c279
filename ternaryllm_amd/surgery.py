"""Model surgery: swap the nn.Linear layers of a Llama-style torch model for TernaryLinear, as the
reference's helpers do (ternaryLLM_GPU/TernaryLLM/TernaryLlama.py:10-75 and TernaryAttn.py:134-147).

Which layers are taken follows the reference: attention projections by name (q_proj, k_proj, v_proj,
o_proj) when `config.ternary_attn_linear`, every nn.Linear under a module whose qualified name contains
"mlp" when `config.ternary_mlp`.  The replacements are random ternary matrices of the configured
sparsity, as in the reference (it has no ternarisation of trained weights either,
TernaryLinear.py:19-20), without bias.  The model is any torch module tree; `transformers` is not needed.
"""
import torch
from torch import nn

from .attention import collect_attn_linear_layers  # noqa: F401  (TernaryAttn.py:134-140; re-exported here)
from .linear import TernaryLinear

_ATTN_NAMES = ("q_proj", "k_proj", "v_proj", "o_proj")


def collect_linear_layers(model, config):
    """(name, module) of every nn.Linear the configuration asks to replace (TernaryLlama.py:10-19).
    A layer that matches both rules is listed once."""
    picked = []
    for name, m in model.named_modules():
        if not isinstance(m, nn.Linear):
            continue
        attn = config.ternary_attn_linear and any(tag in name for tag in _ATTN_NAMES)
        mlp = config.ternary_mlp and "mlp" in name
        if attn or mlp:
            picked.append((name, m))
    return picked


def replace_linear_layers(layers, model, config, *, generator=None, reference_buffers=False, verbose=False,
                          from_weights=False):
    """Puts a TernaryLinear of the same shape in the place of each listed layer (TernaryLlama.py:21-36).
    `generator` seeds the random weights; `reference_buffers` also builds the reference's merged arrays.
    With `from_weights` the layer's own weight is ternarised instead (threshold at the configured
    sparsity's quantile per output channel, with the matching per-channel scale); the bias is dropped
    either way, as in the reference."""
    for name, module in layers:
        parent_name, _, leaf = name.rpartition(".")
        parent = model.get_submodule(parent_name) if parent_name else model
        if verbose:
            print(f"replacing {name}: {module.in_features} -> {module.out_features}")
        if from_weights:
            scale_dtype = module.weight.dtype if module.weight.dtype in (torch.float16, torch.float32) else torch.float32
            setattr(parent, leaf, TernaryLinear.from_float(module.weight.detach().t().float().cpu(), config.sparsity,
                                                           scale_dtype=scale_dtype))
            continue
        ternary = TernaryLinear(module.in_features, module.out_features, sparsity=config.sparsity,
                                uniform=config.uniform_sparsity, uniform_blk_size=config.uniform_sparsity_block_size,
                                padding=False, bias=False, device="cpu", generator=generator,
                                reference_buffers=reference_buffers)
        setattr(parent, leaf, ternary)
    return model


def prepare_ternary_model(model, config, device="cuda", **kwargs):
    """collect + replace on the CPU, then move the model to `device` (TernaryLlama.py:69-75)."""
    model.to("cpu")
    replace_linear_layers(collect_linear_layers(model, config), model, config, **kwargs)
    model.to(device)
    if torch.cuda.is_available():
        torch.cuda.empty_cache()
    return model


def add_padding_to_token(input_ids, tokenizer=None, alignment_size=4, device="cuda", pad_token_id=None):
    """Pads the sequence dimension of `input_ids` [batch, seq] to a multiple of `alignment_size` with the
    pad token and moves it to `device` (TernaryLlama.py:53-66).  The pad id comes from `tokenizer`
    (its eos token when it has no pad token, as the reference sets it) or from `pad_token_id`."""
    if pad_token_id is None:
        if tokenizer is None:
            raise ValueError("pass a tokenizer or pad_token_id")
        if tokenizer.pad_token is None:
            tokenizer.pad_token = tokenizer.eos_token
        pad_token_id = tokenizer.pad_token_id
    remainder = input_ids.size(1) % alignment_size
    if remainder:
        pad = torch.full((input_ids.size(0), alignment_size - remainder), pad_token_id, dtype=input_ids.dtype)
        input_ids = torch.cat((input_ids.cpu(), pad), dim=1)
    return input_ids.to(device)


__all__ = ["collect_attn_linear_layers", "collect_linear_layers", "replace_linear_layers", "prepare_ternary_model",
           "add_padding_to_token"]
