"""Model surgery on a toy module tree with Llama's layer names (no GPU, no transformers)."""
import torch
from torch import nn

from ternaryllm_amd import TernaryConfig, TernaryLinear
from ternaryllm_amd import surgery


class _Attn(nn.Module):
    def __init__(self, h):
        super().__init__()
        self.q_proj, self.k_proj, self.v_proj, self.o_proj = (nn.Linear(h, h, bias=False) for _ in range(4))


class _Mlp(nn.Module):
    def __init__(self, h, i):
        super().__init__()
        self.gate_proj, self.up_proj, self.down_proj = nn.Linear(h, i, bias=False), nn.Linear(h, i, bias=False), nn.Linear(i, h, bias=False)


class _Layer(nn.Module):
    def __init__(self, h, i):
        super().__init__()
        self.self_attn, self.mlp = _Attn(h), _Mlp(h, i)


class _Toy(nn.Module):
    def __init__(self, h=64, i=96, layers=2, vocab=50):
        super().__init__()
        self.layers = nn.ModuleList(_Layer(h, i) for _ in range(layers))
        self.lm_head = nn.Linear(h, vocab, bias=False)


def test_collect_follows_the_configuration():
    m = _Toy()
    both = surgery.collect_linear_layers(m, TernaryConfig(ternary_attn_linear=True, ternary_mlp=True))
    assert len(both) == 2 * 7 and all("lm_head" not in n for n, _ in both)
    only_attn = surgery.collect_linear_layers(m, TernaryConfig(ternary_attn_linear=True, ternary_mlp=False))
    assert sorted(n.rsplit(".", 1)[1] for n, _ in only_attn) == sorted(["q_proj", "k_proj", "v_proj", "o_proj"] * 2)
    only_mlp = surgery.collect_linear_layers(m, TernaryConfig(ternary_attn_linear=False, ternary_mlp=True))
    assert len(only_mlp) == 6 and all(".mlp." in n for n, _ in only_mlp)
    assert [n for n, _ in surgery.collect_attn_linear_layers(m)] == [n for n, _ in only_attn]


def test_replace_keeps_shapes_and_sparsity():
    m = _Toy()
    cfg = TernaryConfig(sparsity=0.75)
    g = torch.Generator().manual_seed(7)
    surgery.replace_linear_layers(surgery.collect_linear_layers(m, cfg), m, cfg, generator=g)
    assert isinstance(m.lm_head, nn.Linear)
    for layer in m.layers:
        for mod, (k, n) in ((layer.self_attn.q_proj, (64, 64)), (layer.mlp.gate_proj, (64, 96)), (layer.mlp.down_proj, (96, 64))):
            assert isinstance(mod, TernaryLinear) and (mod.in_features, mod.out_features) == (k, n) and mod.bias is None
            w = mod.ternary_weight
            assert set(w.unique().tolist()) <= {-1, 0, 1}
            assert abs(float((w == 0).float().mean()) - 0.75) < 0.05
    # nothing is left to replace
    assert surgery.collect_linear_layers(m, cfg) == []


def test_add_padding_to_token():
    ids = torch.arange(10).reshape(2, 5)
    out = surgery.add_padding_to_token(ids, alignment_size=4, device="cpu", pad_token_id=99)
    assert out.shape == (2, 8) and out[:, 5:].eq(99).all() and out[:, :5].equal(ids)
    same = surgery.add_padding_to_token(torch.zeros(1, 8, dtype=torch.long), alignment_size=4, device="cpu", pad_token_id=1)
    assert same.shape == (1, 8)

    class Tok:
        pad_token, eos_token, pad_token_id = None, "</s>", 2
    assert surgery.add_padding_to_token(ids, Tok(), 4, "cpu")[0, -1] == 2
