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


def test_ternarize_threshold_and_from_weights():
    from ternaryllm_amd.linear import ternarize_threshold
    g = torch.Generator().manual_seed(3)
    w = torch.randn(200, 30, generator=g)
    t, scale = ternarize_threshold(w, sparsity=0.6)
    assert t.dtype == torch.int32 and set(t.unique().tolist()) <= {-1, 0, 1}
    assert (t == 0).float().mean(dim=0).sub(0.6).abs().max() < 0.02          # per column
    assert torch.equal(t[t != 0].sign(), w[t != 0].sign().to(torch.int32))
    # the scale is the least-squares one for the chosen support: <w, t> / <t, t> per column
    ls = (w * t).sum(0) / (t * t).sum(0).clamp(min=1)
    assert torch.allclose(scale, ls, atol=1e-6)
    # kept entries are the largest ones
    assert (w.abs() * (t == 0)).max(dim=0).values.le((w.abs() * (t != 0) + 1e9 * (t == 0)).min(dim=0).values).all()
    t2, _ = ternarize_threshold(w)                                           # 0.7 * mean |w| rule
    assert ((w.abs() > 0.7 * w.abs().mean(0, keepdim=True)) == (t2 != 0)).all()
    m = _Toy()
    cfg = TernaryConfig(sparsity=0.5)
    ref_w = m.layers[0].mlp.down_proj.weight.detach().clone()
    surgery.replace_linear_layers(surgery.collect_linear_layers(m, cfg), m, cfg, from_weights=True)
    mod = m.layers[0].mlp.down_proj
    assert isinstance(mod, TernaryLinear) and mod.w_scale is not None
    approx = mod.ternary_weight.float() * mod.w_scale[None, :]
    err = (approx - ref_w.t()).norm() / ref_w.norm()
    assert err < 0.6                                                          # a ternary fit of uniform weights, not noise
