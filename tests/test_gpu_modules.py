"""GPU tests of the drop-in layer: ter_spmm.ter_spmm on merged arrays, TernaryLinear, the fused
MLP block and the attention block, against the CPU oracle / a plain torch fp32 restatement."""
import numpy as np
import pytest
import torch

from tests.util import FP16_TOL, FP32_TOL, activations, max_rel_err, ternary_weight

pytestmark = pytest.mark.gpu


def test_ter_spmm_drop_in_on_merged_arrays(cuda, oracle):
    """The reference call sequence: pack with convert_to_ter_tiled_mcsc, narrow to int16, call ter_spmm.
    The result must equal the oracle's walk of those merged arrays (what the format encodes)."""
    import ter_spmm
    K, N, tk = 1024, 96, 256
    w = ternary_weight(K, N, 0.8, 41)
    wt = torch.from_numpy(w)
    cp, cn = (wt == 1).sum().item(), (wt == -1).sum().item()
    tm = ter_spmm.convert_to_ter_tiled_mcsc(wt, N, K, cp, cn, tk, False, 4)
    rows = torch.tensor(np.array(tm[0]), dtype=torch.int32).to(torch.int16).to(cuda)
    offs = torch.tensor(np.array(tm[1]), dtype=torch.int32).to(cuda)
    tiles = torch.tensor(np.array(tm[2]), dtype=torch.int32).to(torch.int16).to(cuda)
    for bs, M in ((1, 1), (2, 8), (3, 70)):
        x = activations(bs * M, K, 42 + M, torch.float32, integer=True).reshape(bs, M, K)
        y = ter_spmm.ter_spmm(x.to(cuda), rows, offs, tiles, bs, M, N, K, False, False)
        assert y.shape == (bs, M, N) and y.dtype == torch.float32
        ref = oracle.mcsc_product(x.reshape(-1, K).numpy(), tm[0], tm[1], N, tk).reshape(bs, M, N)
        assert np.array_equal(y.cpu().numpy().astype(np.float64), ref)
        # the layout the reference kernel itself reads: [batch, K, M]
        yk = ter_spmm.ter_spmm(x.transpose(1, 2).contiguous().to(cuda), rows, offs, tiles, bs, M, N, K, False, False)
        assert np.array_equal(yk.cpu().numpy().astype(np.float64), ref)
    empty = ter_spmm.ter_spmm(torch.zeros(4, K, device=cuda), rows, offs, tiles, 0, 4, N, K, False, False)
    assert empty.shape == (0, 4, N)  # what the reference returns for a 2-D input (batch_size = 0)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, FP32_TOL), (torch.float16, FP16_TOL)])
def test_ternary_linear_forward_shapes_and_values(cuda, oracle, dtype, tol):
    from ternaryllm_amd import TernaryLinear
    g = torch.Generator().manual_seed(3)
    K, N = 768, 320
    scale = (0.5 + torch.rand(N, generator=g)).to(dtype)
    lin = TernaryLinear(K, N, sparsity=0.7, bias=False, generator=g, scale=scale).to(cuda)
    w = lin.ternary_weight.numpy()
    for shape in ((K,), (5, K), (2, 3, K), (4, 100, K)):
        x = torch.randn(shape, generator=g).to(dtype)
        y = lin(x.to(cuda))
        assert y.shape == shape[:-1] + (N,) and y.dtype == dtype
        x2 = x.reshape(-1, K).double().numpy()
        ref = oracle.fast_product(x2, w) * scale.double().numpy()[None, :]
        assert max_rel_err(y.reshape(-1, N).float().cpu().numpy(), ref, x2, w) <= tol
    with pytest.raises(AssertionError):
        lin(torch.zeros(1, 1, 1, K, device=cuda, dtype=dtype))
    with pytest.raises(ValueError):
        lin(torch.zeros(2, K + 1, device=cuda, dtype=dtype))
    # state_dict carries the packed weight; a fresh module loaded from it computes the same
    lin2 = TernaryLinear(K, N, sparsity=0.7, bias=False, scale=torch.ones(N, dtype=dtype)).to(cuda)
    lin2.load_state_dict(lin.state_dict())
    assert torch.equal(lin2.ternary_weight, lin.ternary_weight)
    x = torch.randn((7, K), generator=g).to(dtype).to(cuda)
    assert torch.equal(lin(x), lin2(x))


def _torch_mlp_reference(mlp, x):
    """Plain fp32 restatement of down(silu(gate(x)) * up(x)) with dense weights and the modules' scales."""
    def dense(lin):
        w = lin.ternary_weight.double()
        s = lin.w_scale.double().cpu() if lin.w_scale is not None else torch.ones(w.shape[1], dtype=torch.float64)
        return w, s
    wg, sg = dense(mlp.gate_proj)
    wu, su = dense(mlp.up_proj)
    wd, sd = dense(mlp.down_proj)
    xd = x.double()
    h = torch.nn.functional.silu((xd @ wg) * sg) * ((xd @ wu) * su)
    return h, (h @ wd) * sd


@pytest.mark.parametrize("tokens", [4, 200])
def test_mlp_block_fp16(cuda, tokens):
    from ternaryllm_amd import LlamaTernaryMLP, TernaryConfig, ops
    g = torch.Generator().manual_seed(8)
    cfg = TernaryConfig(hidden_size=512, intermediate_size=1408, sparsity=0.8)
    sc = {"gate": (0.5 + torch.rand(1408, generator=g)).half(), "up": (0.5 + torch.rand(1408, generator=g)).half(),
          "down": (0.5 + torch.rand(512, generator=g)).half()}
    mlp = LlamaTernaryMLP(cfg, generator=g, scales=sc).to(cuda)
    x = (0.05 * torch.randn((tokens, 512), generator=g)).half()
    h_ref, y_ref = _torch_mlp_reference(mlp, x)
    h = ops.mlp_gate_up(mlp.gate_proj.device_weight(), mlp.up_proj.device_weight(), x.to(cuda), mlp.gate_proj.w_scale,
                        mlp.up_proj.w_scale)
    # the fused gate/up output is fp16: one rounding of h on top of fp32 accumulation
    err_h = (h.double().cpu() - h_ref).abs() / h_ref.abs().clamp_min(h_ref.abs().mean())
    assert err_h.max().item() <= FP16_TOL
    y = mlp(x.to(cuda).reshape(1, tokens, 512))
    assert y.shape == (1, tokens, 512) and y.dtype == torch.float16
    # y carries the rounding of h (fp16) through ~280 signed adds per output: compare on the output's RMS scale
    err_y = (y[0].double().cpu() - y_ref).abs() / y_ref.abs().clamp_min(y_ref.pow(2).mean().sqrt())
    assert err_y.max().item() <= 4 * FP16_TOL


def test_attention_block_against_torch(cuda):
    from ternaryllm_amd import LlamaTernaryAttention, TernaryConfig
    from ternaryllm_amd.attention import apply_rope, rope_tables
    g = torch.Generator().manual_seed(12)
    cfg = TernaryConfig(hidden_size=256, num_attention_heads=4, num_key_value_heads=2, sparsity=0.9)
    attn = LlamaTernaryAttention(cfg, generator=g).to(cuda)
    B, S = 2, 24
    x = (0.1 * torch.randn((B, S, 256), generator=g))
    out, present = attn(x.to(cuda), use_cache=True)
    assert out.shape == (B, S, 256) and present[0].shape == (B, 2, S, 64)
    # fp32 restatement with dense weights
    wq, wk, wv, wo = (p.ternary_weight.float() for p in (attn.q_proj, attn.k_proj, attn.v_proj, attn.o_proj))
    q = (x @ wq).view(B, S, 4, 64).transpose(1, 2)
    k = (x @ wk).view(B, S, 2, 64).transpose(1, 2)
    v = (x @ wv).view(B, S, 2, 64).transpose(1, 2)
    cos, sin = rope_tables(torch.arange(S), 64, cfg.rope_theta, torch.float32, "cpu")
    q, k = apply_rope(q, cos, sin), apply_rope(k, cos, sin)
    k, v = k.repeat_interleave(2, 1), v.repeat_interleave(2, 1)
    scores = (q @ k.transpose(-1, -2)) / 8.0 + torch.full((S, S), float("-inf")).triu(1)
    ref = (torch.softmax(scores, -1) @ v).transpose(1, 2).reshape(B, S, 256) @ wo
    assert torch.allclose(out.cpu(), ref, rtol=2e-4, atol=2e-4 * ref.abs().max().item())
    # one decode step on top of the cache equals the last row of a full pass over S + 1 tokens
    x1 = (0.1 * torch.randn((B, 1, 256), generator=g))
    step, _ = attn(x1.to(cuda), past_key_value=present, position_offset=S, use_cache=True)
    full, _ = attn(torch.cat([x, x1], 1).to(cuda))
    assert torch.allclose(step[:, 0], full[:, -1], rtol=1e-4, atol=1e-4 * full.abs().max().item())


def test_full_size_properties(cuda):
    """At the benchmark's full shape the oracle's triple loop is too slow; the exact product is pinned by
    properties instead: linearity in X, a row permutation of X permutes Y, and a checksum of Y against
    X times the column-sum structure of W (all exact in fp32 for small-integer X)."""
    from ternaryllm_amd import ops
    from ternaryllm_amd.packing import PackedWeight
    M, K, N = 1024, 4096, 11008
    w = ternary_weight(K, N, 0.8, 1237)
    dw = ops.DeviceWeight(PackedWeight.from_dense(w), cuda)
    xa = activations(M, K, 1, torch.float16, integer=True)
    xb = activations(M, K, 2, torch.float16, integer=True)
    ya = ops.spmm(dw, xa.to(cuda), out_dtype=torch.float32)
    yb = ops.spmm(dw, xb.to(cuda), out_dtype=torch.float32)
    yab = ops.spmm(dw, (xa + 2 * xb).to(cuda), out_dtype=torch.float32)
    assert torch.equal(yab, ya + 2 * yb)
    perm = torch.randperm(M, generator=torch.Generator().manual_seed(3))
    assert torch.equal(ops.spmm(dw, xa[perm].to(cuda), out_dtype=torch.float32), ya[perm.to(cuda)])
    # sum over columns of Y == X @ (row sums of W): one matrix-vector product on the CPU
    row_sums = w.astype(np.float64).sum(1)
    assert np.array_equal(ya.double().sum(1).cpu().numpy(), xa.double().numpy() @ row_sums)
    # sum over rows of Y == (column sums of X) @ W
    assert np.array_equal(ya.double().sum(0).cpu().numpy(), xa.double().numpy().sum(0) @ w.astype(np.float64))
    # decode shape (M = 1) on the same weight
    y1 = ops.spmm(dw, xa[:1].to(cuda), out_dtype=torch.float32)
    assert torch.equal(y1, ya[:1])


def test_surgery_on_a_hugging_face_llama(cuda):
    """prepare_ternary_model on a small transformers Llama built from a local config (no download):
    the patched model's logits equal those of the same model with dense linears holding the ternary
    weights."""
    transformers = pytest.importorskip("transformers")
    import copy
    from ternaryllm_amd import TernaryConfig, TernaryLinear, prepare_ternary_model
    torch.manual_seed(11)
    hf_cfg = transformers.LlamaConfig(hidden_size=128, intermediate_size=256, num_hidden_layers=2, num_attention_heads=4,
                                      num_key_value_heads=4, vocab_size=120, max_position_embeddings=64)
    model = transformers.LlamaForCausalLM(hf_cfg).eval()
    cfg = TernaryConfig(sparsity=0.7)
    model = prepare_ternary_model(model, cfg, device=cuda, generator=torch.Generator().manual_seed(12))
    replaced = [m for m in model.modules() if isinstance(m, TernaryLinear)]
    assert len(replaced) == 2 * 7
    dense = copy.deepcopy(model).to("cpu")
    for name, mod in list(dense.named_modules()):
        if isinstance(mod, TernaryLinear):
            lin = torch.nn.Linear(mod.in_features, mod.out_features, bias=False)
            lin.weight.data = mod.ternary_weight.t().float().contiguous()
            parent, _, leaf = name.rpartition(".")
            setattr(dense.get_submodule(parent), leaf, lin)
    dense = dense.to(cuda)
    ids = torch.randint(0, 120, (2, 24), generator=torch.Generator().manual_seed(13)).to(cuda)
    with torch.no_grad():
        got = model(ids).logits.float()
        ref = dense(ids).logits.float()
    assert torch.isfinite(ref).all()
    assert (got - ref).abs().max().item() <= 1e-3 * ref.abs().max().item()


@pytest.mark.parametrize("name,M,K,N,s,dtype", [
    ("config 1", 16, 4096, 4096, 0.5, torch.float32),
    ("config 2", 1, 4096, 4096, 0.66, torch.float16),
    ("config 3 down", 1024, 11008, 4096, 0.8, torch.float16),
    ("config 4 projection", 1024, 4096, 4096, 0.9, torch.float16),
    ("config 5 decode head", 16, 4096, 32000, 0.66, torch.float16),
])
def test_baseline_configs_at_full_size(cuda, name, M, K, N, s, dtype):
    """The other benchmark shapes at their full sizes, on small-integer activations (every partial sum exact):
    the two checksum identities of the product, and for a few rows the product itself."""
    from ternaryllm_amd import ops
    from ternaryllm_amd.packing import PackedWeight
    w = ternary_weight(K, N, s, 1300 + N % 97)
    dw = ops.DeviceWeight(PackedWeight.from_dense(w), cuda)
    x = activations(M, K, 5, dtype, integer=True)
    print(f"case {name}", flush=True)
    y = ops.spmm(dw, x.to(cuda), out_dtype=torch.float32)
    wd = w.astype(np.float64)
    assert np.array_equal(y.double().sum(1).cpu().numpy(), x.double().numpy() @ wd.sum(1))
    assert np.array_equal(y.double().sum(0).cpu().numpy(), x.double().numpy().sum(0) @ wd)
    rows = sorted({0, M // 2, M - 1})
    assert np.array_equal(y[rows].double().cpu().numpy(), x[rows].double().numpy() @ wd)
