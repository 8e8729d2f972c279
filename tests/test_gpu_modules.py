"""GPU tests of the drop-in layer: ter_spmm.ter_spmm on merged arrays, TernaryLinear, the fused
MLP block and the attention block, against the CPU oracle / a plain torch fp32 restatement."""
import numpy as np
import pytest
import torch

from tests.util import FP16_TOL, FP32_TOL, activations, knobs, max_rel_err, ternary_weight

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


def test_ter_spmm_square_input_reads_row_major_unless_told(cuda, oracle):
    """rows == inners: the shape of X does not tell [batch, rows, inners] from [batch, inners, rows].  Without
    x_layout the shim reads it as the reference's modules pass it (row-major); x_layout="k_major" reads the same
    buffer as the reference kernel does; a layout that the shape contradicts is refused."""
    import ter_spmm
    K, N, tk = 256, 48, 64
    w = ternary_weight(K, N, 0.7, 44)
    wt = torch.from_numpy(w)
    tm = ter_spmm.convert_to_ter_tiled_mcsc(wt, N, K, (wt == 1).sum().item(), (wt == -1).sum().item(), tk, False, 4)
    rows = torch.from_numpy(tm[0]).to(torch.int16).to(cuda)
    offs = torch.from_numpy(tm[1]).to(cuda)
    tiles = torch.from_numpy(tm[2]).to(torch.int16).to(cuda)
    bs = 2
    x = activations(bs * K, K, 45, torch.float32, integer=True).reshape(bs, K, K)
    as_rows = np.stack([oracle.mcsc_product(x[b].numpy(), tm[0], tm[1], N, tk) for b in range(bs)])
    as_kmajor = np.stack([oracle.mcsc_product(x[b].t().contiguous().numpy(), tm[0], tm[1], N, tk) for b in range(bs)])
    assert not np.array_equal(as_rows, as_kmajor)
    xd = x.to(cuda)
    for layout, want in ((None, as_rows), ("row_major", as_rows), (0, as_rows), ("k_major", as_kmajor), (1, as_kmajor)):
        y = ter_spmm.ter_spmm(xd, rows, offs, tiles, bs, K, N, K, False, False, x_layout=layout)
        assert np.array_equal(y.cpu().numpy().astype(np.float64), want), layout
    narrow = xd[:, :8].contiguous()   # [batch, 8, K]: only row-major fits
    with pytest.raises(ValueError):
        ter_spmm.ter_spmm(narrow, rows, offs, tiles, bs, 8, N, K, False, False, x_layout="k_major")
    with pytest.raises(ValueError):
        ter_spmm.ter_spmm(narrow, rows, offs, tiles, bs, 8, N, K, False, False, x_layout="columns")


def _hand_cases():
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "mcsc_hand_cases.json")) as f:
        return json.load(f)["cases"]


@pytest.mark.parametrize("case", _hand_cases(), ids=lambda c: c["name"][:40])
def test_ter_spmm_on_hand_worked_arrays(cuda, case):
    """ter_spmm.ter_spmm on the fixture's merged arrays gives the hand-worked sums, bit for bit (integers in
    fp32): lossy tiles, a second tile's row offset, padded arrays that name a row twice, and -- with
    `uniformed` -- the pair part alone."""
    import ter_spmm
    K = case["inners"]
    rows = torch.tensor(case["merged_row_idx"], dtype=torch.int16, device=cuda)
    offs = torch.tensor(case["merged_off"], dtype=torch.int32, device=cuda)
    tiles = torch.tensor(case["col_tile_idx"], dtype=torch.int16, device=cuda)
    x = torch.tensor(case["x"], dtype=torch.float32)
    xs = torch.stack([x, 2 * x + 1, -x]).reshape(1, 3, K).to(cuda)
    signs = sum(sg for sg, _ in case["product_terms"])
    y = ter_spmm.ter_spmm(xs, rows, offs, tiles, 1, 3, 1, K, False, case["padding"])
    assert y.reshape(-1).tolist() == [case["product"], 2 * case["product"] + signs, -case["product"]]
    y1 = ter_spmm.ter_spmm(xs[:, :1], rows, offs, tiles, 1, 1, 1, K, False, case["padding"])   # M = 1: the decode kernel
    assert y1.reshape(-1).tolist() == [case["product"]]
    n_pair_terms = int((offs.cpu().reshape(-1, 4)[:, 1] - offs.cpu().reshape(-1, 4)[:, 0]).sum())
    pairs_only = sum(sg * case["x"][r] for sg, r in case["product_terms"][:n_pair_terms])
    yu = ter_spmm.ter_spmm(xs[:, :1], rows, offs, tiles, 1, 1, 1, K, True, case["padding"])
    assert yu.reshape(-1).tolist() == [pairs_only]


def test_ter_spmm_on_padded_arrays(cuda, oracle):
    """padding=True, padding_size=4 arrays of a random weight through ter_spmm.ter_spmm: the product equals the
    oracle's walk of those arrays, including the tiles whose padding makes the arrays name a row twice
    (what they encode is then not a ternary matrix, and the product still follows the arrays)."""
    import ter_spmm
    from ternaryllm_amd import packing
    K, N, tk = 1024, 80, 256
    w = ternary_weight(K, N, 0.8, 43)
    wt = torch.from_numpy(w)
    cp, cn = (wt == 1).sum().item(), (wt == -1).sum().item()
    tm = ter_spmm.convert_to_ter_tiled_mcsc(wt, N, K, cp, cn, tk, True, 4)
    encoded = packing.PackedWeight.from_mcsc(tm[0], tm[1], N, K, tk).to_dense()
    assert np.abs(encoded).max() >= 2   # the case the test is about does occur in these arrays
    rows = torch.from_numpy(tm[0]).to(torch.int16).to(cuda)
    offs = torch.from_numpy(tm[1]).to(cuda)
    tiles = torch.from_numpy(tm[2]).to(torch.int16).to(cuda)
    for M in (1, 6, 64):
        x = activations(M, K, 50 + M, torch.float32, integer=True)
        y = ter_spmm.ter_spmm(x.reshape(1, M, K).to(cuda), rows, offs, tiles, 1, M, N, K, False, True)
        ref = oracle.mcsc_product(x.numpy(), tm[0], tm[1], N, tk)
        assert np.array_equal(y[0].cpu().numpy().astype(np.float64), ref)


def test_ter_spmm_prepared_weight_follows_its_tensors(cuda, oracle):
    """The device weight ter_spmm builds lives on the row-index tensor: a second weight of the same shape and
    the same number of non-zeros, allocated where a freed one lay, must give its own product; an in-place
    change of the arrays must be noticed; prepare() ahead of the call gives the same result."""
    import gc
    import ter_spmm
    K, N, tk = 512, 64, 64

    def arrays(seed):
        from ternaryllm_amd import random_ternary_weights
        w = random_ternary_weights((K, N), 0.75, uniform=True, block_size=64, generator=torch.Generator().manual_seed(seed))
        cp, cn = (w == 1).sum().item(), (w == -1).sum().item()
        tm = ter_spmm.convert_to_ter_tiled_mcsc(w, N, K, cp, cn, tk, False, 4)
        return w.numpy(), tm

    x = activations(4, K, 77, torch.float32, integer=True)
    xd = x.reshape(1, 4, K).to(cuda)
    for seed in (1, 2, 3):   # same shape, same number of non-zeros: the allocator hands the freed addresses back
        w, tm = arrays(seed)
        rows = torch.from_numpy(tm[0]).to(torch.int16).to(cuda)
        offs = torch.from_numpy(tm[1]).to(cuda)
        tiles = torch.from_numpy(tm[2]).to(torch.int16).to(cuda)
        y = ter_spmm.ter_spmm(xd, rows, offs, tiles, 1, 4, N, K, True, False)
        ref = oracle.mcsc_product(x.numpy(), tm[0], tm[1], N, tk, uniformed=True)
        assert np.array_equal(y[0].cpu().numpy().astype(np.float64), ref)
        assert np.array_equal(ref, oracle.dense_product(x.numpy(), w))   # balanced blocks: nothing is dropped
        del rows, offs, tiles, y
        gc.collect()
    w, tm = arrays(4)
    rows = torch.from_numpy(tm[0]).to(torch.int16).to(cuda)
    offs = torch.from_numpy(tm[1]).to(cuda)
    tiles = torch.from_numpy(tm[2]).to(torch.int16).to(cuda)
    ter_spmm.prepare(rows, offs, N, K, uniformed=False)
    y0 = ter_spmm.ter_spmm(xd, rows, offs, tiles, 1, 4, N, K, False, False)
    w5, tm5 = arrays(5)
    rows.copy_(torch.from_numpy(tm5[0]).to(torch.int16))   # in place: same tensors, new content
    offs.copy_(torch.from_numpy(tm5[1]))
    y1 = ter_spmm.ter_spmm(xd, rows, offs, tiles, 1, 4, N, K, False, False)
    assert np.array_equal(y0[0].cpu().numpy().astype(np.float64), oracle.dense_product(x.numpy(), w))
    assert np.array_equal(y1[0].cpu().numpy().astype(np.float64), oracle.dense_product(x.numpy(), w5))


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
    # the same block on one weight of (gate, up) column pairs with the gate in the product's epilogue
    mlp.paired = True
    yp = mlp(x.to(cuda).reshape(1, tokens, 512))
    assert yp.shape == y.shape and mlp._pairs[0].columns == 2 * 1408
    err_p = (yp[0].double().cpu() - y_ref).abs() / y_ref.abs().clamp_min(y_ref.pow(2).mean().sqrt())
    assert err_p.max().item() <= 4 * FP16_TOL


def test_attention_block_against_torch(cuda):
    from ternaryllm_amd import LlamaTernaryAttention, TernaryConfig
    from ternaryllm_amd.attention import apply_rope, rope_tables
    g = torch.Generator().manual_seed(12)
    cfg = TernaryConfig(hidden_size=256, num_attention_heads=4, num_key_value_heads=2, sparsity=0.9)
    attn = LlamaTernaryAttention(cfg, generator=g).to(cuda)
    B, S = 2, 24
    x = (0.1 * torch.randn((B, S, 256), generator=g))
    out, weights, present = attn(x.to(cuda), use_cache=True)
    assert out.shape == (B, S, 256) and weights is None and present[0].shape == (B, 2, S, 64)
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
    step, _, grown = attn(x1.to(cuda), past_key_value=present, use_cache=True)
    full, _, none = attn(torch.cat([x, x1], 1).to(cuda))
    assert none is None and grown[0].shape == (B, 2, S + 1, 64)
    assert torch.allclose(step[:, 0], full[:, -1], rtol=1e-4, atol=1e-4 * full.abs().max().item())
    # the reference's arguments (TernaryAttn.py:59-70): an additive mask, position ids, externally computed
    # (cos, sin), output_attentions -- all must give the result of the plain causal call
    add_mask = torch.full((S, S + 9), float("-inf")).triu(1)[None, None].to(cuda)    # longer than the keys: cut to them
    pos_ids = torch.arange(S, device=cuda)[None].expand(B, S)
    o2, w2, p2 = attn(x.to(cuda), add_mask, pos_ids, None, True, False)
    assert p2 is None and w2.shape == (B, 4, S, S)
    assert torch.allclose(o2, out, rtol=1e-4, atol=1e-4 * out.abs().max().item())
    assert torch.allclose(w2.sum(-1), torch.ones_like(w2.sum(-1)), atol=1e-5) and float(w2[0, 0].triu(1).abs().max()) == 0.0
    o3, _, _ = attn(x.to(cuda), attention_mask=add_mask, position_embeddings=(cos[None].to(cuda), sin[None].to(cuda)))
    assert torch.allclose(o3, out, rtol=1e-4, atol=1e-4 * out.abs().max().item())
    # no mask and is_causal off: the reference's literal behaviour, every query sees every key
    attn.is_causal = False
    o4, _, _ = attn(x.to(cuda))
    attn.is_causal = True
    ref4 = (torch.softmax((q @ k.transpose(-1, -2)) / 8.0, -1) @ v).transpose(1, 2).reshape(B, S, 256) @ wo
    assert torch.allclose(o4.cpu(), ref4, rtol=2e-4, atol=2e-4 * ref4.abs().max().item())


def test_attention_with_one_weight_for_q_k_v(cuda):
    """fused_qkv: q | k | v as one packed weight gives what the three projections give one by one (integer
    activations: every sum is exact, so bit for bit), with and without scales, for 1, 12 and 200 tokens; the
    side-by-side weight follows a projection that changes."""
    from ternaryllm_amd import LlamaTernaryAttention, TernaryConfig
    g = torch.Generator().manual_seed(14)
    cfg = TernaryConfig(hidden_size=512, num_attention_heads=8, num_key_value_heads=2, sparsity=0.85)
    attn = LlamaTernaryAttention(cfg, generator=g).to(cuda).half()
    other = LlamaTernaryAttention(cfg, generator=g).to(cuda).half()

    def both(x):
        attn.fused_qkv = True
        one = attn(x, use_cache=True)
        attn.fused_qkv = False
        three = attn(x, use_cache=True)
        attn.fused_qkv = True
        return one, three

    for scaled in (False, True):
        if scaled:
            attn.q_proj.w_scale = (0.5 + torch.rand(512, generator=g)).half().to(cuda)
            attn.v_proj.w_scale = (0.5 + torch.rand(128, generator=g)).half().to(cuda)   # k_proj stays without one
        for tokens in (1, 12, 200):
            x = activations(tokens, 512, 70 + tokens, torch.float16, integer=True).reshape(1, tokens, 512).to(cuda) / 64
            one, three = both(x)
            assert attn._qkv[0].columns == 512 + 2 * 128
            assert torch.equal(one[2][0], three[2][0]) and torch.equal(one[2][1], three[2][1])   # keys and values
            assert torch.equal(one[0], three[0])
    before = attn._qkv[0]
    attn.k_proj.load_state_dict(other.k_proj.state_dict())
    x = activations(4, 512, 99, torch.float16, integer=True).reshape(1, 4, 512).to(cuda) / 64
    one, three = both(x)
    assert attn._qkv[0] is not before and torch.equal(one[0], three[0]) and torch.equal(one[2][0], three[2][0])


def test_mlp_block_with_another_activation(cuda):
    """hidden_act other than "silu" (TernaryMLP.py:30-34 looks the activation up by name): the block is two
    products, the named activation in torch and the down product; against an fp64 restatement."""
    from ternaryllm_amd import LlamaTernaryMLP, TernaryConfig
    g = torch.Generator().manual_seed(15)
    for act, fn in (("gelu", torch.nn.functional.gelu), ("relu", torch.relu)):
        cfg = TernaryConfig(hidden_size=256, intermediate_size=768, sparsity=0.8, hidden_act=act)
        for paired in (False, True):
            mlp = LlamaTernaryMLP(cfg, generator=g, paired=paired).to(cuda)
            for tokens in (1, 40):
                x = 0.1 * torch.randn((tokens, 256), generator=g)
                wg, wu, wd = (p.ternary_weight.double() for p in (mlp.gate_proj, mlp.up_proj, mlp.down_proj))
                ref = (fn(x.double() @ wg) * (x.double() @ wu)) @ wd
                y = mlp(x.to(cuda))
                assert y.shape == (tokens, 256) and y.dtype == torch.float32
                assert (y.double().cpu() - ref).abs().max().item() <= FP32_TOL * ref.abs().max().item()


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


def test_attention_module_as_self_attn_of_a_hugging_face_llama(cuda):
    """LlamaTernaryAttention in the place of `self_attn` of a transformers Llama built from a local config (what
    the reference does to the model it patches, TernaryLlama.py:69-75): the decoder layer calls it with its own
    keyword arguments (mask, position embeddings, cache); logits of a forward pass and of a cached two-step
    continuation must equal those of the same model with dense projections holding the ternary weights."""
    transformers = pytest.importorskip("transformers")
    import copy
    import inspect
    from ternaryllm_amd import LlamaTernaryAttention, TernaryConfig
    from ternaryllm_amd.attention import TwoResultAttention, collect_attn_linear_layers, replace_linear_layers
    torch.manual_seed(21)
    hf_cfg = transformers.LlamaConfig(hidden_size=128, intermediate_size=256, num_hidden_layers=2, num_attention_heads=4,
                                      num_key_value_heads=2, vocab_size=120, max_position_embeddings=64)
    model = transformers.LlamaForCausalLM(hf_cfg).eval().to(cuda)
    dense = copy.deepcopy(model)
    theta = getattr(hf_cfg, "rope_theta", None) or hf_cfg.rope_parameters["rope_theta"]
    cfg = TernaryConfig(hidden_size=128, num_attention_heads=4, num_key_value_heads=2, sparsity=0.6, rope_theta=theta)
    two_results = "past_key_values" in inspect.signature(type(model.model.layers[0].self_attn).forward).parameters
    g = torch.Generator().manual_seed(22)
    for li, layer in enumerate(model.model.layers):
        attn = LlamaTernaryAttention(cfg, layer_idx=li, generator=g, reference_buffers=False).to(cuda)
        layer.self_attn = TwoResultAttention(attn) if two_results else attn
        twin = dense.model.layers[li].self_attn
        for name in ("q_proj", "k_proj", "v_proj", "o_proj"):
            getattr(twin, name).weight.data = getattr(attn, name).ternary_weight.t().float().contiguous().to(cuda)
    ids = torch.randint(0, 120, (2, 20), generator=torch.Generator().manual_seed(23)).to(cuda)
    with torch.no_grad():
        got = model(ids).logits.float()
        ref = dense(ids).logits.float()
        assert torch.isfinite(ref).all()
        assert (got - ref).abs().max().item() <= 1e-3 * ref.abs().max().item()
        # prefill 18 tokens with a cache, then two single-token steps on top of it
        out = model(ids[:, :18], use_cache=True)
        cache = out.past_key_values
        for j in (18, 19):
            out = model(ids[:, j:j + 1], past_key_values=cache, use_cache=True)
            cache = out.past_key_values
            assert (out.logits[:, 0].float() - ref[:, j]).abs().max().item() <= 1e-3 * ref.abs().max().item()
    # the reference's per-module helper: swap the nn.Linear projections of one attention module for random ternary ones
    twin = dense.model.layers[0].self_attn
    replace_linear_layers(collect_attn_linear_layers(twin), twin, 0.8)
    from ternaryllm_amd import TernaryLinear
    assert all(isinstance(getattr(twin, n), TernaryLinear) for n in ("q_proj", "k_proj", "v_proj", "o_proj"))


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


def _rows_ref_mlp(x_rows, wg, wu, wd, sg, su, sd):
    """float64 restatement of down(silu(gate(x)) * up(x)) for a few rows; returns (h, y)."""
    g = (x_rows @ wg) * sg
    u = (x_rows @ wu) * su
    h = g / (1.0 + np.exp(-g)) * u
    return h, (h @ wd) * sd


@pytest.mark.parametrize("split", ["0", "1"])
def test_config3_mlp_block_at_full_size(cuda, split):
    """BASELINE config 3 at its size: 1024 tokens, gate/up 4096 -> 11008 fused with the SiLU gate, down
    11008 -> 4096, 80 % sparsity, fp16 activations, per-channel fp16 scales; whole output tiles and shared-out
    K tiles (TL_ROWS_SPLIT).  Full rows of H and of Y against the float64 restatement, every row of Y against the
    float64 product of the H the GPU produced."""
    from ternaryllm_amd import LlamaTernaryMLP, TernaryConfig, ops
    with knobs(TL_ROWS_SPLIT=split):
        g = torch.Generator().manual_seed(31)
        H, I, M = 4096, 11008, 1024
        cfg = TernaryConfig(hidden_size=H, intermediate_size=I, sparsity=0.8)
        sc = {"gate": ((0.5 + torch.rand(I, generator=g)) / 28.0).half(), "up": ((0.5 + torch.rand(I, generator=g)) / 28.0).half(),
              "down": ((0.5 + torch.rand(H, generator=g)) / 47.0).half()}   # ~1 / sqrt(non-zeros per column): outputs stay O(1)
        mlp = LlamaTernaryMLP(cfg, generator=g, scales=sc, reference_buffers=False).to(cuda)
        x = torch.randn((M, H), generator=g).half()
        print(f"case config 3 fused MLP, TL_ROWS_SPLIT={split}", flush=True)
        h = ops.mlp_gate_up(mlp.gate_proj.device_weight(), mlp.up_proj.device_weight(), x.to(cuda), mlp.gate_proj.w_scale,
                            mlp.up_proj.w_scale)
        y = mlp(x.to(cuda).reshape(8, 128, H))
        assert h.shape == (M, I) and h.dtype == torch.float16 and y.shape == (8, 128, H) and y.dtype == torch.float16
        wg, wu, wd = (m.ternary_weight.numpy().astype(np.float64) for m in (mlp.gate_proj, mlp.up_proj, mlp.down_proj))
        sg, su, sd = (sc[k].double().numpy() for k in ("gate", "up", "down"))
        rows = [0, 255, 256, 511, 777, 1023]
        h_ref, y_ref = _rows_ref_mlp(x[rows].double().numpy(), wg, wu, wd, sg, su, sd)
        h_got = h[rows].double().cpu().numpy()
        err_h = np.abs(h_got - h_ref) / np.maximum(np.abs(h_ref), np.abs(h_ref).mean())
        print(f"  max rel err of H rows {err_h.max():.3e}", flush=True)
        assert err_h.max() <= FP16_TOL
        y_got = y.reshape(M, H)[rows].double().cpu().numpy()
        err_y = np.abs(y_got - y_ref) / np.maximum(np.abs(y_ref), np.sqrt((y_ref ** 2).mean()))
        print(f"  max rel err of Y rows (fp16 H in between) {err_y.max():.3e}", flush=True)
        assert err_y.max() <= 1.5 * FP16_TOL   # measured 1.2e-3: the fp16 rounding of H carried through ~2200 signed adds
        # the down projection alone, every row: float64 product of the H the GPU wrote (fp16 values, exact inputs)
        y_all = (h.double().cpu().numpy() @ wd) * sd
        assert max_rel_err(y.reshape(M, H).double().cpu().numpy(), y_all, h.double().cpu().numpy() * 1.0, mlp.down_proj.ternary_weight.numpy()) <= FP16_TOL


def test_config4_attention_block_at_full_size(cuda):
    """BASELINE config 4 at its size: hidden 4096, 32 heads x 128, batch 8 x seq 128 = 1024 tokens, four
    4096 -> 4096 ternary projections at 90 % sparsity, fp16, causal, against an fp32 restatement on dense weights."""
    from ternaryllm_amd import LlamaTernaryAttention, TernaryConfig
    from ternaryllm_amd.attention import apply_rope, rope_tables
    g = torch.Generator().manual_seed(33)
    cfg = TernaryConfig(hidden_size=4096, num_attention_heads=32, num_key_value_heads=32, sparsity=0.9)
    attn = LlamaTernaryAttention(cfg, layer_idx=0, generator=g, reference_buffers=False).to(cuda)
    B, S, H, nh, hd = 8, 128, 4096, 32, 128
    x = (torch.randn((B, S, H), generator=g) / 20.0).half()    # ~1 / sqrt(non-zeros per column): q, k, v stay O(1)
    print("case config 4 attention block", flush=True)
    out, weights, cache = attn(x.to(cuda), use_cache=True)
    assert out.shape == (B, S, H) and out.dtype == torch.float16 and weights is None and cache[0].shape == (B, nh, S, hd)
    xf = x.float().to(cuda)
    wq, wk, wv, wo = (p.ternary_weight.float().to(cuda) for p in (attn.q_proj, attn.k_proj, attn.v_proj, attn.o_proj))
    q = (xf @ wq).view(B, S, nh, hd).transpose(1, 2)
    k = (xf @ wk).view(B, S, nh, hd).transpose(1, 2)
    v = (xf @ wv).view(B, S, nh, hd).transpose(1, 2)
    cos, sin = rope_tables(torch.arange(S, device=cuda), hd, cfg.rope_theta, torch.float32, cuda)
    q, k = apply_rope(q, cos, sin), apply_rope(k, cos, sin)
    scores = (q @ k.transpose(-1, -2)) / hd ** 0.5 + torch.full((S, S), float("-inf"), device=cuda).triu(1)
    ref = (torch.softmax(scores, -1) @ v).transpose(1, 2).reshape(B, S, H) @ wo
    err = (out.float() - ref).abs().max().item() / ref.abs().max().item()
    print(f"  max |out - ref| / max |ref| = {err:.3e}", flush=True)
    assert err <= 1e-3   # measured 3.8e-4: fp16 roundings of q, k, v and the attention output in between
    # the cache holds the rotated keys and the values, as the reference's cache update receives them
    assert (cache[0].float() - k).abs().max().item() <= 2e-3 * k.abs().max().item()
    assert (cache[1].float() - v).abs().max().item() <= 2e-3 * v.abs().max().item()


@pytest.mark.parametrize("blk", [64, 512])
def test_uniform_weights_and_reference_buffers(cuda, oracle, blk):
    """TernaryLinear(uniform=True): block-balanced weights (TernaryLinear.py:39-77) through the module's own
    product and, as merged arrays with the kernels' `uniformed` flag, through ter_spmm.ter_spmm; both equal
    the exact product, because balanced blocks of the merged format's tile height leave no same-sign part."""
    import ter_spmm
    from ternaryllm_amd import TernaryLinear
    K, N = 1024, 192
    lin = TernaryLinear(K, N, sparsity=0.75, uniform=True, uniform_blk_size=blk, bias=False,
                        generator=torch.Generator().manual_seed(90 + blk)).to(cuda)
    w = lin.ternary_weight.numpy()
    counts = np.abs(w).reshape(K // blk, blk, N).sum(1)
    assert counts.min() == counts.max() and (w.reshape(K // blk, blk, N).sum(1) == 0).all()   # every block balanced
    for M in (1, 16, 130):
        x = activations(M, K, 91 + M, torch.float32, integer=True)
        ref = oracle.fast_product(x.double().numpy(), w)
        assert np.array_equal(lin(x.to(cuda)).cpu().numpy().astype(np.float64), ref)
        for uniformed in (False, True):
            y = ter_spmm.ter_spmm(x.reshape(1, M, K).to(cuda), lin.w_row_indices, lin.w_col_offsets, lin.w_col_tile_indices, 1, M, N, K,
                                  uniformed, False)
            if blk == 64 or not uniformed:
                # blocks of 64 rows nest in the 256-row tiles: every tile is balanced.  With 512-row blocks a tile
                # is half a block and need not be, so only the full walk is exact there -- and only where the
                # packer's alignment rule drops nothing, which the oracle's walk of the same arrays tells
                want = oracle.mcsc_product(x.numpy(), lin.w_row_indices.cpu().numpy(), lin.w_col_offsets.cpu().numpy(), N, 256, uniformed)
                assert np.array_equal(y[0].cpu().numpy().astype(np.float64), want)
                if blk == 64:
                    assert np.array_equal(want, ref)


def test_ternarised_float_weights(cuda):
    """TernaryLinear.from_float: threshold ternarisation with a per-channel scale; the module's product equals
    (x @ t) * scale for its own t and scale, and approximates x @ w."""
    from ternaryllm_amd import TernaryLinear
    from ternaryllm_amd.linear import ternarize_threshold
    g = torch.Generator().manual_seed(95)
    K, N = 1024, 320
    wf = torch.randn((K, N), generator=g) / 32.0
    for sparsity in (None, 0.7):
        lin = TernaryLinear.from_float(wf, sparsity).to(cuda)
        t, scale = ternarize_threshold(wf, sparsity)
        assert torch.equal(lin.ternary_weight, t)
        if sparsity is not None:
            assert abs((t == 0).float().mean().item() - sparsity) < 0.01
        for M, dtype, tol in ((1, torch.float32, FP32_TOL), (24, torch.float16, FP16_TOL), (200, torch.float16, FP16_TOL)):
            x = torch.randn((M, K), generator=g).to(dtype)
            y = lin(x.to(cuda))
            ref = (x.double().numpy() @ t.double().numpy()) * scale.double().numpy()[None, :]
            floor = np.linalg.norm(x.double().numpy(), axis=1, keepdims=True) * np.sqrt((t != 0).float().mean().item()) * scale.double().numpy()[None, :]
            err = np.abs(y.double().cpu().numpy() - ref) / np.maximum(np.abs(ref), floor)
            assert err.max() <= tol
            # ... and it is a ternary approximation of the float product: well correlated with it
            exact = x.double().numpy() @ wf.double().numpy()
            corr = np.corrcoef(exact.reshape(-1), ref.reshape(-1))[0, 1]
            assert corr > 0.8
