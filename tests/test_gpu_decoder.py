"""The ternary Llama-shaped decoder against a plain fp32 torch restatement that multiplies by the
dense weights decoded from the packed blobs: prefill logits, teacher-forced decode logits, and the
HIP-graph replay of the decode step against its eager run."""
import pytest
import torch

pytestmark = pytest.mark.gpu

# Logit error of the fp16 pipeline against the fp32 restatement, relative to the largest logit.  An fp16
# rounding is 2^-11 = 4.9e-4 relative; a logit sums thousands of rounded O(1) values with random signs, and a
# layer rounds its activations about ten times.  The bounds are about twice what was measured on MI355X:
# 1.3e-3 for TINY (2 layers x 256 wide), 1.7e-3 for FULL_WIDTH (2 layers x 4096 wide, 512 + 4 positions).
TINY_TOL = 3e-3
FULL_WIDTH_TOL = 4e-3


def _reference_logits(model, tokens):
    """fp32 forward over the whole sequence with dense weights; returns logits [B, S, vocab]."""
    c = model.config
    dev = tokens.device
    B, S = tokens.shape
    nh, hd, H = c.num_attention_heads, c.head_dim, c.hidden_size

    def lin(m, x):
        w = m.ternary_weight.to(dev, torch.float32)
        y = x @ w
        return y * m.w_scale.float() if m.w_scale is not None else y

    def norm(n, x):
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + n.eps) * n.weight.float()

    def rope(x):
        cos, sin = model.rope_cos[:S].float(), model.rope_sin[:S].float()
        half = hd // 2
        return x * cos + torch.cat([-x[..., half:], x[..., :half]], -1) * sin

    x = model.embed_tokens.float()[tokens]
    for layer in model.layers:
        h = norm(layer.input_layernorm, x)
        qkv = lin(layer.qkv_proj, h).view(B, S, 3, nh, hd)
        q, k, v = (qkv[:, :, i].transpose(1, 2) for i in range(3))
        q, k = rope(q), rope(k)
        att = (q @ k.transpose(-1, -2)) / hd ** 0.5
        att = att.masked_fill(~torch.tril(torch.ones(S, S, dtype=torch.bool, device=dev)), float("-inf")).softmax(-1)
        a = (att @ v).transpose(1, 2).reshape(B, S, H)
        x = x + lin(layer.o_proj, a)
        h = norm(layer.post_attention_layernorm, x)
        gu = lin(layer.gate_up_proj, h)   # columns 2j, 2j + 1: gate and up of output j
        x = x + lin(layer.down_proj, torch.nn.functional.silu(gu[..., 0::2]) * gu[..., 1::2])
    return lin(model.lm_head, norm(model.norm, x))


@pytest.fixture(scope="module")
def tiny(cuda):
    from ternaryllm_amd import TernaryConfig
    from ternaryllm_amd.llama import TernaryLlamaDecoder
    cfg = TernaryConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                        num_key_value_heads=4, vocab_size=320, max_position_embeddings=96, sparsity=0.66)
    return TernaryLlamaDecoder(cfg, seed=5, device=cuda, pack_threads=2)


def test_prefill_and_decode_match_fp32_reference(tiny, cuda):
    g = torch.Generator().manual_seed(3)
    B, S, extra = 2, 70, 3
    tokens = torch.randint(0, tiny.config.vocab_size, (B, S + extra), generator=g).to(cuda)
    ref = _reference_logits(tiny, tokens)                       # [B, S + extra, V]
    scale = ref.abs().max().item()
    got = tiny.prefill(tokens[:, :S]).float()                   # 140 rows: the row-parallel kernel
    worst = (got - ref[:, S - 1]).abs().max().item() / scale
    st = tiny._decode_state(B)
    for j in range(extra):                                      # teacher-forced single-token steps: the small-M kernel
        st["token"].copy_(tokens[:, S + j])
        st["pos"].fill_(S + j)
        st["mask"].copy_((torch.arange(tiny.max_seq_len, device=cuda) <= S + j)[None, None, None])
        logits = tiny._decode_step(st["token"], st["pos"], st["mask"]).float()
        worst = max(worst, (logits - ref[:, S + j]).abs().max().item() / scale)
    print(f"  tiny decoder: max |logit - ref| / max |ref| = {worst:.3e}", flush=True)
    assert worst <= TINY_TOL


@pytest.fixture(scope="module")
def full_width(cuda):
    """Two layers of BASELINE config 5's decoder at its real width: hidden 4096, FFN 11008, 32 heads x 128,
    vocabulary 32000, 66 % sparsity."""
    from ternaryllm_amd import TernaryConfig
    from ternaryllm_amd.llama import TernaryLlamaDecoder
    cfg = TernaryConfig(hidden_size=4096, intermediate_size=11008, num_hidden_layers=2, num_attention_heads=32,
                        num_key_value_heads=32, vocab_size=32000, max_position_embeddings=528, sparsity=0.66)
    return TernaryLlamaDecoder(cfg, seed=11, device=cuda, pack_threads=8)


@pytest.mark.parametrize("batch", [1, 16])
def test_full_width_prefill_512_and_decode_steps(full_width, cuda, batch):
    """Config 5's shapes (prefill of 512 tokens, then single-token steps, batch 1 and 16) on the two-layer
    full-width model against the fp32 restatement on dense weights: the prefill's logits and four
    teacher-forced decode steps."""
    model = full_width
    g = torch.Generator().manual_seed(20 + batch)
    S, extra = 512, 4
    tokens = torch.randint(0, model.config.vocab_size, (batch, S + extra), generator=g).to(cuda)
    print(f"case full-width decoder batch={batch}", flush=True)
    ref = _reference_logits(model, tokens)[:, S - 1:].clone()          # [B, 1 + extra, V]
    scale = ref.abs().max().item()
    got = model.prefill(tokens[:, :S]).float()
    worst = (got - ref[:, 0]).abs().max().item() / scale
    st = model._decode_state(batch)
    for j in range(extra):
        st["token"].copy_(tokens[:, S + j])
        st["pos"].fill_(S + j)
        st["mask"].copy_((torch.arange(model.max_seq_len, device=cuda) <= S + j)[None, None, None])
        logits = model._decode_step(st["token"], st["pos"], st["mask"]).float()
        worst = max(worst, (logits - ref[:, 1 + j]).abs().max().item() / scale)
    print(f"  max |logit - ref| / max |ref| = {worst:.3e}", flush=True)
    model._state = None
    assert worst <= FULL_WIDTH_TOL


def test_native_decode_step_matches_torch_operators(tiny, cuda):
    """The library's rotary / cache / attention kernels against the same step on torch operators."""
    g = torch.Generator().manual_seed(6)
    B, S = 3, 33
    tokens = torch.randint(0, tiny.config.vocab_size, (B, S + 2), generator=g).to(cuda)
    assert tiny.native_decode
    outs = {}
    for native in (False, True):
        tiny.native_decode = native
        tiny.prefill(tokens[:, :S])
        st = tiny._decode_state(B)
        logits = []
        for j in range(2):
            st["token"].copy_(tokens[:, S + j])
            st["pos"].fill_(S + j)
            st["mask"].copy_((torch.arange(tiny.max_seq_len, device=cuda) <= S + j)[None, None, None])
            logits.append(tiny._decode_step(st["token"], st["pos"], st["mask"]).float())
        outs[native] = (torch.stack(logits), tiny._cache[:, :, :, :, : S + 2].float().clone())
    tiny.native_decode = True
    scale = outs[False][0].abs().max().item()
    assert (outs[True][0] - outs[False][0]).abs().max().item() <= 1e-2 * scale
    assert (outs[True][1] - outs[False][1]).abs().max().item() <= 2e-3 * outs[False][1].abs().max().item()


def test_batched_decode_step_on_k_major_activations(tiny, cuda):
    """Eight rows: the step keeps its activations as K-major images between the kernels; same check as above."""
    g = torch.Generator().manual_seed(7)
    B, S = 8, 20
    tokens = torch.randint(0, tiny.config.vocab_size, (B, S + 2), generator=g).to(cuda)
    outs = {}
    for native in (False, True):
        tiny.native_decode = native
        tiny.prefill(tokens[:, :S])
        st = tiny._decode_state(B)
        logits = []
        for j in range(2):
            st["token"].copy_(tokens[:, S + j])
            st["pos"].fill_(S + j)
            st["mask"].copy_((torch.arange(tiny.max_seq_len, device=cuda) <= S + j)[None, None, None])
            logits.append(tiny._decode_step(st["token"], st["pos"], st["mask"]).float())
        outs[native] = torch.stack(logits)
    tiny.native_decode = True
    tiny._state = None
    assert (outs[True] - outs[False]).abs().max().item() <= 1e-2 * outs[False].abs().max().item()


def test_chained_decode_step_without_elementwise_kernels(tiny, full_width, cuda):
    """9 to 16 rows: the step whose products do the residual adds and the RMSNorms (tl_spmm_chain) against the step with
    tl_add_rmsnorm and tl_silu_mul launches, and against torch operators; then the pieces of one chained pair by
    themselves against a float64 restatement."""
    from tests.util import max_rel_err, ternary_weight
    from ternaryllm_amd import ops
    from ternaryllm_amd.packing import PackedWeight
    g = torch.Generator().manual_seed(33)
    for model, B, S in ((tiny, 16, 20), (tiny, 9, 20), (full_width, 16, 6)):
        tokens = torch.randint(0, model.config.vocab_size, (B, S + 2), generator=g).to(cuda)
        outs = {}
        for mode in ("torch", "launches", "chain"):
            model.native_decode = mode != "torch"
            model.chain_decode = mode == "chain"
            model._graph = None
            model.prefill(tokens[:, :S])
            st = model._decode_state(B)
            logits = []
            for j in range(2):
                st["token"].copy_(tokens[:, S + j])
                st["pos"].fill_(S + j)
                st["mask"].copy_((torch.arange(model.max_seq_len, device=cuda) <= S + j)[None, None, None])
                logits.append(model._decode_step(st["token"], st["pos"], st["mask"]).float())
            outs[mode] = torch.stack(logits)
            if mode == "chain":
                assert model.chain_decode   # the chained kernels exist for these shapes: nothing fell back
        model.native_decode, model.chain_decode, model._state, model._graph = True, True, None, None
        top = outs["torch"].abs().max().item()
        assert (outs["chain"] - outs["launches"]).abs().max().item() <= 4e-3 * top, (B, (outs["chain"] - outs["launches"]).abs().max().item() / top)
        assert (outs["chain"] - outs["torch"]).abs().max().item() <= 1e-2 * top
    # one pair: a product that ends a block, the product behind the norm; widths that are and are not whole blocks of 16
    for K, N, N2, M in ((1000, 272, 96, 13), (520, 270, 40, 9), (300, 43, 33, 16)):
        w1, w2 = ternary_weight(K, N, 0.7, 1), ternary_weight(N, N2, 0.7, 2)
        d1, d2 = ops.DeviceWeight(PackedWeight.from_dense(w1), cuda), ops.DeviceWeight(PackedWeight.from_dense(w2), cuda)
        x = torch.randn((M, K), generator=g).half().to(cuda)
        res = torch.randn((M, N), generator=g).half().to(cuda)
        nw = (1 + 0.1 * torch.randn(N, generator=g)).half().to(cuda)
        sc1, sc2 = (0.05 + 0.01 * torch.rand(N, generator=g)).half().to(cuda), (0.5 + torch.rand(N2, generator=g)).half().to(cuda)
        y, image, squares = ops.spmm_chain(d1, x, sc1, residual=res, next_norm_weight=nw)
        assert torch.equal(y, ops.spmm(d1, x, sc1) + res)                      # the separate add, bit for bit
        assert torch.equal(image.t(), (y.float() * nw.float()).half())         # rows * weight, rounded once
        assert image.stride(0) == 16 and not image.as_strided((N, 16), (16, 1))[:, M:].any()
        blocks = -(-N // 16)
        padded = torch.zeros((M, blocks * 16), device=cuda)
        padded[:, :N] = y.float().pow(2)
        assert squares.shape[0] == blocks
        assert torch.allclose(squares[:, :M], padded.reshape(M, blocks, 16).sum(-1).t(), rtol=1e-5, atol=1e-6)
        out = ops.spmm_chain(d2, image, sc2, x_layout=1, squares_in=squares, eps=1e-5)
        h64 = y.double() * torch.rsqrt(y.double().pow(2).mean(-1, keepdim=True) + 1e-5) * nw.double()
        ref = (h64.cpu().numpy() @ w2.astype("float64")) * sc2.double().cpu().numpy()[None, :]
        assert max_rel_err(out.double().cpu().numpy(), ref, h64.cpu().numpy(), w2) <= 4e-3, (K, N, N2, M)
    with pytest.raises(RuntimeError, match="UNSUPPORTED"):
        ops.spmm_chain(d1, x[:5], sc1, residual=res[:5])                   # five rows: another kernel


def test_decode_kernels_against_fp32(cuda):
    """tl_rope_cache_update and tl_decode_attention alone, fp16 and fp32, against a float64 restatement."""
    from ternaryllm_amd import ops
    g = torch.Generator().manual_seed(9)
    for dtype, tol in ((torch.float32, 2e-5), (torch.float16, 3e-3)):
        for hd in (64, 128):
            B, H, S = 2, 3, 77
            pos = 41
            qkv = torch.randn((B, 3 * H * hd), generator=g).to(dtype).to(cuda)
            inv = 1.0 / (10000.0 ** (torch.arange(0, hd, 2, dtype=torch.float64) / hd))
            ang = torch.arange(S, dtype=torch.float64)[:, None] * inv[None, :]
            ang = torch.cat([ang, ang], -1)
            cos, sin = ang.cos().to(dtype).to(cuda), ang.sin().to(dtype).to(cuda)
            kc = torch.randn((B, H, S, hd), generator=g).to(dtype).to(cuda)
            vc = torch.randn((B, H, S, hd), generator=g).to(dtype).to(cuda)
            kc0, vc0 = kc.clone(), vc.clone()
            q = torch.empty((B, H, hd), dtype=dtype, device=cuda)
            p = torch.tensor([pos], dtype=torch.long, device=cuda)
            ops.rope_cache_update(qkv, cos, sin, p, q, kc, vc)
            x = qkv.double().view(B, 3, H, hd)
            c64, s64 = cos[pos].double(), sin[pos].double()
            rot = lambda t: t * c64 + torch.cat([-t[..., hd // 2:], t[..., : hd // 2]], -1) * s64
            assert (q.double() - rot(x[:, 0])).abs().max().item() <= tol * 4
            assert (kc[:, :, pos].double() - rot(x[:, 1])).abs().max().item() <= tol * 4
            assert torch.equal(vc[:, :, pos], qkv.view(B, 3, H, hd)[:, 2])
            keep = torch.ones(S, dtype=torch.bool, device=cuda)
            keep[pos] = False
            assert torch.equal(kc[:, :, keep], kc0[:, :, keep]) and torch.equal(vc[:, :, keep], vc0[:, :, keep])
            out = ops.decode_attention(q, kc, vc, p)
            sc = (q.double()[:, :, None, :] * kc.double()[:, :, : pos + 1]).sum(-1) / hd ** 0.5
            ref = (sc.softmax(-1)[..., None] * vc.double()[:, :, : pos + 1]).sum(2).reshape(B, H * hd)
            assert (out.double() - ref).abs().max().item() <= tol * 4
            outk = ops.decode_attention(q, kc, vc, p, kmajor=True)   # the same values as a K-major image
            assert outk.shape == (H * hd, B) and outk.stride(0) == 16 and torch.equal(outk.t(), out)


def test_decode_attention_over_a_long_cache(cuda):
    """One pass with running sums: no bound on the cache length (40 000 rows here), few rows, and a
    position past the end (all rows valid, nothing out of bounds)."""
    from ternaryllm_amd import ops
    g = torch.Generator().manual_seed(12)
    B, H, hd, S = 1, 2, 64, 40000
    q = torch.randn((B, H, hd), generator=g).to(torch.float16).to(cuda)
    kc = torch.randn((B, H, S, hd), generator=g).to(torch.float16).to(cuda)
    vc = torch.randn((B, H, S, hd), generator=g).to(torch.float16).to(cuda)
    for pos in (0, 2, 1023, S - 1, S + 5):
        n = min(pos, S - 1) + 1
        out = ops.decode_attention(q, kc, vc, torch.tensor([pos], dtype=torch.long, device=cuda))
        sc = (q.double()[:, :, None, :] * kc.double()[:, :, :n]).sum(-1) / hd ** 0.5
        ref = (sc.softmax(-1)[..., None] * vc.double()[:, :, :n]).sum(2).reshape(B, H * hd)
        assert (out.double() - ref).abs().max().item() <= 3e-3 * max(1.0, ref.abs().max().item()), pos


def test_decode_attention_ignores_what_lies_past_the_position(cuda):
    """Cache rows behind the position are not part of the result whatever they hold (the kernel may ask for some of
    them before it knows the position): NaN and infinities there change nothing, for 1 to 8 workgroups per head."""
    from ternaryllm_amd import ops
    g = torch.Generator().manual_seed(13)
    # (the second shape: more workgroups than compute units, two of which share one)
    for B, H, hd, S, positions in ((2, 4, 128, 700, (0, 5, 63, 64, 127, 128, 300, 698)), (12, 32, 128, 330, (0, 1, 127, 128, 200, 329))):
        _attention_ignores_rows_past(cuda, g, B, H, hd, S, positions)


def _attention_ignores_rows_past(cuda, g, B, H, hd, S, positions):
    from ternaryllm_amd import ops
    q = torch.randn((B, H, hd), generator=g).to(torch.float16).to(cuda)
    kc = torch.randn((B, H, S, hd), generator=g).to(torch.float16).to(cuda)
    vc = torch.randn((B, H, S, hd), generator=g).to(torch.float16).to(cuda)
    for pos in positions:
        p = torch.tensor([pos], dtype=torch.long, device=cuda)
        kz, vz, kn, vn = kc.clone(), vc.clone(), kc.clone(), vc.clone()
        kz[:, :, pos + 1:] = 0
        vz[:, :, pos + 1:] = 0
        kn[:, :, pos + 1:] = float("nan")
        vn[:, :, pos + 1:] = float("inf")
        for splits in (1, 3, 8):
            assert torch.equal(ops.decode_attention(q, kn, vn, p, splits=splits), ops.decode_attention(q, kz, vz, p, splits=splits)), (pos, splits)
        n = pos + 1
        sc = (q.double()[:, :, None, :] * kc.double()[:, :, :n]).sum(-1) / hd ** 0.5
        ref = (sc.softmax(-1)[..., None] * vc.double()[:, :, :n]).sum(2).reshape(B, H * hd)
        out = ops.decode_attention(q, kn, vn, p, splits=1)
        assert (out.double() - ref).abs().max().item() <= 3e-3 * max(1.0, ref.abs().max().item()), pos


def test_split_attention_and_its_fold_inside_the_output_projection(cuda, oracle):
    """tl_decode_attention_split: the cache rows of a head shared out among 1-8 workgroups, folded by the second
    launch, against the single-pass kernel and a float64 restatement (few rows, pieces without rows, a position
    past the end); and the pieces folded inside the output projection (tl_spmv_attn_combine) against the
    separate fold followed by the plain product."""
    from tests.util import knobs, max_rel_err, ternary_weight
    from ternaryllm_amd import ops
    from ternaryllm_amd.packing import PackedWeight
    g = torch.Generator().manual_seed(23)
    for dtype, tol in ((torch.float16, 3e-3), (torch.float32, 2e-5)):
        for B, H, hd, S in ((1, 32, 128, 700), (2, 3, 64, 90)):
            q = torch.randn((B, H, hd), generator=g).to(dtype).to(cuda)
            kc = torch.randn((B, H, S, hd), generator=g).to(dtype).to(cuda)
            vc = torch.randn((B, H, S, hd), generator=g).to(dtype).to(cuda)
            for pos in (0, 2, 6, S // 2, S - 1, S + 3):
                n = min(pos, S - 1) + 1
                p = torch.tensor([pos], dtype=torch.long, device=cuda)
                sc = (q.double()[:, :, None, :] * kc.double()[:, :, :n]).sum(-1) / hd ** 0.5
                ref = (sc.softmax(-1)[..., None] * vc.double()[:, :, :n]).sum(2).reshape(B, H * hd)
                single = ops.decode_attention(q, kc, vc, p, splits=1)
                for splits in (2, 3, 8):
                    out = ops.decode_attention(q, kc, vc, p, splits=splits)
                    assert (out.double() - ref).abs().max().item() <= tol * max(1.0, ref.abs().max().item()), (pos, splits)
                    assert (out.double() - single.double()).abs().max().item() <= tol * max(1.0, ref.abs().max().item())
                    outk = ops.decode_attention(q, kc, vc, p, kmajor=True, splits=splits)
                    assert torch.equal(outk.t(), out)
                    # the pieces folded by the last workgroup to finish (the default) and by a launch of their own;
                    # the counters of the first form are left at zero: a call with another number of pieces follows at once
                    assert torch.equal(out, ops.decode_attention(q, kc, vc, p, splits=splits, fold_inside=False)), (pos, splits)
                assert all(int(c.abs().max()) == 0 for c in ops._attn_arrivals.values())
        # the output projection with the fold inside, batch 1
        H, hd, S, N = 32, 128, 700, 272
        K = H * hd
        w = ternary_weight(K, N, 0.7, 77)
        dw = ops.DeviceWeight(PackedWeight.from_dense(w), cuda)
        scale = (0.5 + torch.rand(N, generator=g)).to(dtype).to(cuda)
        q = torch.randn((1, H, hd), generator=g).to(dtype).to(cuda)
        kc = torch.randn((1, H, S, hd), generator=g).to(dtype).to(cuda)
        vc = torch.randn((1, H, S, hd), generator=g).to(dtype).to(cuda)
        for pos in (1, 333, S - 1):
            p = torch.tensor([pos], dtype=torch.long, device=cuda)
            for splits in (1, 2, 4, 8):
                pieces = ops.decode_attention_pieces(q, kc, vc, p, splits=splits)
                assert pieces.shape == (H, splits, hd + 4)
                out = ops.spmv_attn_combine(dw, pieces, hd, dtype, scale)
                a = ops.decode_attention(q, kc, vc, p, splits=splits)
                unfused = ops.spmm(dw, a, scale)
                # the folded row may differ from the separately folded one in its last bit (fp32 sums in another order)
                assert max_rel_err(out.double().cpu().numpy(), unfused.double().cpu().numpy(), a.double().cpu().numpy(), w) <= tol
                res = torch.randn(N, generator=g).to(dtype).to(cuda)
                summed = ops.spmv_attn_combine(dw, pieces, hd, dtype, scale, residual=res)
                assert torch.equal(summed, out + res[None])
                # the kernel that folds the pieces of each wave's own tiles (the default where the block fits it) and
                # the one that folds all of them first: the same row, summed over K in another order
                with knobs(TL_SPMV_TILES="0"):
                    other = ops.spmv_attn_combine(dw, pieces, hd, dtype, scale)
                    assert max_rel_err(other.double().cpu().numpy(), out.double().cpu().numpy(), a.double().cpu().numpy(), w) <= tol, (pos, splits)
                    assert torch.equal(ops.spmv_attn_combine(dw, pieces, hd, dtype, scale, residual=res), other + res[None])
                # ... and what it leaves for the next norm, as tl_spmv_add_norm leaves it
                nw = (1 + 0.1 * torch.randn(N, generator=g)).to(dtype).to(cuda)
                if splits == 8:   # that many pieces of all of K do not fit the kernel's LDS
                    with pytest.raises(RuntimeError, match="UNSUPPORTED"):
                        ops.spmv_attn_combine(dw, pieces, hd, dtype, scale, residual=res, next_norm_weight=nw)
                    continue
                y, image, squares = ops.spmv_attn_combine(dw, pieces, hd, dtype, scale, residual=res, next_norm_weight=nw)
                assert torch.equal(y, summed)
                assert torch.equal(image, (y.float() * nw.float()[None]).to(dtype))
                want = y[0].double().pow(2).view(N // 16, 16).sum(1)
                assert squares.shape == (N // 16,) and (squares.double() - want).abs().max().item() <= 1e-6 * want.max().item()
        # a weight whose tiles are too many for two per wave at 512 threads: the other kernel takes the product, and
        # there is none that leaves the next norm's inputs
        low = ops.DeviceWeight(PackedWeight.from_dense(w, tile_rows=120), cuda)
        with knobs(TL_SPMV_WIDE="0"):
            base = ops.spmv_attn_combine(low, pieces, hd, dtype, scale)
            assert max_rel_err(base.double().cpu().numpy(), unfused.double().cpu().numpy(), a.double().cpu().numpy(), w) <= tol
            assert torch.equal(ops.spmv_attn_combine(low, pieces, hd, dtype, scale, residual=res), base + res[None])
            with pytest.raises(RuntimeError, match="UNSUPPORTED"):
                ops.spmv_attn_combine(low, pieces, hd, dtype, scale, residual=res, next_norm_weight=nw)
    with pytest.raises(ValueError):
        ops.spmv_attn_combine(dw, torch.zeros((H, 2, hd + 3), device=cuda), hd, torch.float16)
    with pytest.raises(ValueError, match="splits"):
        ops.decode_attention(q, kc, vc, p, splits=9)


def test_attention_that_rotates_and_updates_the_cache_itself(cuda):
    """tl_decode_attention_rope against tl_rope_cache_update followed by tl_decode_attention_split: the output (row-major,
    K-major, and left in pieces) and both caches bit for bit -- first, middle and last cache row, one and several
    workgroups per head, and a position past the cache, which writes nothing."""
    from ternaryllm_amd import ops
    g = torch.Generator().manual_seed(29)
    for dtype in (torch.float16, torch.float32):
        # (the last two: more workgroups than the chip has compute units, which for fp16 is a kernel of its own)
        for B, H, hd, S in ((1, 32, 128, 300), (3, 5, 64, 150), (2, 2, 256, 70), (9, 32, 128, 150), (18, 16, 64, 90)):
            inv = 1.0 / (10000 ** (torch.arange(0, hd, 2).double() / hd))
            ang = torch.arange(S).double()[:, None] * inv[None, :]
            cos = torch.cat([ang.cos(), ang.cos()], 1).to(dtype).to(cuda)
            sin = torch.cat([ang.sin(), ang.sin()], 1).to(dtype).to(cuda)
            kc0 = torch.randn((B, H, S, hd), generator=g).to(dtype).to(cuda)
            vc0 = torch.randn((B, H, S, hd), generator=g).to(dtype).to(cuda)
            for pos in (0, 1, S // 2, S - 1, S):
                qkv = torch.randn((B, 3 * H * hd), generator=g).to(dtype).to(cuda)
                p = torch.tensor([pos], dtype=torch.long, device=cuda)
                for splits in (1, 3, 8):
                    kc1, vc1, kc2, vc2 = kc0.clone(), vc0.clone(), kc0.clone(), vc0.clone()
                    if pos < S:
                        # the row the token will take holds something else: it must not be read
                        kc1[:, :, pos], kc2[:, :, pos] = 7.0, 7.0
                        vc1[:, :, pos], vc2[:, :, pos] = -3.0, -3.0
                    q = torch.zeros((B, H, hd), dtype=dtype, device=cuda)
                    ops.rope_cache_update(qkv, cos, sin, p, q, kc1, vc1)
                    fused = ops.decode_attention(None, kc2, vc2, p, splits=splits, fresh=(qkv, cos, sin))
                    assert torch.equal(kc1, kc2) and torch.equal(vc1, vc2), (dtype, pos, splits)
                    if pos < S:
                        assert torch.equal(fused, ops.decode_attention(q, kc1, vc1, p, splits=splits)), (dtype, B, pos, splits)
                        assert not torch.equal(kc2[:, :, pos], kc0[:, :, pos])
                    else:
                        assert torch.equal(kc2, kc0) and torch.isfinite(fused).all()
                    kc3, vc3 = kc0.clone(), vc0.clone()
                    assert torch.equal(ops.decode_attention(None, kc3, vc3, p, kmajor=True, splits=splits, fresh=(qkv, cos, sin)).t(), fused)
                    assert torch.equal(kc3, kc2)
                    kc5, vc5 = kc0.clone(), vc0.clone()
                    assert torch.equal(ops.decode_attention(None, kc5, vc5, p, splits=splits, fresh=(qkv, cos, sin), fold_inside=False), fused)
                    if pos < S:
                        kc4, vc4 = kc0.clone(), vc0.clone()
                        pieces = ops.decode_attention_pieces(None, kc4, vc4, p, splits=splits, fresh=(qkv, cos, sin))
                        assert torch.equal(pieces[..., :hd + 2], ops.decode_attention_pieces(q, kc1, vc1, p, splits=splits)[..., :hd + 2])
                        assert torch.equal(kc4, kc2) and torch.equal(vc4, vc2)
    with pytest.raises(ValueError, match="q, or fresh"):
        ops.decode_attention(q, kc1, vc1, p, fresh=(qkv, cos, sin))
    with pytest.raises(ValueError, match="rotary tables"):
        ops.decode_attention(None, kc1, vc1, p, fresh=(qkv, cos[:-1], sin))


def test_add_rmsnorm_and_silu_mul(cuda):
    from ternaryllm_amd import ops
    g = torch.Generator().manual_seed(10)
    for dtype, tol in ((torch.float32, 1e-5), (torch.float16, 2e-3)):
        for rows, width in ((1, 4096), (5, 300), (16, 11008)):
            x = torch.randn((rows, width), generator=g).to(dtype).to(cuda)
            y = torch.randn((rows, width), generator=g).to(dtype).to(cuda)
            w = (1 + 0.1 * torch.randn(width, generator=g)).to(dtype).to(cuda)
            xs, h = ops.add_rmsnorm(x, y, w, 1e-5)
            assert torch.equal(xs, x + y)
            ref = xs.double() * torch.rsqrt(xs.double().pow(2).mean(-1, keepdim=True) + 1e-5) * w.double()
            assert (h.double() - ref).abs().max().item() <= tol * ref.abs().max().item()
            xk, hk = ops.add_rmsnorm(x, y, w, 1e-5, kmajor=True)     # the same values as a K-major image
            assert torch.equal(xk, xs) and hk.shape == (width, rows) and hk.stride(0) % 16 == 0 and torch.equal(hk.t(), h)
            x0, h0 = ops.add_rmsnorm(x, None, w, 1e-5)
            assert x0 is x
            ref0 = x.double() * torch.rsqrt(x.double().pow(2).mean(-1, keepdim=True) + 1e-5) * w.double()
            assert (h0.double() - ref0).abs().max().item() <= tol * ref0.abs().max().item()
            gu = torch.randn((rows, 2 * width), generator=g).to(dtype).to(cuda)
            out = ops.silu_mul(gu)
            refs = torch.nn.functional.silu(gu[:, :width].double()) * gu[:, width:].double()
            assert (out.double() - refs).abs().max().item() <= tol * refs.abs().max().item()
            assert torch.equal(ops.silu_mul(gu, kmajor=True).t(), out)


@pytest.mark.parametrize("dtype,tol", [(torch.float16, 2e-3), (torch.float32, 1e-5)])
def test_fused_producers_of_the_single_row_product(cuda, oracle, dtype, tol):
    """tl_spmv_fused: the residual add + RMSNorm and the SiLU gate computed inside the product's kernel, against a
    float64 restatement and against the separate kernels followed by the plain product; the RMSNorm whose factor is
    applied to the sums, and the residual add in a product's epilogue."""
    from tests.util import knobs, max_rel_err, ternary_weight
    from ternaryllm_amd import ops
    from ternaryllm_amd.packing import PackedWeight
    g = torch.Generator().manual_seed(14)
    for K, N in ((4096, 272), (11008, 96), (1000, 40)):   # one group of tiles; many tiles; a ragged last tile and block
        w = ternary_weight(K, N, 0.7, K + N)
        dw = ops.DeviceWeight(PackedWeight.from_dense(w), cuda)
        sc = (0.5 + torch.rand(N, generator=g)).to(dtype).to(cuda)
        x = torch.randn(K, generator=g).to(dtype).to(cuda)
        y = torch.randn(K, generator=g).to(dtype).to(cuda)
        nw = (1 + 0.1 * torch.randn(K, generator=g)).to(dtype).to(cuda)
        gu = torch.randn(2 * K, generator=g).to(dtype).to(cuda)
        wd = w.astype("float64")
        for second in (y, None):
            out, s = ops.spmv_fused(dw, "add_rmsnorm", x, second, nw, 1e-5, sc, want_sum=True)
            s_ref = (x + second) if second is not None else x
            assert torch.equal(s, s_ref)
            h64 = s_ref.double() * torch.rsqrt(s_ref.double().pow(2).mean() + 1e-5) * nw.double()
            ref = (h64.cpu().numpy()[None, :] @ wd) * sc.double().cpu().numpy()[None, :]
            # the activation row is rounded to its type before the product: allow for that rounding on top of the product's
            assert max_rel_err(out.double().cpu().numpy(), ref, h64.cpu().numpy()[None, :], w) <= 2 * tol
            _, h = ops.add_rmsnorm(x[None], second[None] if second is not None else None, nw, 1e-5)
            unfused = ops.spmm(dw, h, sc)
            assert max_rel_err(out.double().cpu().numpy(), unfused.double().cpu().numpy(), h.double().cpu().numpy(), w) <= tol
        out = ops.spmv_fused(dw, "silu_gate", gu, scale=sc)
        a64 = torch.nn.functional.silu(gu[:K].double()) * gu[K:].double()
        ref = (a64.cpu().numpy()[None, :] @ wd) * sc.double().cpu().numpy()[None, :]
        assert max_rel_err(out.double().cpu().numpy(), ref, a64.cpu().numpy()[None, :], w) <= 2 * tol
        act = ops.silu_mul(gu[None])
        unfused = ops.spmm(dw, act, sc)    # same roundings of the row; the plain product may sum in another order
        assert max_rel_err(out.double().cpu().numpy(), unfused.double().cpu().numpy(), act.double().cpu().numpy(), w) <= tol
        # RMSNorm with the factor applied to the sums (both single-row kernels), and the residual add in the epilogue
        for second in (None, y):
            base = x if second is None else x + second
            h64 = base.double() * torch.rsqrt(base.double().pow(2).mean() + 1e-5) * nw.double()
            ref = (h64.cpu().numpy()[None, :] @ wd) * sc.double().cpu().numpy()[None, :]
            for setting in ({}, {"TL_SPMV_TILES": "0"}, {"TL_SPMV_WIDE": "0"}, {"TL_SPMV_WIDE": "1"}):
                with knobs(**setting):
                    out = ops.spmv_fused(dw, "rmsnorm", base, None, nw, 1e-5, sc)
                    assert max_rel_err(out.double().cpu().numpy(), ref, h64.cpu().numpy()[None, :], w) <= 2 * tol, (K, N, setting)
                    if N % 2 == 0:
                        assert torch.equal(ops.spmv_fused(dw, "rmsnorm", base, None, nw, 1e-5, sc, gated=True), ops.silu_mul(out, pairs=True))
                    res = torch.randn(N, generator=g).to(dtype).to(cuda)
                    act = torch.randn((1, K), generator=g).to(dtype).to(cuda)
                    assert torch.equal(ops.spmv_add(dw, act, res, sc), ops.spmm(dw, act, sc) + res[None]), (K, N, setting)
        with pytest.raises(ValueError, match="residual add belongs"):
            ops.spmv_fused(dw, "rmsnorm", x, y, nw, 1e-5, sc)
    with pytest.raises(RuntimeError, match="UNSUPPORTED"):   # a tile height that is not whole 16-byte pieces: the separate kernels are the way then
        odd = ops.DeviceWeight(PackedWeight.from_dense(ternary_weight(1000, 40, 0.7, 3), tile_rows=250), cuda)
        ops.spmv_fused(odd, "silu_gate", torch.zeros(2000, dtype=dtype, device=cuda))


@pytest.mark.parametrize("dtype,tol", [(torch.float16, 2e-3), (torch.float32, 1e-5)])
def test_single_row_product_prepares_the_next_norm(cuda, dtype, tol):
    """tl_spmv_add_norm and TL_PRODUCER_RMSNORM_SUMS: the product that ends a block leaves, beside the new residual
    row, that row times the next norm's weight and the sums of its squares over runs of 16; the product behind the
    norm starts from those.  The row bit for bit against tl_spmv_add, the image against the rounded product of row
    and weight, the sums and the second product against float64 and against TL_PRODUCER_RMSNORM on the row."""
    from tests.util import knobs, max_rel_err, ternary_weight
    from ternaryllm_amd import ops
    from ternaryllm_amd.packing import PackedWeight
    g = torch.Generator().manual_seed(77)
    eps = 1e-5
    for K1, N1, N2 in ((4096, 1024, 272), (1000, 1000, 40), (11008, 4096, 96)):   # whole blocks; a ragged last block and tile; many tiles
        w1, w2 = ternary_weight(K1, N1, 0.7, K1 + N1), ternary_weight(N1, N2, 0.66, N1 + N2)
        d1, d2 = (ops.DeviceWeight(PackedWeight.from_dense(w), cuda) for w in (w1, w2))
        s1 = (0.01 + 0.01 * torch.rand(N1, generator=g)).to(dtype).to(cuda)
        s2 = (0.5 + torch.rand(N2, generator=g)).to(dtype).to(cuda)
        act = torch.randn((1, K1), generator=g).to(dtype).to(cuda)
        res = torch.randn(N1, generator=g).to(dtype).to(cuda)
        nw = (1 + 0.1 * torch.randn(N1, generator=g)).to(dtype).to(cuda)
        for setting in ({}, {"TL_SPMV_WIDE": "1"}) if K1 == 11008 else ({}, {"TL_SPMV_WIDE": "0"}):
            with knobs(**setting):
                y, image, squares = ops.spmv_add(d1, act, res, s1, next_norm_weight=nw)
                assert torch.equal(y, ops.spmv_add(d1, act, res, s1)), (K1, N1, setting)
                assert torch.equal(image, (y.float() * nw.float()[None]).to(dtype)) if dtype == torch.float16 else torch.equal(image, y * nw[None])
                blocks = (N1 + 15) // 16
                padded = torch.zeros(blocks * 16, dtype=torch.float64, device=cuda)
                padded[:N1] = y[0].double()
                want = padded.view(blocks, 16).pow(2).sum(1)
                assert squares.shape == (blocks,) and (squares.double() - want).abs().max().item() <= 1e-6 * want.max().item()
                h64 = y[0].double() * torch.rsqrt(y[0].double().pow(2).mean() + eps) * nw.double()
                ref = (h64.cpu().numpy()[None, :] @ w2.astype("float64")) * s2.double().cpu().numpy()[None, :]
                out = ops.spmv_fused(d2, "rmsnorm_sums", image, squares, None, eps, s2)
                assert max_rel_err(out.double().cpu().numpy(), ref, h64.cpu().numpy()[None, :], w2) <= 2 * tol, (K1, N1, N2, setting)
                other = ops.spmv_fused(d2, "rmsnorm", y, None, nw, eps, s2)
                assert max_rel_err(out.double().cpu().numpy(), other.double().cpu().numpy(), h64.cpu().numpy()[None, :], w2) <= tol
                assert torch.equal(ops.spmv_fused(d2, "rmsnorm_sums", image, squares, None, eps, s2, gated=True), ops.silu_mul(out, pairs=True))
        with pytest.raises(ValueError, match="one float32 sum"):
            ops.spmv_fused(d2, "rmsnorm_sums", image, squares[:-1].contiguous(), None, eps, s2)
        with pytest.raises(ValueError, match="already holds"):
            ops.spmv_fused(d2, "rmsnorm_sums", image, squares, nw, eps, s2)
    # 86 tiles are more than the eight waves of the tile-per-wave kernel own at 512 threads, and the other kernel has no such epilogue
    low = ops.DeviceWeight(PackedWeight.from_dense(ternary_weight(4096, 64, 0.7, 3), tile_rows=48), cuda)
    act, res, nw = (torch.ones(n, dtype=dtype, device=cuda) for n in (4096, 64, 64))
    with knobs(TL_SPMV_WIDE="0"):
        assert torch.equal(ops.spmv_add(low, act, res), ops.spmm(low, act[None]) + res[None])
        with pytest.raises(RuntimeError, match="UNSUPPORTED"):
            ops.spmv_add(low, act, res, next_norm_weight=nw)
        with pytest.raises(RuntimeError, match="UNSUPPORTED"):
            ops.spmv_fused(low, "rmsnorm_sums", act, torch.ones(256, dtype=torch.float32, device=cuda), None, eps)
    # wide outputs.  More than four blocks per compute unit: where four workgroups with an fp32 row's images do not fit a
    # compute unit's LDS, fewer of them share it.  Between one and three: workgroups of nine waves where K's 17 tiles
    # are then two per wave at most.
    units = torch.cuda.get_device_properties(cuda).multi_processor_count
    for K, halves in ((4096, 9), (1000, 9), (4096, 3)):
        N = 16 * (halves * units // 2) + 6
        w = ternary_weight(K, N, 0.66, K + 1)
        dw = ops.DeviceWeight(PackedWeight.from_dense(w), cuda)
        sc = (0.5 + torch.rand(N, generator=g)).to(dtype).to(cuda)
        y = torch.randn(K, generator=g).to(dtype).to(cuda)
        nw = (1 + 0.1 * torch.randn(K, generator=g)).to(dtype).to(cuda)
        image = (y.float() * nw.float()).to(dtype)[None]
        squares = torch.nn.functional.pad(y.float().pow(2), (0, -K % 16)).view(-1, 16).sum(1).contiguous()
        h64 = y.double() * torch.rsqrt(y.double().pow(2).mean() + eps) * nw.double()
        ref = (image[0].double() * torch.rsqrt(y.double().pow(2).mean() + eps)).cpu().numpy()[None, :] @ w.astype("float64") * sc.double().cpu().numpy()[None, :]
        out = ops.spmv_fused(dw, "rmsnorm_sums", image, squares, None, eps, sc)
        assert max_rel_err(out.double().cpu().numpy(), ref, h64.cpu().numpy()[None, :], w) <= 2 * tol, K
        assert torch.equal(ops.spmv_fused(dw, "rmsnorm_sums", image, squares, None, eps, sc, gated=True), ops.silu_mul(out, pairs=True))


def test_silu_gate_in_the_epilogue_of_the_gate_up_product(cuda):
    """tl_spmm_gated / tl_spmv_fused_gated on a weight whose columns are (gate, up) pairs against the product followed
    by tl_silu_mul_pairs: bit for bit -- one row (both single-row kernels, with and without a producer), 9 to 16 fp16
    rows on a wide output (row-major and as a K-major image with zeroed padding rows), more than 48 rows (the
    row-parallel kernel), and the shapes without the epilogue, which take the two launches."""
    import ctypes
    from tests.util import knobs, ternary_weight
    from ternaryllm_amd import _lib, ops
    from ternaryllm_amd.packing import PackedWeight
    g = torch.Generator().manual_seed(31)
    L = _lib.lib()

    def fused_rc(dw, x, M, layout=0):
        """status of the one-launch call by itself (ops.spmm_gated falls back silently)"""
        # (a K-major image has 16 rows per column whatever M is)
        out = torch.empty((M, dw.columns // 2) if layout == 0 else (dw.columns // 2, 16), dtype=x.dtype, device=cuda)
        ws = torch.empty(1 << 22, dtype=torch.uint8, device=cuda)
        return L.tl_spmm_gated(ctypes.byref(dw.header), dw.blob.data_ptr(), x.data_ptr(), ops._code(x.dtype, "x"), 0, dw.inners, M,
                               out.data_ptr(), ops._code(x.dtype, "x"), dw.columns // 2 if layout == 0 else 16, layout, None, 0,
                               ws.data_ptr(), ws.numel(), None)

    # the separate operator on pairs
    gu = torch.randn((5, 600), generator=g).half().to(cuda)
    ref = (torch.nn.functional.silu(gu[:, 0::2].float()).half().float() * gu[:, 1::2].float()).half()
    assert torch.equal(ops.silu_mul(gu, pairs=True), ref)
    assert torch.equal(ops.silu_mul(gu, kmajor=True, pairs=True).t(), ref)
    for dtype in (torch.float16, torch.float32):
        for K, N in ((4096, 544), (11008, 96), (1000, 40)):   # the tile-per-wave kernel; a block too tall for it at 512 threads; ragged
            w = ternary_weight(K, N, 0.7, K + N)
            dw = ops.DeviceWeight(PackedWeight.from_dense(w), cuda)
            sc = (0.5 + torch.rand(N, generator=g)).to(dtype).to(cuda)
            x = torch.randn((1, K), generator=g).to(dtype).to(cuda)
            want = ops.silu_mul(ops.spmm(dw, x, sc), pairs=True)
            assert fused_rc(dw, x, 1) == 0
            for setting in ({}, {"TL_SPMV_TILES": "0"}):
                with knobs(**setting):
                    assert torch.equal(ops.spmm_gated(dw, x, sc), ops.silu_mul(ops.spmm(dw, x, sc), pairs=True)), (dtype, K, N, setting)
            # with the residual add + RMSNorm in front
            y = torch.randn(K, generator=g).to(dtype).to(cuda)
            nw = (1 + 0.1 * torch.randn(K, generator=g)).to(dtype).to(cuda)
            plain, s1 = ops.spmv_fused(dw, "add_rmsnorm", x[0], y, nw, 1e-5, sc, want_sum=True)
            gated, s2 = ops.spmv_fused(dw, "add_rmsnorm", x[0], y, nw, 1e-5, sc, want_sum=True, gated=True)
            assert torch.equal(s1, s2) and gated.shape == (1, N // 2)
            assert torch.equal(gated, ops.silu_mul(plain, pairs=True))
    # 9 to 16 fp16 rows, an output wide enough for the eight-rows-per-lane kernel
    units = torch.cuda.get_device_properties(cuda).multi_processor_count
    K, N = 520, 64 * units + 48
    w = ternary_weight(K, N, 0.8, 5)
    dw = ops.DeviceWeight(PackedWeight.from_dense(w), cuda)
    sc = (0.5 + torch.rand(N, generator=g)).half().to(cuda)
    for M in (16, 9, 13):
        x = torch.randn((M, K), generator=g).half().to(cuda)
        want = ops.silu_mul(ops.spmm(dw, x, sc), pairs=True)
        assert fused_rc(dw, x, M) == 0 and fused_rc(dw, x, M, layout=1) == 0
        assert torch.equal(ops.spmm_gated(dw, x, sc), want), M
        image = ops.spmm_gated(dw, x, sc, kmajor=True)
        assert torch.equal(image.t(), want)
        assert image.stride(0) == 16 and not image.as_strided((N // 2, 16), (16, 1))[:, M:].any()   # the padding rows of the image
        xk, _ = ops._kmajor_image(M, K, x)
        xk[:, :M] = x.t()
        assert torch.equal(ops.spmm_gated(dw, xk[:, :M], sc, x_layout=1), want)
    # shapes whose kernels have no such epilogue: same result from two launches
    x32 = torch.randn((16, K), generator=g).to(cuda)
    assert fused_rc(dw, x32, 16) == _lib.TL_ERR_UNSUPPORTED
    for x in (torch.randn((5, K), generator=g).half().to(cuda), torch.randn((3, K), generator=g).half().to(cuda), x32):
        assert fused_rc(dw, x, x.shape[0]) == _lib.TL_ERR_UNSUPPORTED
        assert torch.equal(ops.spmm_gated(dw, x, sc.to(x.dtype)), ops.silu_mul(ops.spmm(dw, x, sc.to(x.dtype)), pairs=True))
    # 17 to 48 fp16 rows on a wide output: the eight-rows-per-lane kernel, one workgroup per 16 rows
    x40 = torch.randn((40, K), generator=g).half().to(cuda)
    assert fused_rc(dw, x40, 40) == 0
    assert torch.equal(ops.spmm_gated(dw, x40, sc), ops.silu_mul(ops.spmm(dw, x40, sc), pairs=True))
    narrow = ops.DeviceWeight(PackedWeight.from_dense(ternary_weight(K, 96, 0.8, 6)), cuda)
    assert fused_rc(narrow, torch.zeros((16, K), dtype=torch.float16, device=cuda), 16) == _lib.TL_ERR_UNSUPPORTED
    # more than 48 rows: the row-parallel kernel with the pair epilogue, whole output tiles and tiles that the matrix
    # edge cuts, with and without K tiles shared out among the workgroups
    sc96 = (0.5 + torch.rand(96, generator=g)).half().to(cuda)
    for dtype in (torch.float16, torch.float32):
        for M in (60, 300, 1100):
            x = torch.randn((M, K), generator=g).to(dtype).to(cuda)
            for weight, scale in ((dw, sc), (narrow, sc96)):
                assert fused_rc(weight, x, M) == 0
                for setting in ({}, {"TL_ROWS_SPLIT": "0"}):
                    with knobs(**setting):
                        got = ops.spmm_gated(weight, x, scale.to(dtype))
                        want = ops.silu_mul(ops.spmm(weight, x, scale.to(dtype)), pairs=True)
                    assert got.shape == (M, weight.columns // 2)
                    assert torch.equal(got, want), (dtype, M, weight.columns, setting)
    image = torch.empty((dw.columns // 2, 64), dtype=torch.float16, device=cuda)
    x60 = torch.zeros((60, K), dtype=torch.float16, device=cuda)
    assert L.tl_spmm_gated(ctypes.byref(dw.header), dw.blob.data_ptr(), x60.data_ptr(), 1, 0, K, 60, image.data_ptr(), 1, 64, 1, None, 0,
                           None, 0, None) == _lib.TL_ERR_UNSUPPORTED   # no K-major image of that many rows
    odd = ops.DeviceWeight(PackedWeight.from_dense(ternary_weight(K, 33, 0.8, 7)), cuda)
    with pytest.raises(ValueError, match="pairs"):
        ops.spmm_gated(odd, torch.zeros((1, K), dtype=torch.float16, device=cuda))


def test_fused_single_row_step_equals_the_unfused_one(tiny, cuda):
    """Batch 1: the step with the norms and the SiLU gate folded into the products against the same step on
    separate kernels, eager and as a replayed graph."""
    g = torch.Generator().manual_seed(21)
    tokens = torch.randint(0, tiny.config.vocab_size, (1, 30), generator=g).to(cuda)
    assert tiny.fused_decode
    outs = {}
    assert not tiny.split_attention   # a short cache: one workgroup per head; the split form is forced below
    assert tiny.row_chain
    assert tiny.piece_fold == 2
    # "plain": the products behind a norm multiply the row and sum its squares themselves; "whole": one workgroup per
    # head writes the attention's output row (the default leaves two pieces per head for the o projection to fold);
    # "split": the rows of a head shared out as for a long cache, the pieces folded by the last workgroup to finish;
    # "split4": four pieces per head folded by the o projection
    for fused in (False, True, "split", "split4", "plain", "whole"):
        tiny.fused_decode = bool(fused)
        tiny.split_attention = fused in ("split", "split4")
        tiny.row_chain = fused != "plain"
        tiny.piece_fold = 0 if fused in ("whole", "split") else 2
        assert not fused or tiny.pieces_per_head() == {True: 2, "split4": 4}.get(fused, 0)
        tiny._graph = None
        tiny.prefill(tokens[:, :28])
        st = tiny._decode_state(1)
        logits = []
        for j in range(2):
            st["token"].copy_(tokens[:, 28 + j])
            st["pos"].fill_(28 + j)
            st["mask"].copy_((torch.arange(tiny.max_seq_len, device=cuda) <= 28 + j)[None, None, None])
            logits.append(tiny._decode_step(st["token"], st["pos"], st["mask"]).float())
        outs[fused] = torch.stack(logits)
        assert tiny.row_chain == (fused != "plain") and tiny.piece_fold == (0 if fused in ("whole", "split") else 2)   # no step fell back
    tiny.piece_fold = 2
    tiny.fused_decode = True
    tiny.split_attention = False
    tiny.row_chain = True
    tiny._state = None
    tiny._graph = None
    assert (outs[True] - outs[False]).abs().max().item() <= 2e-3 * outs[False].abs().max().item()
    assert (outs["plain"] - outs[False]).abs().max().item() <= 2e-3 * outs[False].abs().max().item()
    assert (outs["split"] - outs[False]).abs().max().item() <= 2e-3 * outs[False].abs().max().item()
    assert (outs["whole"] - outs[False]).abs().max().item() <= 2e-3 * outs[False].abs().max().item()
    assert (outs["split4"] - outs[False]).abs().max().item() <= 2e-3 * outs[False].abs().max().item()
    eager = tiny.generate(tokens, 10, use_graph=False)
    graphed = tiny.generate(tokens, 10, use_graph=True)
    again = tiny.generate(tokens, 10, use_graph=True)
    assert torch.equal(eager, graphed) and torch.equal(eager, again)
    # the split attention under a captured graph, replayed: four pieces per head folded by the o projection, then the
    # pieces folded by the last workgroup to finish
    for fold in (2, 0):
        tiny._graph = None
        tiny._state = None
        tiny.split_attention = True
        tiny.piece_fold = fold
        split_eager = tiny.generate(tokens, 10, use_graph=False)
        split_graphed = tiny.generate(tokens, 10, use_graph=True)
        split_again = tiny.generate(tokens, 10, use_graph=True)
        assert tiny.piece_fold == fold and tiny.row_chain
        tiny.split_attention = False
        tiny.piece_fold = 2
        assert torch.equal(split_eager, split_graphed) and torch.equal(split_eager, split_again)
    tiny._graph = None
    tiny._state = None


def test_greedy_advance_is_argmax_position_and_mask_in_one_launch(cuda):
    """tl_greedy_advance against torch.argmax (first of equal values, NaN above every number), with the position
    moved on and held at its maximum and the mask bit set."""
    from ternaryllm_amd import ops
    g = torch.Generator().manual_seed(9)
    for dtype in (torch.float16, torch.float32):
        for B, V in ((1, 32000), (3, 320), (16, 1031)):
            logits = torch.randn((B, V), generator=g).to(dtype).to(cuda)
            logits[0, V // 3] = logits[0, V // 2] = logits[0].max() + 1      # a tie: the first one wins
            if B > 1:
                logits[1, 7] = float("nan")
                logits[1, V - 1] = float("nan")
            token = torch.full((B,), -5, dtype=torch.long, device=cuda)
            pos = torch.tensor([10], dtype=torch.long, device=cuda)
            mask = torch.zeros((1, 1, 1, 13), dtype=torch.bool, device=cuda)
            for expect in (11, 12, 12):                                      # held at max_pos = 12
                ops.greedy_advance(logits, token, pos, 12, mask)
                assert torch.equal(token, logits.argmax(-1)), (dtype, B, V)
                assert int(pos) == expect and bool(mask.view(-1)[expect])
            assert mask.view(-1).nonzero().flatten().tolist() == [11, 12]
            only = torch.zeros(B, dtype=torch.long, device=cuda)
            ops.greedy_advance(logits, only)                                  # the argmax alone
            assert torch.equal(only, logits.argmax(-1))
    with pytest.raises(ValueError):
        ops.greedy_advance(logits, token.int())


def test_graph_replay_equals_eager_decode(tiny, cuda):
    g = torch.Generator().manual_seed(4)
    tokens = torch.randint(0, tiny.config.vocab_size, (3, 40), generator=g).to(cuda)
    eager = tiny.generate(tokens, 12, use_graph=False)
    tiny._graph = None
    graphed = tiny.generate(tokens, 12, use_graph=True)
    again = tiny.generate(tokens, 12, use_graph=True)           # replays of a graph captured earlier
    assert torch.equal(eager, graphed)
    assert torch.equal(eager, again)
    assert eager.shape == (3, 12) and int(eager.min()) >= 0 and int(eager.max()) < tiny.config.vocab_size
