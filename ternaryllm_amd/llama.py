"""A minimal Llama-shaped decoder whose linear layers are all ternary: RMSNorm, rotary embedding,
a preallocated KV cache, causal softmax attention, the SiLU-gated MLP, and a greedy generation loop.

It stands where the reference patches a Hugging Face Llama with its ternary modules
(ternaryLLM_GPU/TernaryLLM/TernaryLlama.py:69-75) and drives it with `generate`
(ternaryLLM_GPU/benchmark_ternary_llama.py:81-105); the CPU twin of the same structure is
ternaryLLM_CPU/src/LlamaModel.hpp:457-527.  Weights are random ternary matrices, drawn as the
reference draws them; every product runs in libternary_spmm.so.  A prefill pass uses torch operators
for normalisation, rotary embedding and attention; a single-token step uses the library's kernels
for them (rotary + cache update, attention over the cache, residual add + RMSNorm, SiLU gate).

The decode step has static shapes (the cache has its full length, a mask hides what is not
written yet, position and token live in device tensors), so it can be captured once in a HIP graph
and replayed for every generated token.
"""
import math
from concurrent.futures import ThreadPoolExecutor

import numpy as np
import torch
from torch import nn

from . import _lib, ops, packing
from .linear import TernaryLinear


def _draw_ternary(K, N, sparsity, generator, device):
    """The reference's i.i.d. rule (TernaryLinear.py:79-83) evaluated on `device`: r < s -> 0,
    s <= r < (s + 1) / 2 -> -1, else +1.  Returns an int32 [K, N] tensor on the CPU."""
    r = torch.rand((K, N), generator=generator, device=device)
    w = (r >= (sparsity + 1) / 2).to(torch.int32) - ((r >= sparsity) & (r < (sparsity + 1) / 2)).to(torch.int32)
    return w.cpu()


class RMSNorm(nn.Module):
    def __init__(self, size, eps, dtype, device):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(size, dtype=dtype, device=device), requires_grad=False)
        self.eps = eps

    def forward(self, x):
        return torch.nn.functional.rms_norm(x, (x.shape[-1],), self.weight, self.eps)


class DecoderLayer(nn.Module):
    """One block.  q, k and v share their input, so their weights are packed side by side as one
    [hidden, 3 * hidden] matrix and run as one product; likewise gate and up as one
    [hidden, 2 * intermediate] matrix."""

    def __init__(self, config, linears, dtype, device):
        super().__init__()
        self.qkv_proj, self.o_proj, self.gate_up_proj, self.down_proj = linears
        self.input_layernorm = RMSNorm(config.hidden_size, config.rms_norm_eps, dtype, device)
        self.post_attention_layernorm = RMSNorm(config.hidden_size, config.rms_norm_eps, dtype, device)


class TernaryLlamaDecoder(nn.Module):
    """config: TernaryConfig (or any object with its attributes).  `sparsity` of the config applies to
    every linear layer, the output head included.  Each linear carries a per-output-channel scale
    1 / sqrt(non-zeros per column) so that activations keep their magnitude through the stack."""

    LINEARS = ("qkv", "o", "gate_up", "down")

    def __init__(self, config, *, seed=0, device="cuda", dtype=torch.float16, max_seq_len=None, pack_threads=8):
        super().__init__()
        if config.num_key_value_heads != config.num_attention_heads:
            raise ValueError("grouped-query attention is not supported by this decoder")
        self.config = config
        self.dtype = dtype
        self.max_seq_len = int(max_seq_len or config.max_position_embeddings)
        H, I, V = config.hidden_size, config.intermediate_size, config.vocab_size
        dev = torch.device(device)
        gen = torch.Generator(device=dev if dev.type == "cuda" else "cpu")
        gen.manual_seed(seed)
        draw_dev = dev if dev.type == "cuda" else "cpu"

        shapes = {"qkv": (H, 3 * H), "o": (H, H), "gate_up": (H, 2 * I), "down": (I, H)}

        def make(shape):
            K, N = shape
            w = _draw_ternary(K, N, config.sparsity, gen, draw_dev)
            return w.numpy()

        def pack(w):
            K, N = w.shape
            pw = packing.PackedWeight.from_dense(w)
            nnz_col = np.maximum(np.count_nonzero(w, axis=0), 1)
            return pw, torch.from_numpy((1.0 / np.sqrt(nnz_col)).astype(np.float16))

        # Draw in layer order (so the seed fixes the model) and pack on worker threads: the packers run
        # outside the interpreter lock.  Only a few dense matrices are alive at a time.
        todo = [(li, name) for li in range(config.num_hidden_layers) for name in self.LINEARS] + [(-1, "head")]
        shapes["head"] = (H, V)
        done = {}
        with ThreadPoolExecutor(max_workers=max(1, pack_threads)) as pool:
            pending = []
            for key in todo:
                pending.append((key, pool.submit(pack, make(shapes[key[1]]))))
                if len(pending) >= 2 * max(1, pack_threads):
                    k0, job = pending.pop(0)
                    done[k0] = TernaryLinear.from_packed(*job.result(), device=dev)
            for k0, job in pending:
                done[k0] = TernaryLinear.from_packed(*job.result(), device=dev)
        layers = [DecoderLayer(config, [done[(li, name)] for name in self.LINEARS], dtype, dev)
                  for li in range(config.num_hidden_layers)]
        self.lm_head = done[(-1, "head")]
        self.layers = nn.ModuleList(layers)
        cpu_gen = torch.Generator().manual_seed(seed + 1)
        self.embed_tokens = nn.Parameter((0.02 * torch.randn((V, H), generator=cpu_gen)).to(dev, dtype), requires_grad=False)
        for layer in self.layers:
            for norm in (layer.input_layernorm, layer.post_attention_layernorm):
                norm.weight.copy_((1.0 + 0.02 * torch.randn(H, generator=cpu_gen)).to(dev, dtype))
        self.norm = RMSNorm(H, config.rms_norm_eps, dtype, dev)
        hd = config.head_dim
        inv = 1.0 / (config.rope_theta ** (torch.arange(0, hd, 2, dtype=torch.float32) / hd))
        ang = torch.arange(self.max_seq_len, dtype=torch.float32)[:, None] * inv[None, :]
        ang = torch.cat([ang, ang], dim=-1)
        self.register_buffer("rope_cos", ang.cos().to(dev, dtype), False)
        self.register_buffer("rope_sin", ang.sin().to(dev, dtype), False)
        self._cache = None
        self._graph = None
        # single-token steps use the library's rotary / cache / attention kernels; False keeps them on torch operators
        self.native_decode = config.head_dim in (64, 128, 256) and self.max_seq_len * 4 <= 120 * 1024
        # single-row steps fold the norms and the SiLU gate into the products' kernels; that kernel wants rows and
        # tiles of whole 16-byte pieces
        self.fused_decode = all(m._header.tile_rows % 8 == 0 and m.in_features % 8 == 0
                                for layer in self.layers for m in (layer.qkv_proj, layer.o_proj, layer.gate_up_proj, layer.down_proj)) and \
            self.lm_head._header.tile_rows % 8 == 0 and H % 8 == 0
        # the attention kernel rotates q and k and writes the token's cache row itself; False runs the separate kernel first
        self.fused_rope = True
        # single-row steps: share the cache rows of a head out among several workgroups, the last of which to finish
        # folds their pieces.  That pays once a head's rows are many: up to about a thousand rows one workgroup per
        # head is as quick.
        self.split_attention = self.max_seq_len > 1024
        # steps of 9 to 16 fp16 rows: the products do the residual adds and the RMSNorms around them (tl_spmm_chain);
        # switched off by the first step whose shapes have no such kernel
        self.chain_decode = dtype == torch.float16
        # single-row steps: the o and down projections prepare the row for the norm behind them (spmv_add with
        # next_norm_weight); switched off by the first step whose shapes have no such kernel
        self.row_chain = True
        # single-row steps with row_chain: the attention leaves this many pieces per head (their workgroups fill more of
        # the chip than one per head does; four with a long cache, split_attention) and the o projection folds the
        # pieces of each wave's own tiles on the way in (spmv_attn_combine); 0: the attention writes the output row
        # (one workgroup per head, or the last of several to finish).  Switched off by the first step whose shapes
        # have no such kernel.
        self.piece_fold = 2
        self._layer_index = {id(layer): i for i, layer in enumerate(self.layers)}

    # -- pieces ------------------------------------------------------------------------------
    @staticmethod
    def _rope(x, cos, sin):
        half = x.shape[-1] // 2
        rot = torch.cat([-x[..., half:], x[..., :half]], dim=-1)
        return x * cos + rot * sin

    def _mlp(self, layer, x2):
        # columns 2j, 2j + 1 of the gate|up weight are gate and up of output j: the product's epilogue applies the gate
        gated = ops.spmm_gated(layer.gate_up_proj.device_weight(), x2, layer.gate_up_proj.w_scale)
        return layer.down_proj(gated)

    def allocate_cache(self, batch):
        c = self.config
        shape = (c.num_hidden_layers, 2, batch, c.num_attention_heads, self.max_seq_len, c.head_dim)
        self._cache = torch.zeros(shape, dtype=self.dtype, device=self.embed_tokens.device)
        self._graph = None
        return self._cache

    def _block(self, layer, li, x, cos, sin, write_pos, attend):
        """x: [B, S, H]; cos/sin: [S, head_dim]; write_pos: LongTensor [S] of cache slots;
        attend(q, k_cache, v_cache) -> [B, heads, S, head_dim]."""
        c = self.config
        B, S, H = x.shape
        nh, hd = c.num_attention_heads, c.head_dim
        h = layer.input_layernorm(x)
        qkv = layer.qkv_proj(h.reshape(B * S, H)).view(B, S, 3, nh, hd)
        q = self._rope(qkv[:, :, 0].transpose(1, 2), cos, sin)
        k = self._rope(qkv[:, :, 1].transpose(1, 2), cos, sin)
        v = qkv[:, :, 2].transpose(1, 2)
        kc, vc = self._cache[li, 0], self._cache[li, 1]
        kc.index_copy_(2, write_pos, k)
        vc.index_copy_(2, write_pos, v)
        a = attend(q, kc, vc).transpose(1, 2).reshape(B * S, H)
        x = x + layer.o_proj(a).view(B, S, H)
        h = layer.post_attention_layernorm(x)
        return x + self._mlp(layer, h.reshape(B * S, H)).view(B, S, H)

    # -- prefill -----------------------------------------------------------------------------
    @torch.no_grad()
    def prefill(self, tokens):
        """tokens: LongTensor [B, S].  Fills the cache slots [0, S) and returns the logits of the last
        position, [B, vocab]."""
        B, S = tokens.shape
        if S > self.max_seq_len:
            raise ValueError("prompt longer than the cache")
        if self._cache is None or self._cache.shape[2] != B:
            self.allocate_cache(B)
        x = self.embed_tokens[tokens]
        pos = torch.arange(S, device=x.device)
        cos, sin = self.rope_cos[:S], self.rope_sin[:S]

        def attend(q, kc, vc):
            return torch.nn.functional.scaled_dot_product_attention(q, kc[:, :, :S], vc[:, :, :S], is_causal=True)

        for li, layer in enumerate(self.layers):
            x = self._block(layer, li, x, cos, sin, pos, attend)
        last = self.norm(x[:, -1])
        return self.lm_head(last)

    # -- decode ------------------------------------------------------------------------------
    def _decode_step(self, token, pos, mask):
        """token: LongTensor [B]; pos: LongTensor [1] (cache slot to write); mask: bool [1, 1, 1, max_seq]
        true on slots <= pos.  Static shapes throughout.  Returns logits [B, vocab]."""
        if self.native_decode:
            return self._decode_step_native(token, pos)
        x = self.embed_tokens[token][:, None]
        cos, sin = self.rope_cos.index_select(0, pos), self.rope_sin.index_select(0, pos)

        def attend(q, kc, vc):
            return torch.nn.functional.scaled_dot_product_attention(q, kc, vc, attn_mask=mask)

        for li, layer in enumerate(self.layers):
            x = self._block(layer, li, x, cos, sin, pos, attend)
        return self.lm_head(self.norm(x[:, 0]))

    def _decode_step_native(self, token, pos):
        """The decode step with rotary embedding, cache update and the attention over the cache as one
        library kernel (activations stay [B, hidden] throughout)."""
        c = self.config
        x = self.embed_tokens[token]
        B = x.shape[0]
        eps = c.rms_norm_eps
        # 5 to 48 rows: the products read a K-major image, so whatever feeds one writes it in that layout
        # (its transpose as a view) and no re-layout pass runs in front of the products
        if B == 1 and self.fused_decode:
            while self.row_chain:
                try:
                    return self._decode_step_fused(x, pos)
                except RuntimeError as e:
                    if "TL_ERR_UNSUPPORTED" not in str(e) or torch.cuda.is_current_stream_capturing():
                        raise
                    if self.piece_fold:
                        self.piece_fold = 0     # first without the fold in the o projection,
                    else:
                        self.row_chain = False  # then without the chain
            return self._decode_step_fused(x, pos)
        km = 5 <= B <= 48 and c.hidden_size != B and c.intermediate_size != B
        if km and 9 <= B <= 16 and self.chain_decode:
            try:
                return self._decode_step_chain(x, pos)
            except RuntimeError as e:
                if "TL_ERR_UNSUPPORTED" not in str(e) or torch.cuda.is_current_stream_capturing():
                    raise
                self.chain_decode = False
        _, h = ops.add_rmsnorm(x, None, self.layers[0].input_layernorm.weight, eps, kmajor=km)
        for li, layer in enumerate(self.layers):
            qkv = layer.qkv_proj(h)
            a = self._attend(qkv, self._cache[li, 0], self._cache[li, 1], pos, km)
            x, h = ops.add_rmsnorm(x, layer.o_proj(a), layer.post_attention_layernorm.weight, eps, kmajor=km)
            # the SiLU gate in the epilogue of the gate | up product where its kernel has one (else a launch of its own)
            gated = ops.spmm_gated(layer.gate_up_proj.device_weight(), h, layer.gate_up_proj.w_scale,
                                   x_layout=_lib.TL_X_K_MAJOR if km else _lib.TL_X_ROW_MAJOR, kmajor=km)
            y = layer.down_proj(gated)
            nxt = self.layers[li + 1].input_layernorm.weight if li + 1 < len(self.layers) else self.norm.weight
            x, h = ops.add_rmsnorm(x, y, nxt, eps, kmajor=km)  # the residual add, and the norm the next layer (or the head) starts with
        return self.lm_head(h)

    def _decode_step_chain(self, x, pos):
        """9 to 16 rows, five launches per layer, none of them elementwise: the o and down projections add the residual
        rows and leave the next norm's image (rows * norm weight) and sums of squares; q|k|v, gate|up (SiLU gate in
        its epilogue) and the head apply the normalisation factor to their sums.  Only the very first norm has a
        kernel of its own."""
        eps = self.config.rms_norm_eps
        K_MAJOR = _lib.TL_X_K_MAJOR
        _, h = ops.add_rmsnorm(x, None, self.layers[0].input_layernorm.weight, eps, kmajor=True)
        squares = None
        for li, layer in enumerate(self.layers):
            if squares is None:
                qkv = layer.qkv_proj(h)
            else:
                qkv = ops.spmm_chain(layer.qkv_proj.device_weight(), h, layer.qkv_proj.w_scale, K_MAJOR, squares_in=squares, eps=eps)
            a = self._attend(qkv, self._cache[li, 0], self._cache[li, 1], pos, True)
            x, h, squares = ops.spmm_chain(layer.o_proj.device_weight(), a, layer.o_proj.w_scale, K_MAJOR, residual=x,
                                           next_norm_weight=layer.post_attention_layernorm.weight)
            gated = ops.spmm_chain(layer.gate_up_proj.device_weight(), h, layer.gate_up_proj.w_scale, K_MAJOR, squares_in=squares, eps=eps,
                                   gated=True, kmajor=True)
            nxt = self.layers[li + 1].input_layernorm.weight if li + 1 < len(self.layers) else self.norm.weight
            x, h, squares = ops.spmm_chain(layer.down_proj.device_weight(), gated, layer.down_proj.w_scale, K_MAJOR, residual=x,
                                           next_norm_weight=nxt)
        return ops.spmm_chain(self.lm_head.device_weight(), h, self.lm_head.w_scale, K_MAJOR, squares_in=squares, eps=eps)

    def _decode_step_fused(self, x, pos):
        """One row, five launches per layer instead of nine, none of them an elementwise kernel: q|k|v and gate|up
        normalise their input themselves (RMSNorm with the factor applied to the sums, tl_spmv_fused "rmsnorm"); the
        gate|up product applies the SiLU gate in its epilogue (columns packed as gate/up pairs); the attention rotates
        q and k and writes the cache row; with a long cache (split_attention) it shares the cache rows of a head out
        among several workgroups (32 heads alone leave seven compute units in eight idle); it leaves two pieces per head
        (four with a long cache) that the o projection folds on its way in (piece_fold), or, without that, the last
        of its workgroups to finish folds them (tl_decode_attention_fold); the o and down projections add their
        result to the residual stream in their epilogue."""
        eps = self.config.rms_norm_eps
        # x is the residual stream: every product that ends a block adds its result to it in the epilogue, and the
        # products that start one normalise it on the way in (the factor applied to their sums).  With row_chain the
        # product that ends a block also leaves the row multiplied by the next norm's weight and the sums of its
        # squares (spmv_add(..., next_norm_weight=)), and the product after the norm is the plain kernel with one
        # factor at the end ("rmsnorm_sums"): it keeps one image of the row in LDS, not two.
        chain = self.row_chain
        image = squares = None
        for li, layer in enumerate(self.layers):
            if squares is None:
                qkv = ops.spmv_fused(layer.qkv_proj.device_weight(), "rmsnorm", x, None, layer.input_layernorm.weight, eps, layer.qkv_proj.w_scale)
            else:
                qkv = ops.spmv_fused(layer.qkv_proj.device_weight(), "rmsnorm_sums", image, squares, None, eps, layer.qkv_proj.w_scale)
            squares = None
            caches = self._cache_of(layer, 0), self._cache_of(layer, 1)
            if self.pieces_per_head():
                # two pieces per head (four with a long cache), folded by the o projection as it reads them
                pieces = self._attend(qkv, *caches, pos, False, pieces=True, splits=self.pieces_per_head())
                x, image, squares = ops.spmv_attn_combine(layer.o_proj.device_weight(), pieces, self.config.head_dim, qkv.dtype, layer.o_proj.w_scale,
                                                          residual=x, next_norm_weight=layer.post_attention_layernorm.weight)
            else:
                # a long cache: the rows of a head shared out among several workgroups, the last of which folds their pieces
                att = self._attend(qkv, *caches, pos, False, splits=None if self.split_attention else 1)
                if chain:
                    x, image, squares = ops.spmv_add(layer.o_proj.device_weight(), att, x, layer.o_proj.w_scale,
                                                     next_norm_weight=layer.post_attention_layernorm.weight)
                else:
                    x = ops.spmv_add(layer.o_proj.device_weight(), att, x, layer.o_proj.w_scale)
            if squares is None:
                gated = ops.spmv_fused(layer.gate_up_proj.device_weight(), "rmsnorm", x, None, layer.post_attention_layernorm.weight, eps,
                                       layer.gate_up_proj.w_scale, gated=True)
            else:
                gated = ops.spmv_fused(layer.gate_up_proj.device_weight(), "rmsnorm_sums", image, squares, None, eps,
                                       layer.gate_up_proj.w_scale, gated=True)
            squares = None
            if chain:
                nxt = self.layers[li + 1].input_layernorm.weight if li + 1 < len(self.layers) else self.norm.weight
                x, image, squares = ops.spmv_add(layer.down_proj.device_weight(), gated, x, layer.down_proj.w_scale, next_norm_weight=nxt)
            else:
                x = ops.spmv_add(layer.down_proj.device_weight(), gated, x, layer.down_proj.w_scale)
        if squares is None:
            return ops.spmv_fused(self.lm_head.device_weight(), "rmsnorm", x, None, self.norm.weight, eps, self.lm_head.w_scale)
        return ops.spmv_fused(self.lm_head.device_weight(), "rmsnorm_sums", image, squares, None, eps, self.lm_head.w_scale)

    def pieces_per_head(self):
        """Pieces the attention of a single-row step leaves per head for the o projection to fold; 0: it folds them itself."""
        if not (self.row_chain and self.piece_fold):
            return 0
        return max(self.piece_fold, 4) if self.split_attention else self.piece_fold

    def _attend(self, qkv, k_cache, v_cache, pos, kmajor, pieces=False, splits=None):
        """Rotary embedding, cache update and attention for the token whose q | k | v the projection just wrote: one
        launch, or (fused_rope False) the rotary + cache kernel followed by the attention."""
        q, fresh = None, (qkv, self.rope_cos, self.rope_sin)
        if not self.fused_rope:
            c = self.config
            q = torch.empty((qkv.shape[0], c.num_attention_heads, c.head_dim), dtype=qkv.dtype, device=qkv.device)
            ops.rope_cache_update(qkv, self.rope_cos, self.rope_sin, pos, q, k_cache, v_cache)
            fresh = None
        if pieces:
            return ops.decode_attention_pieces(q, k_cache, v_cache, pos, splits=splits, fresh=fresh)
        return ops.decode_attention(q, k_cache, v_cache, pos, kmajor=kmajor, splits=splits, fresh=fresh)

    def _cache_of(self, layer, which):
        return self._cache[self._layer_index[id(layer)], which]

    @torch.no_grad()
    def generate(self, tokens, new_tokens, use_graph=True):
        """Greedy decoding: prefill `tokens` [B, S], then `new_tokens` steps.  Returns LongTensor
        [B, new_tokens].  With use_graph the decode step is captured once and replayed."""
        B, S = tokens.shape
        if S + new_tokens > self.max_seq_len:
            raise ValueError("prompt plus new tokens exceed the cache")
        dev = self.embed_tokens.device
        logits = self.prefill(tokens)
        out = torch.empty((B, new_tokens), dtype=torch.long, device=dev)
        st = self._decode_state(B)
        st["token"].copy_(logits.argmax(-1))
        st["pos"].fill_(S)
        st["mask"].copy_((torch.arange(self.max_seq_len, device=dev) <= S)[None, None, None])
        for i in range(new_tokens):
            out[:, i] = st["token"]
            if i + 1 == new_tokens:
                break
            self.decode_once(st, use_graph)
        return out

    def _decode_state(self, B):
        dev = self.embed_tokens.device
        st = getattr(self, "_state", None)
        if st is None or st["token"].shape[0] != B:
            st = {"token": torch.zeros(B, dtype=torch.long, device=dev), "pos": torch.zeros(1, dtype=torch.long, device=dev),
                  "mask": torch.zeros((1, 1, 1, self.max_seq_len), dtype=torch.bool, device=dev)}
            self._state = st
            self._graph = None
        return st

    def _advance(self, st):
        logits = self._decode_step(st["token"], st["pos"], st["mask"])
        self.last_logits = logits  # (under a captured graph: the tensor every replay writes)
        # positions stay inside the cache even if a caller steps past its end (the results are then
        # meaningless, but nothing is written out of bounds; generate() checks the length up front)
        if logits.is_cuda and logits.dtype in (torch.float16, torch.float32) and logits.is_contiguous():
            # argmax, the new position and its mask bit in one launch
            ops.greedy_advance(logits, st["token"], st["pos"], self.max_seq_len - 1, st["mask"])
            return
        st["token"].copy_(logits.argmax(-1))
        st["pos"].add_(1).clamp_(max=self.max_seq_len - 1)
        st["mask"].index_fill_(3, st["pos"], True)

    @torch.no_grad()
    def decode_once(self, st, use_graph=True):
        """One greedy step on the state tensors (token, pos, mask), in place."""
        if not use_graph:
            self._advance(st)
            return
        if self._graph is None:
            # warm-up on a side stream (first calls set kernel attributes and grow workspaces), with the
            # state restored afterwards; then capture
            keep = {k: v.clone() for k, v in st.items()}
            cache_keep = None
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _ in range(2):
                    for k, v in keep.items():
                        st[k].copy_(v)
                    self._advance(st)
            torch.cuda.current_stream().wait_stream(side)
            for k, v in keep.items():
                st[k].copy_(v)
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                self._advance(st)
            for k, v in keep.items():
                st[k].copy_(v)
            self._graph = g
            del cache_keep
        self._graph.replay()


__all__ = ["TernaryLlamaDecoder", "RMSNorm", "DecoderLayer"]
