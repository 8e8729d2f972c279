#!/usr/bin/env python3
"""Benchmark of the ternary SpMM hot path on one MI355X.

Workload (the Llama-2-7B ternary MLP block, the shape the headline metric is quoted on):
one step = one ternary SpMM of the gate projection: 8 x 128 = 1024 token rows, fp16 activations
~N(0,1), W ternary [4096 -> 11008] at 80 % sparsity (10 % +1, 10 % -1, i.i.d., seeded), per-output
fp16 scale ~U(0.5, 1.5), fp32 accumulation, fp16 output.  Inputs are resident in HBM before the
timed region.  The value is algorithmic GB/s: bytes every operand must move at least once
(index stream as stored, chunk table, X, Y, scale) divided by the step time.

Prints ONE JSON line.  Besides the contract fields it carries
  roofline      HBM roofline of the dominant kernel, timed with HIP events on the kernel's stream
  cpu_baseline  the reference's CPU SIMD kernel on the same W and X, on this host's cores
  extra         the other regimes of the path (decode SpMV, small batch, fused MLP block), add-rate
                figures, and tokens/s
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
VALU_PEAK_GADDS = 39321.6      # 256 CU x 64 lanes x 2.4 GHz fp32 adds/s without packed-fp32 forms


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary workloads")
    ap.add_argument("--no-decoder", action="store_true", help="skip the 32-layer decoder (prefill 512 + 128 greedy steps)")
    ap.add_argument("--only-decoder", action="store_true", help="of the secondary workloads run the 32-layer decoder alone (for profiling it)")
    ap.add_argument("--only-decode-shapes", action="store_true", help="of the secondary workloads run the cold decode shapes alone (for profiling them)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run one plain 256 MiB device copy (reference for scaling rocprof's FETCH_SIZE / WRITE_SIZE)")
    return ap.parse_args()


_packed = {}


def weight_and_packed(K, N, sparsity, seed, device):
    """(dense int32 weight, PackedWeight, DeviceWeight) of a seeded random weight; legs that name the same shape,
    sparsity and seed share one (packing is host work of seconds, not part of anything timed)."""
    import torch
    from ternaryllm_amd import ops
    from ternaryllm_amd.linear import random_ternary_weights
    from ternaryllm_amd.packing import PackedWeight
    key = (K, N, sparsity, seed, str(device))
    if key not in _packed:
        g = torch.Generator().manual_seed(seed)
        w = random_ternary_weights((K, N), sparsity, generator=g)
        pw = PackedWeight.from_dense(w)
        _packed[key] = (w, pw, ops.DeviceWeight(pw, device))
    return _packed[key]


def kernel_source_hash():
    """sha256 over the sources the headline's three kernels and their launcher are built from (the row-parallel
    kernels' translation unit, what it shares with the others, the blob builder, the shared constants): a traffic
    figure recorded for other sources is not reported."""
    import hashlib
    h = hashlib.sha256()
    csrc = os.path.join(ROOT, "ternaryllm_amd", "csrc")
    for name in ("tl_rows.hip", "tl_device.h", "tl_layout.cpp", "tl_common.h"):
        with open(os.path.join(csrc, name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def best_k_mean(samples, k):
    s = sorted(samples)[:k]
    return sum(s) / len(s)


def time_spmm(dw, x, scale, steps, warmup, x_layout=0):
    """Wall-clock ms per step (synchronise, K steps, synchronise) and event-timed ms per launch."""
    import torch
    from ternaryllm_amd import ops
    for _ in range(warmup):
        ops.spmm(dw, x, scale, x_layout=x_layout)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        ops.spmm(dw, x, scale, x_layout=x_layout)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    ev_ms, _ = ops.spmm_time(dw, x, steps, scale, x_layout=x_layout)
    return wall_ms, ev_ms


def graph_us_per_node(fn, nodes, replays, full=False):
    """Median, 10th percentile and best-10 mean of the time per node of a HIP graph of fn(0) ... fn(nodes - 1),
    replayed `replays` times (launch gaps are then the hardware's, not the interpreter's).  With `full`: a dict
    that also holds the fastest and the slowest replay."""
    import torch
    for i in range(2):
        fn(i)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for i in range(nodes):
                fn(i)
    torch.cuda.synchronize()
    for _ in range(2):
        graph.replay()
    torch.cuda.synchronize()
    samples = []
    for _ in range(replays):
        t0 = time.perf_counter()
        graph.replay()
        torch.cuda.synchronize()
        samples.append((time.perf_counter() - t0) / nodes)
    samples.sort()
    if full:
        return {"median": samples[len(samples) // 2], "p10": samples[len(samples) // 10], "best10_mean": best_k_mean(samples, 10),
                "min": samples[0], "max": samples[-1], "replays": replays, "nodes": nodes}
    return samples[len(samples) // 2], samples[len(samples) // 10], best_k_mean(samples, 10)


def us_fields(t, prefix="us_per_call"):
    """The fields of a graph-replay timing, in microseconds."""
    return {prefix + "_median": round(t["median"] * 1e6, 3), prefix + "_min": round(t["min"] * 1e6, 3), prefix + "_max": round(t["max"] * 1e6, 3),
            prefix + "_p10": round(t["p10"] * 1e6, 3), "replays": t["replays"], "calls_per_replay": t["nodes"]}


def small_shape_leg(dev, M, K, N, sparsity, dtype, seed, calls=400, replays=15):
    """A product of few rows, timed as the median of `replays` replays of a HIP graph of `calls` calls on ONE weight
    (it stays in the last-level cache: the warm figure) with an x of its own for every call; the spread of the
    replays beside it.  Event-timed single launches of a few microseconds wobble by 20 %; a graph's replays do not."""
    import torch
    from ternaryllm_amd import ops
    w, pw, dw = weight_and_packed(K, N, sparsity, seed, dev)
    g = torch.Generator().manual_seed(seed + 1)
    xs = torch.randn((calls, M, K), generator=g).to(dtype).to(dev)
    ys = torch.empty((calls, M, N), dtype=dtype, device=dev)
    t = graph_us_per_node(lambda i: ops.spmm(dw, xs[i], out=ys[i]), calls, replays, full=True)
    ref = xs[calls - 1].double().cpu().numpy() @ w.double().numpy()
    err = float(abs(ys[calls - 1].double().cpu().numpy() - ref).max() / max(1e-9, abs(ref).max()))
    B = pw.algorithmic_bytes(M, xs.element_size(), xs.element_size())
    out = {"M": M, "K": K, "N": N, "sparsity": sparsity, "dtype": str(dtype).replace("torch.", ""), "weights": "one copy (warm)", "distinct_x": calls,
           "kernel_ms": round(t["median"] * 1e3, 5), "GB_per_s": round(B / t["median"] / 1e9, 1),
           "pct_hbm_peak": round(100 * B / t["median"] / 1e9 / HBM_PEAK_GBS, 2), "tokens_per_s": round(M / t["median"], 1),
           "max_err_over_max": err}
    out.update(us_fields(t))
    return out


def attention_block_leg(dev, tokens=(8, 128), runs=10):
    """The attention block of a Llama-2-7B-shaped layer with ternary q, k, v, o at 90 % sparsity: 8 x 128 tokens of
    fp16, 32 heads of 128, causal, dense softmax attention between the products.  Wall-clock per forward over
    `runs` calls; q | k | v as one packed weight (the module's default) and as three products beside it."""
    import torch
    from ternaryllm_amd import LlamaTernaryAttention, TernaryConfig
    cfg = TernaryConfig(sparsity=0.9)
    gen = torch.Generator().manual_seed(1245)
    attn = LlamaTernaryAttention(cfg, generator=gen, reference_buffers=False).to(dev)
    x = torch.randn((tokens[0], tokens[1], cfg.hidden_size), generator=gen).to(torch.float16).to(dev)
    n = tokens[0] * tokens[1]
    res = {"tokens": n, "batch": tokens[0], "seq": tokens[1], "heads": cfg.num_attention_heads, "head_dim": cfg.hidden_size // cfg.num_attention_heads,
           "sparsity": cfg.sparsity, "dtype": "float16"}
    for name, fused in (("qkv_one_weight", True), ("qkv_three_products", False)):
        attn.fused_qkv = fused
        for _ in range(3):
            attn(x)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(runs):
            attn(x)
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / runs
        res[name] = {"ms": round(ms, 4), "tokens_per_s": round(n / (ms * 1e-3), 1)}
    res["ms"], res["tokens_per_s"] = res["qkv_one_weight"]["ms"], res["qkv_one_weight"]["tokens_per_s"]
    return res


def sparsity_sweep_leg(dev, x, steps, sparsities=(0.70, 0.75, 0.80, 0.85, 0.90, 0.95, 0.99)):
    """The headline product (1024 x 4096 -> 11008, fp16, row-major activations) over the share of zeros, the sweep
    of the reference's benchmark (ternaryLLM_GPU/benchmark_ternary_mlp.py:59-101): event-timed ms per call, the
    adds per second that is, and that as a fraction of the vector units' add ceiling."""
    from ternaryllm_amd import ops
    rows = []
    M, K = x.shape
    for i, s in enumerate(sparsities):
        w, pw, dw = weight_and_packed(K, 11008, s, 1250 + i, dev)
        for _ in range(5):
            ops.spmm(dw, x)
        ms, _ = ops.spmm_time(dw, x, steps)
        B = pw.algorithmic_bytes(M, 2, 2)
        rows.append({"sparsity": s, "nnz": int(pw.nnz), "kernel_ms": round(ms, 5), "gadd_per_s": round(M * pw.nnz / (ms * 1e-3) / 1e9, 1),
                     "valu_add_roofline_frac": round(M * pw.nnz / (ms * 1e-3) / 1e9 / VALU_PEAK_GADDS, 4),
                     "GB_per_s": round(B / (ms * 1e-3) / 1e9, 1), "tokens_per_s": round(M / (ms * 1e-3), 1)})
        _packed.pop((K, 11008, s, 1250 + i, str(dev)), None)   # nothing else uses these
    return rows


def cold_decode_leg(dev, K=4096, N=4096, sparsity=0.66, copies=48, calls=1000, M=1, kmajor=False):
    """Config 2 as the decoder meets it: `calls` SpMV calls, each with an x of its own, over `copies` distinct
    copies of the weight (about 300 MB, more than the last-level cache holds), captured as one HIP graph
    and replayed.  With M > 1: the same for a batch of M rows (row-major).  Beside it, under the same replay, the
    box's own floors for a call that must stream that much memory: a launch that only READS one weight copy
    (tl_stream_read_probe: 16 bytes per lane, one store per workgroup) and a plain device copy of it (which reads
    and writes)."""
    import torch
    from ternaryllm_amd import ops
    w, pw, dw = weight_and_packed(K, N, sparsity, 1244, dev)
    ws = [dw]
    for _ in range(copies - 1):
        c = ops.DeviceWeight.__new__(ops.DeviceWeight)
        c.header, c.blob = dw.header, dw.blob.clone()
        ws.append(c)
    g = torch.Generator().manual_seed(1245)
    xs = torch.randn((calls, M, K), generator=g).to(torch.float16).to(dev)  # a fresh x for every call of the graph
    ys = torch.empty((calls, M, N), dtype=torch.float16, device=dev)
    if kmajor:  # the activations as the decoder's kernels hand them from one product to the next: [K][M], M contiguous
        xk = xs.transpose(1, 2).contiguous()
        t = graph_us_per_node(lambda i: ops.spmm(ws[i % copies], xk[i], x_layout=ops._lib.TL_X_K_MAJOR, out=ys[i]), calls, 12, full=True)
    else:
        t = graph_us_per_node(lambda i: ops.spmm(ws[i % copies], xs[i], out=ys[i]), calls, 12, full=True)
    med = t["median"]
    # parity of the last replay: first and last call
    err = 0.0
    for i in (0, calls - 1):
        ref = xs[i].double().cpu().numpy() @ w.double().numpy()
        err = max(err, float(abs(ys[i].double().cpu().numpy() - ref).max() / max(1e-9, abs(ref).max())))
    dst = torch.empty_like(dw.blob)
    nodes = min(calls, 4 * copies)
    copy_t = graph_us_per_node(lambda i: dst.copy_(ws[i % copies].blob), nodes, 12, full=True)
    folds = torch.empty(ops._lib.lib().tl_read_probe_workgroups(), dtype=torch.int32, device=dev)
    whole = (dw.blob.numel() // 16) * 16
    read_t = graph_us_per_node(lambda i: ops.stream_read_probe(ws[i % copies].blob[:whole], folds), nodes, 12, full=True)
    B = pw.algorithmic_bytes(M, 2, 2)
    out = {"M": M, "K": K, "N": N, "sparsity": sparsity, "x_layout": "K-major [K][M]" if kmajor else "row-major [M][K]", "weight_copies": copies,
           "distinct_x": calls, "us_per_call_best10_mean": round(t["best10_mean"] * 1e6, 3),
           "GB_per_s": round(B / med / 1e9, 1), "pct_hbm_peak": round(100 * B / med / 1e9 / HBM_PEAK_GBS, 2),
           "tokens_per_s": round(M / med, 1), "max_err_over_max": err, "weight_bytes": int(dw.blob.numel()),
           "read_only_stream_of_one_weight_us": round(read_t["median"] * 1e6, 3),
           "read_only_stream_GB_per_s": round(dw.blob.numel() / read_t["median"] / 1e9, 1),
           "time_over_read_floor": round(med / read_t["median"], 2),
           "plain_copy_of_one_weight_us": round(copy_t["median"] * 1e6, 3), "time_over_plain_copy": round(med / copy_t["median"], 2)}
    out.update(us_fields(t))
    return out


def same_weight_decode_leg(dev, K=4096, N=4096, sparsity=0.66, calls=1000):
    """Config 2 as BASELINE.json words it: ONE weight, 1000 calls, a fresh x for every call, replayed from a HIP
    graph (the weight then stays in the last-level cache between calls)."""
    return small_shape_leg(dev, 1, K, N, sparsity, __import__("torch").float16, 1244, calls=calls, replays=12)


def balanced_leg(dev, steps, warmup):
    """Block-balanced weights (the reference's `uniform=True` generator, TernaryLinear.py:39-77: every block of a
    column holds the same number of +1 and of -1) against i.i.d. weights with the same number of non-zeros, on
    config 2's and config 3's shapes: the reference's kernels have a path of their own for balanced weights
    (no same-sign remainder, ter_spmm_kernel.cuh:59,249); here both run through the same kernels.  The single-row
    shape is timed as graph replays (median of 15, 400 calls with an x each, one warm weight): its launches are
    too short for event timing to hold still."""
    import torch
    from ternaryllm_amd import ops
    from ternaryllm_amd.linear import random_ternary_weights
    from ternaryllm_amd.packing import PackedWeight
    out = []
    for name, M, K, N, s in (("config 2 (M=1)", 1, 4096, 4096, 0.66), ("config 3 gate (M=1024)", 1024, 4096, 11008, 0.8)):
        g = torch.Generator().manual_seed(1250)
        calls = 400 if M == 1 else 1
        xs = torch.randn((calls, M, K), generator=g).to(torch.float16).to(dev)
        row = {"shape": name}
        for kind, uniform in (("iid", False), ("balanced_blocks_of_256", True)):
            w = random_ternary_weights((K, N), s, uniform, 256, generator=g)
            pw = PackedWeight.from_dense(w)
            dw = ops.DeviceWeight(pw, dev)
            row[kind] = {"nnz": int(pw.nnz), "stream_bytes": int(pw.header.stream_bytes)}
            if M == 1:
                ys = torch.empty((calls, M, N), dtype=torch.float16, device=dev)
                t = graph_us_per_node(lambda i: ops.spmm(dw, xs[i], out=ys[i]), calls, 15, full=True)
                row[kind].update({"kernel_ms": round(t["median"] * 1e3, 5)})
                row[kind].update(us_fields(t))
            else:
                _, ev_ms = time_spmm(dw, xs[0], None, max(steps, 50), warmup)
                row[kind]["kernel_ms"] = round(ev_ms, 5)
        row["balanced_over_iid"] = round(row["balanced_blocks_of_256"]["kernel_ms"] / row["iid"]["kernel_ms"], 4)
        out.append(row)
    return out


def decode_nodes_leg(model, dev, pos_value):
    """What bounds the single-row decode step, node by node: every kind of node of the captured step is replayed from a
    graph of its 32 instances (one per layer, each with its own weights and cache: cold, as in the step), beside a
    graph of read-only launches that stream the same bytes (the floor of a launch on this box).  The sum of the floors
    is the step's bound here; the step's time over the sum of its nodes' is what the gaps between 162 nodes cost."""
    import torch
    from ternaryllm_amd import ops
    c = model.config
    eps, H, L = c.rms_norm_eps, c.hidden_size, model.layers
    n_layers = len(L)
    g = torch.Generator().manual_seed(1246)
    x = (0.05 * torch.randn((1, H), generator=g)).to(model.dtype).to(dev)
    pos = torch.full((1,), pos_value, dtype=torch.long, device=dev)
    folds = torch.empty(ops._lib.lib().tl_read_probe_workgroups(), dtype=torch.int32, device=dev)
    qkv_row = ops.spmv_fused(L[0].qkv_proj.device_weight(), "rmsnorm", x, None, L[0].input_layernorm.weight, eps, L[0].qkv_proj.w_scale)
    att_row = model._attend(qkv_row, model._cache_of(L[0], 0), model._cache_of(L[0], 1), pos, False, splits=None if model.split_attention else 1)
    gated_row = ops.spmv_fused(L[0].gate_up_proj.device_weight(), "rmsnorm", x, None, L[0].post_attention_layernorm.weight, eps,
                               L[0].gate_up_proj.w_scale, gated=True)
    # the step's own launches: with row_chain the o and down products leave the next norm's image and sums of squares,
    # and the products behind a norm start from those
    chain = model.row_chain
    fold = model.pieces_per_head()   # the attention leaves pieces, the o product folds them
    if fold:
        pieces_row = model._attend(qkv_row, model._cache_of(L[0], 0), model._cache_of(L[0], 1), pos, False, pieces=True, splits=fold)
    if chain:
        _, image, squares = ops.spmv_add(L[0].o_proj.device_weight(), att_row, x, L[0].o_proj.w_scale, next_norm_weight=L[0].post_attention_layernorm.weight)

    def behind_norm(m, norm, gated=False):
        if chain:
            return ops.spmv_fused(m.device_weight(), "rmsnorm_sums", image, squares, None, eps, m.w_scale, gated=gated)
        return ops.spmv_fused(m.device_weight(), "rmsnorm", x, None, norm.weight, eps, m.w_scale, gated=gated)

    def ends_block(m, row, next_norm):
        if chain:
            return ops.spmv_add(m.device_weight(), row, x, m.w_scale, next_norm_weight=next_norm.weight)
        return ops.spmv_add(m.device_weight(), row, x, m.w_scale)

    def attention(i):
        caches = model._cache_of(L[i], 0), model._cache_of(L[i], 1)
        if fold:
            return model._attend(qkv_row, *caches, pos, False, pieces=True, splits=fold)
        return model._attend(qkv_row, *caches, pos, False, splits=None if model.split_attention else 1)

    def o_product(i):
        if fold:
            return ops.spmv_attn_combine(L[i].o_proj.device_weight(), pieces_row, c.head_dim, model.dtype, L[i].o_proj.w_scale, residual=x,
                                         next_norm_weight=L[i].post_attention_layernorm.weight)
        return ends_block(L[i].o_proj, att_row, L[i].post_attention_layernorm)

    norm_note = "RMSNorm factor from the sums that came with its input" if chain else "RMSNorm on its input"
    add_note = " + residual + next norm's image and sums" if chain else " + residual"
    kv_bytes = 2 * c.num_attention_heads * (pos_value + 1) * c.head_dim * x.element_size()
    kv_bytes -= kv_bytes % 16

    def blob(m):
        b = m.device_weight().blob
        return b[:(b.numel() // 16) * 16]

    kinds = [
        ("q|k|v product, " + norm_note, lambda i: behind_norm(L[i].qkv_proj, L[i].input_layernorm),
         lambda i: ops.stream_read_probe(blob(L[i].qkv_proj), folds), blob(L[0].qkv_proj).numel()),
        ("rotary + cache row + attention over %d rows" % (pos_value + 1) + (", left as %d pieces per head" % fold if fold else ""), attention,
         lambda i: ops.stream_read_probe(model._cache[i].reshape(-1).view(torch.uint8)[:kv_bytes], folds), kv_bytes),
        ("o product" + (" on the fold of the attention's pieces" if fold else "") + add_note, o_product,
         lambda i: ops.stream_read_probe(blob(L[i].o_proj), folds), blob(L[0].o_proj).numel()),
        ("gate|up product, " + norm_note + ", SiLU gate in its epilogue", lambda i: behind_norm(L[i].gate_up_proj, L[i].post_attention_layernorm, gated=True),
         lambda i: ops.stream_read_probe(blob(L[i].gate_up_proj), folds), blob(L[0].gate_up_proj).numel()),
        ("down product" + add_note, lambda i: ends_block(L[i].down_proj, gated_row, L[i].input_layernorm),
         lambda i: ops.stream_read_probe(blob(L[i].down_proj), folds), blob(L[0].down_proj).numel()),
    ]
    rows, sum_nodes, sum_floor = [], 0.0, 0.0
    for name, node, probe, nbytes in kinds:
        t = graph_us_per_node(node, n_layers, 12, full=True)
        f = graph_us_per_node(probe, n_layers, 12, full=True)
        rows.append({"node": name, "per_step": n_layers, "bytes": int(nbytes), "us": round(t["median"] * 1e6, 3), "us_min": round(t["min"] * 1e6, 3),
                     "us_max": round(t["max"] * 1e6, 3), "read_floor_us": round(f["median"] * 1e6, 3),
                     "time_over_read_floor": round(t["median"] / f["median"], 2)})
        sum_nodes += n_layers * t["median"]
        sum_floor += n_layers * f["median"]
    # the head: once per step; timed behind the 32 q|k|v products of a graph (which push it out of the caches) as the
    # difference to that graph without it
    def with_head(i):
        if i < n_layers:
            return kinds[0][1](i)
        return behind_norm(model.lm_head, model.norm)

    def with_head_probe(i):
        return kinds[0][2](i) if i < n_layers else ops.stream_read_probe(blob(model.lm_head), folds)

    t_head = graph_us_per_node(with_head, n_layers + 1, 12, full=True)["median"] * (n_layers + 1) - rows[0]["us"] * 1e-6 * n_layers
    f_head = graph_us_per_node(with_head_probe, n_layers + 1, 12, full=True)["median"] * (n_layers + 1) - rows[0]["read_floor_us"] * 1e-6 * n_layers
    rows.append({"node": "head product, " + norm_note, "per_step": 1, "bytes": int(blob(model.lm_head).numel()), "us": round(t_head * 1e6, 3),
                 "read_floor_us": round(f_head * 1e6, 3), "time_over_read_floor": round(t_head / f_head, 2)})
    sum_nodes += t_head
    sum_floor += f_head
    return {"nodes": rows, "sum_of_nodes_ms": round(sum_nodes * 1e3, 4), "sum_of_read_floors_ms": round(sum_floor * 1e3, 4),
            "note": "each node kind replayed alone from a graph of its 32 per-layer instances; floors: read-only launches over the same bytes"}


def decoder_leg(dev, prompt=512, new_tokens=128):
    """Llama-2-7B-shaped ternary decoder on random weights: prefill of `prompt` random ids, then
    `new_tokens` greedy steps (the step captured once in a HIP graph), at batch 1 and 16.  The timed run is
    checked: the logits of the first replayed step equal those of the same step run eagerly, bit for bit, and
    two further runs from the same prompt produce the same `new_tokens` tokens."""
    import torch
    from ternaryllm_amd import TernaryConfig, TernaryLlamaDecoder
    cfg = TernaryConfig(sparsity=0.66, max_position_embeddings=prompt + new_tokens)
    t0 = time.perf_counter()
    model = TernaryLlamaDecoder(cfg, seed=1242, device=dev, pack_threads=16)
    torch.cuda.synchronize()
    res = {"layers": cfg.num_hidden_layers, "hidden": cfg.hidden_size, "ffn": cfg.intermediate_size, "vocab": cfg.vocab_size,
           "sparsity": cfg.sparsity, "build_s": round(time.perf_counter() - t0, 1),
           "weights_GB": round(sum(b.numel() for n, b in model.named_buffers() if n.endswith("w_packed")) / 1e9, 3)}
    g = torch.Generator().manual_seed(1243)

    def start(tokens):
        logits = model.prefill(tokens)
        st = model._decode_state(tokens.shape[0])
        st["token"].copy_(logits.argmax(-1))
        st["pos"].fill_(prompt)
        st["mask"].copy_((torch.arange(model.max_seq_len, device=dev) <= prompt)[None, None, None])
        return st

    for B in (1, 16):
        tokens = torch.randint(0, cfg.vocab_size, (B, prompt), generator=g).to(dev)
        model.allocate_cache(B)
        model.prefill(tokens)  # warm-up: kernel attributes, workspaces
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        st = start(tokens)
        torch.cuda.synchronize()
        t_prefill = time.perf_counter() - t0
        eager = model._decode_step(st["token"], st["pos"], st["mask"]).clone()  # the first step, launched one by one
        model.decode_once(st, True)  # captures the graph; counts as the first of the new tokens' steps
        torch.cuda.synchronize()
        first_step_equal = bool(torch.equal(eager, model.last_logits))
        t0 = time.perf_counter()
        for _ in range(new_tokens - 1):
            model.decode_once(st, True)
        torch.cuda.synchronize()
        t_decode = (time.perf_counter() - t0) * new_tokens / (new_tokens - 1)
        runs = []
        for _ in range(2):  # untimed: the tokens of two more runs from the same prompt
            st = start(tokens)
            seq = []
            for _ in range(new_tokens):
                seq.append(st["token"].clone())
                model.decode_once(st, True)
            runs.append(torch.stack(seq, 1))
        tokens_repeat = bool(torch.equal(runs[0], runs[1]))
        if not (first_step_equal and tokens_repeat):
            print("bench.py: decoder check failed at batch %d (first replayed step equals eager: %s, tokens repeat: %s)"
                  % (B, first_step_equal, tokens_repeat), file=sys.stderr)
            sys.exit(1)
        nodes = None
        if B == 1 and model.fused_decode and model.native_decode:
            nodes = decode_nodes_leg(model, dev, prompt + new_tokens // 2)
        res["batch_%d" % B] = {"prefill_ms": round(t_prefill * 1e3, 2), "prefill_tokens_per_s": round(B * prompt / t_prefill, 1),
                               "decode_ms_per_step": round(t_decode * 1e3 / new_tokens, 4),
                               "decode_tokens_per_s": round(B * new_tokens / t_decode, 1),
                               "end_to_end_tokens_per_s": round(B * (prompt + new_tokens) / (t_prefill + t_decode), 1),
                               "checked": "first replayed step == eager step bit for bit; %d greedy tokens repeat over two runs" % new_tokens}
        if nodes is not None:
            step_ms = res["batch_1"]["decode_ms_per_step"]
            nodes["step_ms"] = step_ms
            nodes["step_over_sum_of_nodes"] = round(step_ms / nodes["sum_of_nodes_ms"], 3)
            nodes["step_over_sum_of_read_floors"] = round(step_ms / nodes["sum_of_read_floors_ms"], 3)
            res["batch_1"]["per_node"] = nodes
    del model
    torch.cuda.empty_cache()
    return res


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only; --gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)
    import numpy as np
    import torch
    from ternaryllm_amd import _lib, ops
    _lib.lib()  # no fallback: fail now if the HIP library is missing
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")

    if args.copy_probe:
        src = torch.ones(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---- headline workload -------------------------------------------------
    M, K, N, sparsity = 1024, 4096, 11008, 0.8
    w, pw, dw = weight_and_packed(K, N, sparsity, 1237, dev)
    g = torch.Generator().manual_seed(4242)
    x = torch.randn((M, K), generator=g).to(torch.float16)
    scale = (0.5 + torch.rand(N, generator=g)).to(torch.float16)
    xd, sd = x.to(dev), scale.to(dev)
    # row-major [M][K] activations, what TernaryLinear.forward passes: one call is the re-layout pre-pass, the row
    # kernel and its fix-up launch
    wall_ms, ev_ms = time_spmm(dw, xd, sd, args.steps, args.warmup)
    # beside it: activations already in the kernel's own layout ([K][M], M contiguous), no pre-pass
    xk = xd.t().contiguous()
    wall_km_ms, ev_km_ms = time_spmm(dw, xk, sd, args.steps, args.warmup, x_layout=_lib.TL_X_K_MAJOR)
    y = ops.spmm(dw, xd, sd)
    ref = (x.double().numpy() @ w.double().numpy()) * scale.double().numpy()[None, :]
    err = np.abs(y.float().cpu().numpy() - ref)
    floor = np.linalg.norm(x.double().numpy(), axis=1, keepdims=True) * np.sqrt(1 - sparsity)
    max_rel = float(np.max(err / np.maximum(np.abs(ref), floor)))
    if max_rel > 2e-3:
        print("bench.py: result differs from the exact product (max rel err %g)" % max_rel, file=sys.stderr)
        sys.exit(1)
    B = pw.algorithmic_bytes(M, 2, 2, 2)
    nnz = pw.nnz
    gbs = B / (wall_ms * 1e-3) / 1e9
    # HBM bytes per call from rocprofv3's FETCH_SIZE / WRITE_SIZE (profiles/): reported only while the kernels are
    # still the ones it was recorded for
    traffic, traffic_note = None, "no traffic record"
    tpath = os.path.join(ROOT, "profiles", "spmm_rows_c3_gate_traffic.json")
    if os.path.exists(tpath):
        with open(tpath) as f:
            rec = json.load(f)
        if rec.get("kernel_source_sha16") == kernel_source_hash():
            traffic, traffic_note = rec.get("hbm_bytes_per_launch"), "rocprofv3 FETCH_SIZE + WRITE_SIZE, profiles/spmm_rows_c3_gate_traffic.json"
        else:
            traffic_note = "profiles/spmm_rows_c3_gate_traffic.json was recorded for other kernel sources (%s)" % rec.get("kernel_source_sha16")
    out = {
        "metric": "ternary SpMM GB/s (% HBM peak) + tokens/s, Llama-2-7B ternary MLP shape",
        "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 in / f32 accumulate / f16 out", "data": "synthetic",
        "config": {"workload": "Llama-2-7B ternary MLP gate projection SpMM: M=1024 (8x128 tokens), K=4096, N=11008, "
                               "80% sparsity, fp16 activations, per-output fp16 scale, u8 tile-local indices",
                   "M": M, "K": K, "N": N, "sparsity": sparsity, "nnz": int(nnz), "algorithmic_bytes": int(B),
                   "x_layout": "row-major [M][K]", "max_rel_err": max_rel},
        "pct_hbm_peak": round(100 * gbs / HBM_PEAK_GBS, 3),
        "tokens_per_s": round(M / (wall_ms * 1e-3), 1),
        "roofline": {"bound": "hbm", "achieved": round(B / (ev_ms * 1e-3) / 1e9, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(B / (ev_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 5), "traffic": traffic, "traffic_note": traffic_note,
                     "kernel": "tl_relayout_rows_h + tl_spmm_rows<__half, 4, 8, 16, false, false> + tl_rows_fixup<__half, 4, 8, 16, false, false> "
                               "(the three launches of one tl_spmm call on row-major activations)",
                     "kernel_ms": round(ev_ms, 5)},
    }
    extra = {
        "gadd_per_s": round(M * nnz / (ev_ms * 1e-3) / 1e9, 1),
        "valu_add_roofline_frac": round(M * nnz / (ev_ms * 1e-3) / 1e9 / VALU_PEAK_GADDS, 4),
        "gop_equiv_per_s": round(2.0 * M * K * N / (ev_ms * 1e-3) / 1e9, 1),
        "k_major_input": {"ms_per_step": round(wall_km_ms, 5), "kernel_ms": round(ev_km_ms, 5),
                          "note": "activations handed over as [K][M]: no re-layout pre-pass"},
    }
    # the reference's own statistic (benchmark_ternary_mlp.py:51-53,98): 100 single calls timed one by one,
    # mean of the fastest 10; median and 10th percentile beside it
    singles = sorted(ops.spmm_time(dw, xd, 1, sd)[0] for _ in range(100))
    extra["headline_single_call_ms"] = {"best10_of_100_mean": round(best_k_mean(singles, 10), 5), "median": round(singles[50], 5),
                                        "p10": round(singles[10], 5)}

    # ---- CPU baseline on the same W and X ------------------------------------
    if not args.no_cpu:
        try:
            from oracle import cpu_baseline
            entries = []
            for r in cpu_baseline.time_gemm_all(w.numpy(), x.float().numpy(), runs=10):
                G = r["group"]
                idx_bytes = 2 * nnz + (N // G) * (2 + 2 * G) * 4  # int16 indices + the group table (2 + 2G ints per group of G columns)
                Bc = idx_bytes + M * K * 4 + M * N * 4
                entries.append({"value": round(Bc / r["seconds"] / 1e9, 3), "unit": "GB/s", "cores": r["threads"], "kind": r["kind"],
                                "sample": "the whole headline SpMM (same W, same X as fp32), mean of %d runs" % r["runs"],
                                "kernel": r["kernel"], "ms": round(r["seconds"] * 1e3, 3), "ms_min": round(r["seconds_min"] * 1e3, 3),
                                "ms_median": round(r["seconds_median"] * 1e3, 3), "ms_max": round(r["seconds_max"] * 1e3, 3),
                                "cpu": r["cpu"], "threads": r["binding"], "tokens_per_s": round(M / r["seconds"], 1), "max_rel_err": r["max_rel_err"]})
            # the reference's own headline choice first ("MergedMin_32G8_AVX2", ternaryLLM_CPU/src/main.cpp:1018,1088); its AVX-512 sibling beside it
            out["cpu_baseline"] = entries[0]
            out["cpu_baseline"]["note"] = "the reference's headline kernel; every other kernel the host runs is under `also`"
            out["cpu_baseline"]["also"] = entries[1:]
        except Exception as e:  # the baseline is reported, never required
            out["cpu_baseline"] = {"value": None, "unit": "GB/s", "cores": 0, "kind": "port", "sample": "failed: %s" % e}

    # ---- the other regimes of the path ---------------------------------------
    only = args.only_decoder or args.only_decode_shapes
    if not args.no_extra and not only:
        # what a plain device copy reaches on this box, beside the 8 TB/s the fractions are quoted against
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(10):
            dst.copy_(src)
        e1.record()
        torch.cuda.synchronize()
        extra["device_copy_1GiB"] = {"GB_per_s_read_plus_write": round(2 * src.numel() * 10 / (e0.elapsed_time(e1) * 1e-3) / 1e9, 1),
                                     "pct_hbm_peak": round(100 * 2 * src.numel() * 10 / (e0.elapsed_time(e1) * 1e-3) / 1e9 / HBM_PEAK_GBS, 1)}
        del src, dst
        def one(name, M2, K2, N2, s2, dt, seed):
            w2, pw2, dw2 = weight_and_packed(K2, N2, s2, seed, dev)
            x2 = torch.randn((M2, K2), generator=g).to(dt).to(dev)
            wms, ems = time_spmm(dw2, x2, None, max(args.steps, 50), args.warmup)
            B2 = pw2.algorithmic_bytes(M2, x2.element_size(), x2.element_size())
            extra[name] = {"M": M2, "K": K2, "N": N2, "sparsity": s2, "dtype": str(dt).replace("torch.", ""),
                           "kernel_ms": round(ems, 5), "GB_per_s": round(B2 / (ems * 1e-3) / 1e9, 1),
                           "pct_hbm_peak": round(100 * B2 / (ems * 1e-3) / 1e9 / HBM_PEAK_GBS, 2),
                           "tokens_per_s": round(M2 / (ems * 1e-3), 1)}
        extra["c1_spmm_m16_fp32"] = small_shape_leg(dev, 16, 4096, 4096, 0.5, torch.float32, 1235)
        extra["c2_decode_spmv_m1_fp16"] = small_shape_leg(dev, 1, 4096, 4096, 0.66, torch.float16, 1244)
        extra["decode_spmv_m1_fp16_n11008"] = small_shape_leg(dev, 1, 4096, 11008, 0.66, torch.float16, 1244)
        one("c3_down_m1024_fp16", 1024, 11008, 4096, 0.8, torch.float16, 1240)
        one("c4_proj_m1024_fp16", 1024, 4096, 4096, 0.9, torch.float16, 1238)
        # fused MLP block: gate+up+SiLU-gate in one kernel, then down
        from ternaryllm_amd import TernaryConfig, LlamaTernaryMLP
        cfg = TernaryConfig(sparsity=0.8)
        gen = torch.Generator().manual_seed(1241)
        sc = {k: (0.5 + torch.rand(n, generator=gen)).to(torch.float16) for k, n in (("gate", 11008), ("up", 11008), ("down", 4096))}
        mlp = LlamaTernaryMLP(cfg, generator=gen, scales=sc, reference_buffers=False).to(dev)
        xb = xd.reshape(8, 128, K)
        for _ in range(3):
            mlp(xb)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(10):
            mlp(xb)
        torch.cuda.synchronize()
        mlp_ms = (time.perf_counter() - t0) * 1e3 / 10
        extra["c3_mlp_block_fused"] = {"ms": round(mlp_ms, 4), "tokens_per_s": round(M / (mlp_ms * 1e-3), 1)}
        # the same block on one gate|up weight of (gate, up) column pairs, the gate in that product's epilogue
        mlp.paired = True
        for _ in range(3):
            mlp(xb)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(10):
            mlp(xb)
        torch.cuda.synchronize()
        pair_ms = (time.perf_counter() - t0) * 1e3 / 10
        extra["c3_mlp_block_pairs"] = {"ms": round(pair_ms, 4), "tokens_per_s": round(M / (pair_ms * 1e-3), 1)}
        del mlp
        extra["c4_attention_block"] = attention_block_leg(dev)
        extra["headline_sparsity_sweep"] = sparsity_sweep_leg(dev, xd, max(args.steps, 20))
    if not args.no_extra and not args.only_decoder:
        if not only:
            extra["balanced_vs_iid_weights"] = balanced_leg(dev, args.steps, args.warmup)
        extra["c2_decode_cold_weights_graph"] = cold_decode_leg(dev)
        if not only:
            extra["c2_decode_same_weight_graph"] = same_weight_decode_leg(dev)
        if not args.no_cpu and not only:
            try:  # the reference's decode kernels (ported) on the host's cores, same W, beside config 2
                from oracle import cpu_baseline
                w2, pw2, _ = weight_and_packed(4096, 4096, 0.66, 1244, dev)
                B2 = 4 * int(pw2.nnz) + 4096 * 4 + 4096 * 4  # int32 indices, as the reference's decode format holds them
                rows = [{"value": round(B2 / r2["seconds"] / 1e9, 3), "unit": "GB/s", "cores": r2["threads"], "kind": r2["kind"], "kernel": r2["kernel"],
                         "us": round(r2["seconds"] * 1e6, 1), "us_min": round(r2["seconds_min"] * 1e6, 1), "us_median": round(r2["seconds_median"] * 1e6, 1),
                         "tokens_per_s": round(1 / r2["seconds"], 1), "max_err_over_max": r2["max_err_over_max"]}
                        for r2 in cpu_baseline.time_gemv_all(w2.numpy(), torch.randn(4096, generator=g).numpy(), runs=50)]
                extra["c2_cpu_baseline"] = rows[0]
                extra["c2_cpu_baseline"]["also"] = rows[1:]
            except Exception as e:  # noqa: BLE001 - the baseline is optional, the GPU figures are not
                extra["c2_cpu_baseline"] = {"value": None, "sample": "failed: %s" % e}
        # the decoder's other products, one row and sixteen, over 24 cold copies each
        extra["decode_cold_shapes"] = [cold_decode_leg(dev, K, N, copies=24, calls=240, M=M, kmajor=km)
                                       for K, N in ((4096, 4096), (4096, 11008), (11008, 4096)) for M, km in ((1, False), (16, False), (16, True))]
    # ---- whole decoder: 32 layers, every linear ternary at 66 % sparsity -------
    if not args.no_extra and not args.no_decoder and not args.only_decode_shapes:
        extra["c5_decoder"] = decoder_leg(dev)
    out["extra"] = extra
    print(json.dumps(out))


if __name__ == "__main__":
    main()
