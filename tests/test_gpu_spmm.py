"""GPU parity of the ternary product against the CPU oracle, through the C ABI."""
import numpy as np
import pytest
import torch

from tests.util import FP16_TOL, FP32_TOL, activations, knobs, max_rel_err, ternary_weight

pytestmark = pytest.mark.gpu


def _run(cuda, oracle, M, K, N, s, dtype, seed, integer=False, scale=False, out_dtype=None, tile_rows=0):
    from ternaryllm_amd import ops
    from ternaryllm_amd.packing import PackedWeight
    w = ternary_weight(K, N, s, seed)
    x = activations(M, K, seed + 1, dtype, integer)
    pw = PackedWeight.from_dense(w, tile_rows)
    dw = ops.DeviceWeight(pw, cuda)
    sc = None
    ref = oracle.fast_product(x.double().numpy(), w)
    if scale:
        g = torch.Generator().manual_seed(seed + 2)
        sc = (0.5 + torch.rand(N, generator=g)).to(dtype)
        ref = ref * sc.double().numpy()[None, :]
    print(f"case M={M} K={K} N={N} s={s} dtype={dtype} int={integer} scale={scale}", flush=True)
    y = ops.spmm(dw, x.to(cuda), sc.to(cuda) if sc is not None else None, out_dtype)
    torch.cuda.synchronize()
    return y.float().cpu().numpy(), ref, x.float().numpy(), w


SHAPES = [
    (1, 512, 256, 0.66), (1, 4096, 4096, 0.66), (2, 1000, 130, 0.5), (3, 777, 65, 0.8), (5, 4096, 1024, 0.9),
    (8, 2048, 512, 0.8), (16, 4096, 4096, 0.5), (17, 1024, 320, 0.66), (33, 600, 200, 0.8), (48, 512, 512, 0.9),
    (49, 512, 192, 0.8), (64, 1024, 256, 0.66), (100, 777, 130, 0.5), (256, 2048, 512, 0.8), (300, 4096, 1000, 0.9),
    (1024, 4096, 1024, 0.8), (77, 520, 96, 0.7),
]


@pytest.mark.parametrize("M,K,N,s", SHAPES)
def test_fp32_exact_on_integer_activations(cuda, oracle, M, K, N, s):
    y, ref, x, w = _run(cuda, oracle, M, K, N, s, torch.float32, 11, integer=True)
    assert np.array_equal(y.astype(np.float64), ref)


@pytest.mark.parametrize("M,K,N,s", SHAPES)
def test_fp16_exact_on_integer_activations(cuda, oracle, M, K, N, s):
    y, ref, x, w = _run(cuda, oracle, M, K, N, s, torch.float16, 12, integer=True, out_dtype=torch.float32)
    assert np.array_equal(y.astype(np.float64), ref)


@pytest.mark.parametrize("M,K,N,s", SHAPES)
def test_fp32_within_tolerance(cuda, oracle, M, K, N, s):
    y, ref, x, w = _run(cuda, oracle, M, K, N, s, torch.float32, 21)
    assert max_rel_err(y, ref, x, w) <= FP32_TOL


@pytest.mark.parametrize("M,K,N,s", SHAPES)
def test_fp16_within_tolerance(cuda, oracle, M, K, N, s):
    y, ref, x, w = _run(cuda, oracle, M, K, N, s, torch.float16, 22, scale=True)
    assert max_rel_err(y, ref, x, w) <= FP16_TOL


@pytest.mark.parametrize("M", [1, 16, 128])
def test_small_oracle_triple_loop(cuda, oracle, M):
    """Same check against the oracle's own scalar triple loop (not BLAS) on a small case."""
    K, N = 300, 70
    w = ternary_weight(K, N, 0.6, 5)
    x = activations(M, K, 6, torch.float32)
    y, ref_fast, _, _ = _run(cuda, oracle, M, K, N, 0.6, torch.float32, 5)
    ref = oracle.dense_product(x.numpy(), w)
    assert np.allclose(ref, ref_fast, rtol=0, atol=1e-9)
    assert max_rel_err(y, ref, x.numpy(), w) <= FP32_TOL


@pytest.mark.parametrize("M", [1, 7, 200])
@pytest.mark.parametrize("kind", ["zero", "one_per_column", "all_plus", "dense_pm"])
def test_special_weights(cuda, oracle, M, kind):
    from ternaryllm_amd import ops
    from ternaryllm_amd.packing import PackedWeight
    K, N = 520, 96
    rng = np.random.default_rng(3)
    w = np.zeros((K, N), np.int32)
    if kind == "one_per_column":
        rows = rng.integers(0, K, N)
        signs = rng.choice([-1, 1], N)
        w[rows, np.arange(N)] = signs
    elif kind == "all_plus":
        w[:, :] = 1
    elif kind == "dense_pm":
        w[:, :] = rng.choice([-1, 1], (K, N))
    x = activations(M, K, 9, torch.float32, integer=True)
    dw = ops.DeviceWeight(PackedWeight.from_dense(w), cuda)
    y = ops.spmm(dw, x.to(cuda)).cpu().numpy()
    xn = x.numpy().astype(np.float64)
    if kind == "zero":
        assert not y.any()
    elif kind == "one_per_column":
        assert np.array_equal(y, (xn[:, rows] * signs[None, :]).astype(np.float32))
    elif kind == "all_plus":
        assert np.array_equal(y, np.repeat(xn.sum(1, keepdims=True), N, 1).astype(np.float32))
    else:
        assert np.array_equal(y.astype(np.float64), xn @ w)


def test_k_major_input_and_tile_heights(cuda, oracle):
    from ternaryllm_amd import ops
    from ternaryllm_amd.packing import PackedWeight
    K, N = 1024, 256
    w = ternary_weight(K, N, 0.7, 31)
    for M in (4, 160):
        x = activations(M, K, 32, torch.float32, integer=True)
        ref = oracle.fast_product(x.numpy(), w)
        for tile_rows in (0, 255, 128, 64, 100):
            dw = ops.DeviceWeight(PackedWeight.from_dense(w, tile_rows), cuda)
            y = ops.spmm(dw, x.to(cuda)).cpu().numpy()
            assert np.array_equal(y.astype(np.float64), ref), (M, tile_rows)
            yk = ops.spmm(dw, x.t().contiguous().to(cuda), x_layout=1).cpu().numpy()
            assert np.array_equal(yk.astype(np.float64), ref), (M, tile_rows, "k-major")


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("M", [49, 200, 257])
def test_row_kernel_activation_layouts(cuda, oracle, M, dtype):
    """Every way activations reach the row-parallel kernel: contiguous rows of whole 16-byte pieces (the 16-byte-per-lane
    re-layout for fp16), rows with an odd leading dimension or an odd K (the element-wise re-layout), a K-major image
    padded to the row tile (no pre-pass) and K-major with an odd leading dimension."""
    from ternaryllm_amd import ops
    from ternaryllm_amd.packing import PackedWeight
    for K, N in ((520, 96), (777, 50)):
        w = ternary_weight(K, N, 0.7, 43 + K)
        dw = ops.DeviceWeight(PackedWeight.from_dense(w), cuda)
        x = activations(M, K, 44 + M, dtype, integer=True)
        ref = oracle.fast_product(x.double().numpy(), w)
        xd = x.to(cuda)
        cases = {"row-major": (xd, 0)}
        wide = torch.zeros((M, K + 3), dtype=dtype, device=cuda)           # rows with an odd leading dimension
        wide[:, :K] = xd
        cases["row-major, strided"] = (wide[:, :K], 0)
        wide8 = torch.zeros((M, K + 8), dtype=dtype, device=cuda)          # aligned rows further apart than K
        wide8[:, :K] = xd
        cases["row-major, aligned stride"] = (wide8[:, :K], 0)
        padded = torch.zeros((K, -(-M // 256) * 256), dtype=dtype, device=cuda)  # the kernel's own layout
        padded[:, :M] = xd.t()
        cases["k-major, padded"] = (padded[:, :M], 1)
        widek = torch.zeros((K, M + 5), dtype=dtype, device=cuda)          # K-major with an odd leading dimension
        widek[:, :M] = xd.t()
        cases["k-major, strided"] = (widek[:, :M], 1)
        for name, (xin, layout) in cases.items():
            print(f"case M={M} K={K} dtype={dtype} {name}", flush=True)
            y = ops.spmm(dw, xin, x_layout=layout).float().cpu().numpy()
            assert np.array_equal(y.astype(np.float64), ref), (M, K, name)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("M", [1, 3, 4, 9, 16, 40])
def test_small_m_activation_layouts(cuda, oracle, M, dtype):
    """Every way the small-M kernel stages activations: whole row vectors, single elements (odd leading
    dimension, odd K), K-major vectors, and the K-major pre-pass for 8 rows and more."""
    from ternaryllm_amd import ops
    from ternaryllm_amd.packing import PackedWeight
    for K, N in ((1024, 96), (777, 50)):
        w = ternary_weight(K, N, 0.7, 41 + K)
        dw = ops.DeviceWeight(PackedWeight.from_dense(w), cuda)
        x = activations(M, K, 42 + M, dtype, integer=True)
        ref = oracle.fast_product(x.double().numpy(), w)
        xd = x.to(cuda)
        cases = {"row-major": (xd, 0), "k-major": (xd.t().contiguous(), 1)}
        wide = torch.zeros((M, K + 3), dtype=dtype, device=cuda)           # rows with an odd leading dimension
        wide[:, :K] = xd
        cases["row-major, strided"] = (wide[:, :K], 0)
        widek = torch.zeros((K, M + 5), dtype=dtype, device=cuda)          # K-major with an odd leading dimension
        widek[:, :M] = xd.t()
        cases["k-major, strided"] = (widek[:, :M], 1)
        for name, (xin, layout) in cases.items():
            print(f"case M={M} K={K} dtype={dtype} {name}", flush=True)
            y = ops.spmm(dw, xin, x_layout=layout).float().cpu().numpy()
            assert np.array_equal(y.astype(np.float64), ref), (M, K, name)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_rows_kernel_with_and_without_shared_out_tiles(cuda, oracle, dtype):
    """The row-parallel kernel in both launch modes (one workgroup per output tile; K tiles shared out
    among one workgroup per compute unit, partial sums added by the fix-up launch), plain and fused."""
    from ternaryllm_amd import ops
    from ternaryllm_amd.packing import PackedWeight
    for M, K, N in ((70, 1300, 200), (520, 2100, 130), (1100, 777, 330)):
        wg = ternary_weight(K, N, 0.75, 51 + M)
        wu = ternary_weight(K, N, 0.75, 52 + M)
        dg, du = ops.DeviceWeight(PackedWeight.from_dense(wg), cuda), ops.DeviceWeight(PackedWeight.from_dense(wu), cuda)
        x = activations(M, K, 53 + M, dtype, integer=True)
        ref = oracle.fast_product(x.double().numpy(), wg)
        xf = activations(M, K, 54 + M, dtype)
        sg = (0.5 + torch.rand(N, generator=torch.Generator().manual_seed(55))).to(dtype)
        g = (xf.double() @ torch.from_numpy(wg).double()) * sg.double()
        u = (xf.double() @ torch.from_numpy(wu).double()) * sg.double()
        ref_fused = (torch.nn.functional.silu(g) * u).numpy()
        fused = {}
        for mode in ("0", "1"):
            print(f"case M={M} K={K} N={N} dtype={dtype} split={mode}", flush=True)
            with knobs(TL_ROWS_SPLIT=mode):
                y = ops.spmm(dg, x.to(cuda), out_dtype=torch.float32).cpu().numpy()
                h = ops.mlp_gate_up(dg, du, xf.to(cuda), sg.to(cuda), sg.to(cuda), out_dtype=torch.float32).cpu().numpy()
            assert np.array_equal(y.astype(np.float64), ref), (M, K, N, mode)
            scale = np.abs(ref_fused).max()
            assert np.abs(h - ref_fused).max() <= (FP16_TOL if dtype == torch.float16 else 1e-4) * scale, (M, K, N, mode)
            fused[mode] = h


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_output_into_a_strided_buffer(cuda, oracle, dtype):
    """`out=` as a column slice of a wider buffer: leading dimensions that allow the row kernel's whole-row
    stores and ones that do not, for both kernels; nothing outside the slice may be touched."""
    from ternaryllm_amd import ops
    from ternaryllm_amd.packing import PackedWeight
    K, N = 600, 256
    w = ternary_weight(K, N, 0.8, 61)
    dw = ops.DeviceWeight(PackedWeight.from_dense(w), cuda)
    for M in (3, 20, 300):
        x = activations(M, K, 62 + M, dtype, integer=True)
        ref = oracle.fast_product(x.double().numpy(), w)
        for width, first in ((N + 4, 4), (N + 5, 3), (N + 8, 0), (N + 1, 1)):
            buf = torch.full((M, width), 7.0, dtype=torch.float32, device=cuda)
            out = buf[:, first:first + N]
            print(f"case M={M} dtype={dtype} width={width} first={first}", flush=True)
            ops.spmm(dw, x.to(cuda), out_dtype=torch.float32, out=out)
            got = buf.cpu().numpy()
            assert np.array_equal(got[:, first:first + N].astype(np.float64), ref), (M, width, first)
            mask = np.ones(width, bool)
            mask[first:first + N] = False
            assert (got[:, mask] == 7.0).all(), (M, width, first)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_small_m_kernels_in_every_mode(cuda, oracle, dtype):
    """The direct-load kernels in the modes a default launch of a small shape does not reach: 8- and 16-row
    slots, one group of tiles or two alternating buffers, several lane groups per run or one, 512 or 1024
    threads for a single row; and the register-staged kernel on a single row."""
    from ternaryllm_amd import ops
    from ternaryllm_amd.packing import PackedWeight
    K, N = 2100, 200  # 9 tiles, the last one short; 13 column blocks, the last one narrow
    w = ternary_weight(K, N, 0.7, 71)
    dw = ops.DeviceWeight(PackedWeight.from_dense(w), cuda)
    settings = [{}, {"TL_TILE_GROUP": "1"}, {"TL_TILE_GROUP": "4"}, {"TL_LW": "1"}, {"TL_LW": "8", "TL_TILE_GROUP": "2"}]
    for M in (1, 6, 16, 37):
        x = activations(M, K, 72 + M, dtype, integer=True)
        ref = oracle.fast_product(x.double().numpy(), w)
        extra = [{"TL_SPMV_DIRECT": "0"}, {"TL_SPMV_WIDE": "0"}, {"TL_SPMV_WIDE": "1"}, {"TL_SPMV_WIDE": "1", "TL_TILE_GROUP": "2"},
                 {"TL_SPMV_TILES": "1"}, {"TL_SPMV_TILES": "1", "TL_SPMV_WIDE": "0"}, {"TL_SPMV_TILES": "0"}] if M == 1 else [{"TL_SMALL_MT": "8"}, {"TL_SMALL_MT": "16"}, {"TL_SMALL_MT": "16", "TL_TILE_GROUP": "2"},
                                   {"TL_SMALL_MT": "16", "TL_OCTET": "1"}, {"TL_SMALL_MT": "16", "TL_OCTET": "1", "TL_TILE_GROUP": "1"},
                                   {"TL_SMALL_MT": "16", "TL_OCTET": "1", "TL_LW": "1", "TL_TILE_GROUP": "8"},
                                   {"TL_QUAD_WIDE": "0"}, {"TL_QUAD_WIDE": "1", "TL_LW": "2"}, {"TL_QUAD_WIDE": "1", "TL_TILE_GROUP": "1"},
                                   {"TL_RES16": "1"}, {"TL_RES16": "0"}]
        for env in settings + extra:
            print(f"case M={M} dtype={dtype} env={env}", flush=True)
            with knobs(**env):
                y = ops.spmm(dw, x.to(cuda), out_dtype=torch.float32).cpu().numpy()
            assert np.array_equal(y.astype(np.float64), ref), (M, env)


def test_resident_16_row_kernel_and_its_epilogues(cuda, oracle):
    """9 to 16 rows with the activation image resident in LDS (tl_spmm_res, TL_RES16=1): exact on integer
    activations against the oracle -- one and several blocks per workgroup, ragged K and N, dense and sparse
    weights (runs longer than a lane's registers hold), a tile height with a single zero slot -- and every epilogue
    (scale, fp32 output, SiLU gate row-major and K-major, residual, next-norm image and squares, row factors)
    bit for bit against the kernels it stands in for (TL_RES16=0)."""
    from ternaryllm_amd import ops, _lib
    from ternaryllm_amd.packing import PackedWeight
    for K, N, M, s, tile_rows in ((2100, 200, 16, 0.7, 0), (4096, 4720, 13, 0.66, 0), (1000, 40, 9, 0.2, 0), (4000, 4400, 16, 0.9, 0),
                                  (1530, 336, 16, 0.62, 255), (300, 16, 11, 0.05, 0)):
        w = ternary_weight(K, N, s, 90 + M)
        dw = ops.DeviceWeight(PackedWeight.from_dense(w, tile_rows), cuda)
        x = activations(M, K, 91 + M, torch.float16, integer=True)
        ref = oracle.fast_product(x.double().numpy(), w)
        g = torch.Generator().manual_seed(92 + M)
        scale = (0.5 + torch.rand(N, generator=g)).half().to(cuda) / 32
        res = torch.randn((M, N), generator=g).half().to(cuda)
        nw = (0.5 + torch.rand(N, generator=g)).half().to(cuda)
        xd = x.to(cuda)
        ximg, _ = ops._kmajor_image(M, K, xd)
        ximg[:, :M] = xd.t()
        xk = ximg[:, :M]
        sq = torch.rand(((K + 15) // 16, 16), generator=g).to(cuda) * 50
        outs = {}
        for tag, env in (("old", {"TL_RES16": "0"}), ("new", {"TL_RES16": "1"})):
            print(f"case K={K} N={N} M={M} s={s} tile_rows={tile_rows} {tag}", flush=True)
            with knobs(**env):
                o = {"plain32": ops.spmm(dw, xd, out_dtype=torch.float32), "plain": ops.spmm(dw, xd, scale),
                     "kmajor": ops.spmm(dw, xk, scale, x_layout=_lib.TL_X_K_MAJOR),
                     "res": ops.spmm_chain(dw, xk, scale, x_layout=_lib.TL_X_K_MAJOR, residual=res),
                     "factors": ops.spmm_chain(dw, xk, scale, x_layout=_lib.TL_X_K_MAJOR, squares_in=sq, eps=1e-5)}
                if tag == "new" or N < 16384:  # (the kernel for wide outputs has no image epilogue)
                    o["image"] = ops.spmm_chain(dw, xk, scale, x_layout=_lib.TL_X_K_MAJOR, residual=res, next_norm_weight=nw, squares_in=sq, eps=1e-5)
                if N % 2 == 0:
                    o["gated"] = ops.spmm_gated(dw, xd, scale)
                    o["gated_k"] = ops.spmm_gated(dw, xk, scale, x_layout=_lib.TL_X_K_MAJOR, kmajor=True)
                    o["gated_factors"] = ops.spmm_chain(dw, xk, scale, x_layout=_lib.TL_X_K_MAJOR, squares_in=sq, eps=1e-5, gated=True, kmajor=True)
            torch.cuda.synchronize()
            outs[tag] = o
        assert np.array_equal(outs["new"]["plain32"].cpu().numpy().astype(np.float64), ref), (K, N, M)
        for name, got in outs["new"].items():
            want = outs["old"].get(name)
            if want is None:
                continue
            pairs = zip(got, want) if isinstance(got, tuple) else ((got, want),)
            for a, b in pairs:
                assert torch.equal(a, b), (K, N, M, name)
        if "gated_k" in outs["new"]:  # the padding rows of a K-major image are zeros
            img = outs["new"]["gated_k"]
            assert not img.as_strided((N // 2, 16), (16, 1))[:, M:].any()
        # fp32 rows: slots of eight, two workgroups side by side; row-major rows (turned inside the kernel) and a K-major image
        x32 = x.float().to(cuda)
        scale32 = scale.float()
        for tag, env in (("old", {"TL_RES16": "0"}), ("new", {"TL_RES16": "1"})):
            print(f"case K={K} N={N} M={M} s={s} tile_rows={tile_rows} fp32 {tag}", flush=True)
            with knobs(**env):
                outs[tag] = {"plain": ops.spmm(dw, x32), "scaled": ops.spmm(dw, x32, scale32),
                             "kmajor": ops.spmm(dw, x32.t().contiguous(), scale32, x_layout=_lib.TL_X_K_MAJOR),
                             "strided": ops.spmm(dw, torch.cat([x32, x32], 1)[:, :K], scale32)}
            torch.cuda.synchronize()
        assert np.array_equal(outs["new"]["plain"].cpu().numpy().astype(np.float64), ref), (K, N, M)
        for name in outs["new"]:
            assert torch.equal(outs["new"][name], outs["old"][name]), (K, N, M, name)
