"""Host packers of the library against the oracle (bit-exact), the device blob round trip, the
drop-in module surface and the error behaviour at the C boundary.  No GPU needed."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from tests.util import ternary_weight

from ternaryllm_amd import _lib, packing


CASES = [(16, 16, 8), (64, 24, 16), (512, 96, 64), (1024, 40, 256), (1000, 70, 256), (2048, 33, 256), (4096, 16, 512),
         (300, 130, 100), (8, 200, 4)]


@pytest.mark.parametrize("K,N,tk", CASES)
@pytest.mark.parametrize("sparsity", [0.0, 0.5, 0.9])
def test_packers_bit_exact(oracle, K, N, tk, sparsity):
    w = ternary_weight(K, N, sparsity, K + 3 * N)
    cp, cn = packing.count_nnz(w)
    assert (cp, cn) == oracle.count_nnz(w)
    for got, want in zip(packing.convert_to_ter_csc(w, N, K, cp, cn), oracle.csc(w)):
        assert got.dtype == np.int32 and np.array_equal(got, want)
    for got, want in zip(packing.convert_to_ter_tiled_csc(w, N, K, cp, cn, tk), oracle.tiled_csc(w, tk)):
        assert np.array_equal(got, want)
    for padding in (False, True):
        got = packing.convert_to_ter_tiled_mcsc(w, N, K, cp, cn, tk, padding, 4)
        want = oracle.tiled_mcsc(w, tk, padding, 4)
        assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])
        T = -(-K // tk)
        if T <= 16:   # above 16 tiles per column the reference's std::sort leaves tie order to the implementation
            assert np.array_equal(got[2], want[2])
        else:
            lengths = (got[1].reshape(-1, 4)[:, 2] - got[1].reshape(-1, 4)[:, 0]).reshape(N, T)
            perm = got[2].reshape(N, T)
            assert np.array_equal(np.sort(perm, axis=1), np.tile(np.arange(T), (N, 1)))
            assert np.all(np.diff(np.take_along_axis(lengths, perm, axis=1), axis=1) >= 0)


def test_empty_and_extreme_weights(oracle):
    for w in (np.zeros((64, 20), np.int32), np.ones((64, 20), np.int32), -np.ones((300, 3), np.int32)):
        K, N = w.shape
        cp, cn = packing.count_nnz(w)
        for got, want in zip(packing.convert_to_ter_tiled_mcsc(w, N, K, cp, cn, 32, False, 4), oracle.tiled_mcsc(w, 32)):
            assert np.array_equal(got, want)
        pw = packing.PackedWeight.from_dense(w)
        pw.validate()
        assert np.array_equal(pw.to_dense(), w)


@pytest.mark.parametrize("K,N", [(1, 1), (255, 16), (256, 17), (4096, 64), (11008 // 4, 48), (777, 130)])
@pytest.mark.parametrize("tile_rows", [0, 255, 128, 37])
def test_device_blob_round_trip(K, N, tile_rows):
    w = ternary_weight(K, N, 0.66, K * 7 + N)
    pw = packing.PackedWeight.from_dense(w, tile_rows)
    pw.validate()
    h = pw.header
    assert h.inners == K and h.columns == N and h.nnz_pos == (w == 1).sum() and h.nnz_neg == (w == -1).sum()
    assert 1 <= h.tile_rows <= 255 and h.n_tiles == -(-K // h.tile_rows) and h.n_blocks == -(-N // 16)
    assert h.total_bytes == pw.blob.size and h.total_bytes % 256 == 0 and h.stream_bytes % 16 == 0
    assert np.array_equal(pw.to_dense(), w)
    # the same blob comes out of the tiled-CSC entry point, whatever tile height the API arrays use
    cp, cn = packing.count_nnz(w)
    for tk in (256, 64):
        arrs = packing.convert_to_ter_tiled_csc(w, N, K, cp, cn, tk)
        pw2 = packing.PackedWeight.from_tiled_csc(*arrs, N, K, tk, tile_rows)
        assert np.array_equal(pw2.blob, pw.blob)


def test_blob_does_not_depend_on_the_packing_threads(monkeypatch):
    """The row-ordering pass of tl_layout_build runs on worker threads (TL_PACK_THREADS, read at every call): the
    blob is the same byte for byte for 1, 3 and 8 of them, and when several calls pack at the same time."""
    from concurrent.futures import ThreadPoolExecutor
    w = ternary_weight(1000, 200, 0.66, 31)
    blobs = []
    for n in ("1", "3", "8"):
        monkeypatch.setenv("TL_PACK_THREADS", n)
        blobs.append(bytes(packing.PackedWeight.from_dense(w).blob))
    assert blobs[0] == blobs[1] == blobs[2]
    monkeypatch.delenv("TL_PACK_THREADS")
    with ThreadPoolExecutor(max_workers=4) as pool:
        together = list(pool.map(lambda _: bytes(packing.PackedWeight.from_dense(w).blob), range(6)))
    assert all(b == blobs[0] for b in together)


def test_blob_validation_catches_corruption():
    w = ternary_weight(512, 40, 0.6, 77)
    pw = packing.PackedWeight.from_dense(w)
    h = pw.header
    for pos in (0, 4, int(h.off_chunkstart) + 4, int(h.off_stream) + 3, int(h.off_stream) + 16 * 4 + 1):
        bad = pw.blob.copy()
        bad[pos] ^= 0x5A
        with pytest.raises(ValueError):
            packing.PackedWeight(bad).validate()
    with pytest.raises(ValueError):
        packing.PackedWeight(pw.blob[:300])


def test_mcsc_decodes_to_the_matrix_it_encodes(oracle):
    """tl_tiled_mcsc_to_dense against the oracle's walk of the merged arrays."""
    rng = np.random.default_rng(2)
    w = ternary_weight(256, 24, 0.6, 5)
    cp, cn = packing.count_nnz(w)
    rows, off, _ = packing.convert_to_ter_tiled_mcsc(w, 24, 256, cp, cn, 64, False, 4)
    w_eff = packing.tiled_mcsc_to_dense(rows.astype(np.int16), off, 24, 256, 64)
    x = rng.standard_normal((5, 256))
    assert np.allclose(oracle.mcsc_product(x, rows, off, 24, 64), oracle.dense_product(x, w_eff), atol=1e-12)
    assert np.count_nonzero(w_eff) <= np.count_nonzero(w)  # the alignment rule only ever drops entries
    with pytest.raises(ValueError):
        packing.tiled_mcsc_to_dense(rows.astype(np.int16), off[:-4], 24, 256, 64)


def _hand_cases():
    import json
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "mcsc_hand_cases.json")) as f:
        return json.load(f)["cases"]


@pytest.mark.parametrize("case", _hand_cases(), ids=lambda c: c["name"][:40])
def test_blob_from_merged_arrays_encodes_the_hand_worked_terms(case):
    """tl_layout_from_mcsc on the fixture's arrays: the integer matrix the blob decodes to is the sum of the
    hand-worked terms (a row named twice counts twice), also with the same-sign part left out."""
    rows = np.array(case["merged_row_idx"], np.int16)
    off = np.array(case["merged_off"], np.int32)
    K, tk = case["inners"], case["tile_k"]
    o = off.reshape(-1, 4)
    n_pair_terms = int((o[:, 1] - o[:, 0]).sum())
    for uniformed, terms in ((False, case["product_terms"]), (True, case["product_terms"][:n_pair_terms])):
        want = np.zeros((K, 1), np.int32)
        for s, r in terms:
            want[r, 0] += s
        pw = packing.PackedWeight.from_mcsc(rows, off, 1, K, tk, uniformed)
        pw.validate()
        assert np.array_equal(pw.to_dense(), want)
    if np.abs(want).max() <= 1 and not case["padding"]:
        assert np.array_equal(packing.tiled_mcsc_to_dense(rows, off, 1, K, tk), packing.PackedWeight.from_mcsc(rows, off, 1, K, tk).to_dense())


@pytest.mark.parametrize("padding", [False, True])
def test_blob_from_merged_arrays_matches_the_oracle_walk(oracle, padding):
    rng = np.random.default_rng(4)
    K, N, tk = 512, 40, 256
    w = ternary_weight(K, N, 0.7, 15)
    cp, cn = packing.count_nnz(w)
    rows, off, _ = packing.convert_to_ter_tiled_mcsc(w, N, K, cp, cn, tk, padding, 4)
    x = rng.integers(-8, 9, (3, K)).astype(np.float64)
    for uniformed in (False, True):
        pw = packing.PackedWeight.from_mcsc(rows.astype(np.int16), off, N, K, tk, uniformed)
        pw.validate()
        assert np.array_equal(x @ pw.to_dense().astype(np.float64), oracle.mcsc_product(x, rows, off, N, tk, uniformed))
    with pytest.raises(ValueError):
        bad = rows.copy()
        bad[off[0]] = tk  # a row index outside its tile
        packing.PackedWeight.from_mcsc(bad, off, N, K, tk)


@pytest.mark.parametrize("K,N,s,seed", [(4096, 11008, 0.8, 1237), (2048, 2048, 0.9, 3), (256, 16, 0.99, 1), (4096, 48, 0.0, 2)])
def test_index_prefetch_stays_inside_the_blob(K, N, s, seed):
    """The row kernel requests 192 index dwords from the start of every wave's piece of a chunk (a wave owns 4 or
    8 neighbouring columns) and, for longer pieces, whole 64-dword groups up to 63 dwords past the piece's end:
    the furthest byte either touches must lie inside the blob as trimmed to header.total_bytes."""
    if K * N > 1 << 24:
        rng = np.random.default_rng(seed)   # the torch generator is slow at this size
        r = rng.random((K, N), dtype=np.float32)
        w = np.zeros((K, N), np.int32)
        w[r >= s] = -1
        w[r >= (s + 1) / 2] = 1
    else:
        w = ternary_weight(K, N, s, seed)
    pw = packing.PackedWeight.from_dense(w)
    h = pw.header
    assert pw.blob.size == h.total_bytes
    stream = pw.blob[h.off_stream:].view(np.uint32)
    cs = pw.blob[h.off_chunkstart:h.off_chunkstart + (h.n_tiles * h.n_blocks + 1) * 4].view(np.uint32).astype(np.int64)
    room = (h.total_bytes - h.off_stream) // 4   # dwords from the stream's start to the blob's end
    for C in (4, 8):
        subs = np.arange(0, 16, C)
        d_first = stream[cs[:-1, None] + subs[None, :]].astype(np.int64)             # descriptor of a wave's first column
        d_last = stream[cs[:-1, None] + subs[None, :] + C - 1].astype(np.int64)      # ... and of its last
        base = cs[:-1, None] + (d_first >> 16)
        end = cs[:-1, None] + (d_last >> 16) + ((d_last & 0xff) + 3) // 4 + (((d_last >> 8) & 0xff) + 3) // 4
        total = end - base
        assert (base + 192).max() <= room
        groups = -(-total // 64)
        assert (base + np.maximum(groups, 3) * 64).max() <= room


def test_error_behaviour():
    w = ternary_weight(64, 8, 0.5, 1)
    cp, cn = packing.count_nnz(w)
    with pytest.raises(ValueError):   # counts that do not match the matrix (the reference would overrun its vectors)
        packing.convert_to_ter_csc(w, 8, 64, cp + 1, cn)
    with pytest.raises(ValueError):   # columns / inners swapped
        packing.convert_to_ter_csc(w, 64, 8, cp, cn)
    with pytest.raises(ValueError):   # wrong dtype (the reference's data_ptr<int32_t> throws)
        packing.convert_to_ter_csc(w.astype(np.int64), 8, 64, cp, cn)
    with pytest.raises(ValueError):   # not ternary
        packing.count_nnz(np.full((4, 4), 2, np.int32))
    with pytest.raises(ValueError):
        packing.convert_to_ter_tiled_csc(w, 8, 64, cp, cn, 0)
    with pytest.raises(ValueError):
        packing.PackedWeight.from_dense(w, tile_rows=256)
    assert _lib.lib().tl_last_error()  # a message was recorded


def test_library_exports_every_declared_symbol():
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    header = open(os.path.join(root, "include", "ternary_spmm.h")).read()
    declared = set(re.findall(r"\b(tl_[a-z0-9_]+)\s*\(", header))
    declared -= {"tl_layout_header"}
    assert declared, "no declarations found"
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for name in sorted(declared):
        assert hasattr(handle, name), f"{name} is declared in the header but not exported"
        assert name in _lib.SIGNATURES, f"{name} has no Python binding"
    assert handle.tl_version() >= 1
    assert ctypes.sizeof(_lib.LayoutHeader) == 256


def test_drop_in_module_surface():
    import ter_spmm
    for name in ("ter_spmm", "convert_to_ter_csc", "convert_to_ter_tiled_csc", "convert_to_ter_tiled_mcsc"):
        assert callable(getattr(ter_spmm, name))
    # same call shape as the reference's only caller (TernaryLinear.py:104-112)
    w = torch.from_numpy(ternary_weight(512, 32, 0.8, 3))
    cnt_pos, cnt_neg = (w == 1).sum().item(), (w == -1).sum().item()
    tm = ter_spmm.convert_to_ter_tiled_mcsc(w, w.size(1), w.size(0), cnt_pos, cnt_neg, 64, False, 4)
    rows = torch.tensor(np.array(tm[0]), dtype=torch.int32).to(torch.int16)
    assert rows.numel() == cnt_pos + cnt_neg and len(tm) == 3
    with pytest.raises(RuntimeError):  # CPU tensors are refused, as the reference's device assert does
        ter_spmm.ter_spmm(torch.zeros(1, 4, 512), rows, torch.tensor(tm[1]), torch.tensor(tm[2]), 1, 4, 32, 512, False, False)


def test_modules_build_on_cpu_and_refuse_to_run_there():
    from ternaryllm_amd import LlamaTernaryMLP, TernaryConfig, TernaryLinear, random_ternary_weights
    g = torch.Generator().manual_seed(0)
    lin = TernaryLinear(512, 96, sparsity=0.8, bias=False, generator=g)
    assert lin.w_row_indices.dtype == torch.int16 and lin.w_col_offsets.dtype == torch.int32
    assert lin.w_col_offsets.numel() == 96 * (512 // 64) * 4 and lin.w_col_tile_indices.numel() == 96 * (512 // 64)
    assert "w_packed" in lin.state_dict() and "w_row_indices" not in lin.state_dict()
    with pytest.raises(RuntimeError):
        lin(torch.zeros(2, 512))
    # the i.i.d. generator follows the reference's thresholds
    w = random_ternary_weights((2000, 100), 0.8, generator=g)
    frac = [(w == v).float().mean().item() for v in (0, -1, 1)]
    assert abs(frac[0] - 0.8) < 0.01 and abs(frac[1] - 0.1) < 0.01 and abs(frac[2] - 0.1) < 0.01
    # the uniform generator: every block of a column balanced
    wu = random_ternary_weights((512, 64), 0.75, True, 64, g)
    blocks = wu.T.reshape(64, 8, 64)
    assert torch.all((blocks == 1).sum(-1) == 8) and torch.all((blocks == -1).sum(-1) == 8)
    cfg = TernaryConfig(hidden_size=256, intermediate_size=512, sparsity=0.9)
    mlp = LlamaTernaryMLP(cfg, generator=g)
    assert mlp.gate_proj.out_features == 512 and mlp.down_proj.in_features == 512


def test_cpu_baselines_match_exact_product():
    from oracle import cpu_baseline
    w = ternary_weight(1024, 64, 0.7, 4)
    x = np.random.default_rng(1).standard_normal((64, 1024)).astype(np.float32)
    r = cpu_baseline.time_gemm(w, x, runs=1, prefer_reference=False)
    assert r["kind"] == "port" and r["max_rel_err"] < 1e-5
    try:
        cpu_baseline.ReferenceProvider()
    except (RuntimeError, OSError):
        pytest.skip("reference CPU build not present on this host")
    r = cpu_baseline.time_gemm(w, x, runs=1, prefer_reference=True)
    assert r["kind"] == "reference" and r["max_rel_err"] < 1e-5
    p = cpu_baseline.PortProvider()
    xv = x[0]
    assert np.allclose(p.gemv(np.ascontiguousarray(w, np.int8), xv, 64, 1024), xv.astype(np.float64) @ w, atol=1e-3)
    if "avx512f" in cpu_baseline._cpu_flags():
        assert np.allclose(p.gemv(np.ascontiguousarray(w, np.int8), xv, 64, 1024, wide=True), xv.astype(np.float64) @ w, atol=1e-3)
    # every kernel the host can run, one bound thread per physical core, run statistics beside the mean
    both = cpu_baseline.time_gemm_all(w, x, runs=2)
    assert both[0]["kernel"].endswith("32xG8_AVX2_OpenMP") and all(r["seconds_min"] <= r["seconds_median"] <= r["seconds_max"] for r in both)
    assert both[0]["threads"] == cpu_baseline.threads() <= cpu_baseline.physical_cores()
    for r in cpu_baseline.time_gemv_all(w, xv, runs=2):
        assert r["max_err_over_max"] < 1e-5


def test_compute_entry_points_reject_bad_arguments_before_any_launch():
    """Argument checks of the compute calls run on the host: they must answer without a GPU."""
    L = _lib.lib()
    w = ternary_weight(64, 32, 0.5, 2)
    pw = packing.PackedWeight.from_dense(w)
    hdr = ctypes.byref(pw.header)
    need = ctypes.c_int64(-1)
    assert L.tl_spmm_workspace(hdr, 1, _lib.TL_F16, 0, ctypes.byref(need)) == 0 and need.value == 0
    assert L.tl_spmm_workspace(hdr, 16, _lib.TL_F16, 0, ctypes.byref(need)) == 0 and need.value == 64 * 16 * 2
    assert L.tl_spmm_workspace(hdr, 100, _lib.TL_F16, 0, ctypes.byref(need)) == 0 and need.value > 64 * 256 * 2
    assert L.tl_spmm_workspace(hdr, 0, _lib.TL_F16, 0, ctypes.byref(need)) < 0
    assert L.tl_spmm_workspace(hdr, 4, 7, 0, ctypes.byref(need)) < 0
    fake = ctypes.c_void_p(256 * 1024)  # never dereferenced: every call below fails its checks first
    assert L.tl_spmm(hdr, None, fake, 0, 0, 64, 1, fake, 0, 32, None, 0, None, 0, None) < 0            # null blob
    assert L.tl_spmm(hdr, fake, fake, 0, 0, 10, 1, fake, 0, 32, None, 0, None, 0, None) < 0            # ldx < K
    assert L.tl_spmm(hdr, fake, fake, 0, 0, 64, 1, fake, 0, 8, None, 0, None, 0, None) < 0             # ldy < N
    assert L.tl_spmm(hdr, fake, fake, 0, 2, 64, 1, fake, 0, 32, None, 0, None, 0, None) < 0            # unknown layout
    assert L.tl_spmm(hdr, ctypes.c_void_p(257), fake, 0, 0, 64, 1, fake, 0, 32, None, 0, None, 0, None) < 0  # unaligned blob
    # a chained product outside 9 .. 16 rows is refused, one row or eight included (no launch, nothing ignored)
    chain = _lib.Chain()
    chain.residual, chain.residual_ld = fake.value, 32
    for rows in (1, 8, 17):
        assert L.tl_spmm_chain(hdr, fake, fake, _lib.TL_F16, 0, 64, rows, fake, _lib.TL_F16, 32, -1, None, 0, ctypes.byref(chain), fake, 1 << 20, None) \
            == _lib.TL_ERR_UNSUPPORTED, rows
    pos = ctypes.c_void_p(4096)
    assert L.tl_rope_cache_update(fake, 5, 1, 2, 64, fake, fake, pos, fake, fake, fake, 16, None) < 0  # dtype
    assert L.tl_rope_cache_update(fake, 1, 1, 2, 63, fake, fake, pos, fake, fake, fake, 16, None) < 0  # odd head_dim
    assert L.tl_rope_cache_update(fake, 1, 1, 2, 64, fake, fake, None, fake, fake, fake, 16, None) < 0  # no position
    assert L.tl_decode_attention(fake, fake, fake, 1, 1, 2, 96, 16, pos, fake, 0, None) < 0             # head_dim not served
    assert L.tl_decode_attention(fake, fake, ctypes.c_void_p(4104), 1, 1, 2, 64, 16, pos, fake, 0, None) < 0  # unaligned cache
    assert L.tl_decode_attention(fake, fake, fake, 1, 6, 2, 64, 16, pos, fake, 4, None) < 0             # K-major leading dimension below the batch
    assert L.tl_add_rmsnorm(fake, None, fake, 9, 1, 64, 1e-5, None, fake, 0, None) < 0
    assert L.tl_add_rmsnorm(fake, fake, fake, 1, 1, 64, 1e-5, None, fake, 0, None) < 0                  # y without x_out
    assert L.tl_add_rmsnorm(fake, None, fake, 1, 0, 64, 1e-5, None, fake, 0, None) < 0
    assert L.tl_add_rmsnorm(fake, None, fake, 1, 9, 64, 1e-5, None, fake, 8, None) < 0                  # K-major leading dimension below the rows
    assert L.tl_silu_mul(None, 1, 1, 64, fake, 0, None) < 0
    assert L.tl_silu_mul(fake, 1, 1, 0, fake, 0, None) < 0
    assert L.tl_silu_mul(fake, 1, 9, 64, fake, 8, None) < 0
    assert L.tl_last_error()


def test_library_packer_on_the_hand_worked_tiles():
    """The library's merged packer against tests/golden/mcsc_hand_cases.json (outputs derived by hand from
    the reference's source)."""
    from tests.test_oracle_pins import hand_case_weight, hand_cases
    for case in hand_cases():
        w = hand_case_weight(case)
        cp, cn = packing.count_nnz(w)
        rows, off, tiles = packing.convert_to_ter_tiled_mcsc(w, 1, case["inners"], cp, cn, case["tile_k"], case["padding"],
                                                             case["padding_size"])
        assert rows.tolist() == case["merged_row_idx"], case["name"]
        assert off.tolist() == case["merged_off"], case["name"]
        assert tiles.tolist() == case["col_tile_idx"], case["name"]
