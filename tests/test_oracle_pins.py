"""Pins the CPU oracle itself: every check here would fail on a plausible mistake in the oracle
(a dropped term, a wrong sign or index, a transposed operand).  The reference holds no golden
vectors for this path, so the pins are library routines (scipy CSC), closed forms, brute force
on tiny inputs, hand-worked tiles and special cases that reduce to simpler formats."""
import numpy as np
import pytest
import scipy.sparse as sp

from tests.util import ternary_weight


def rand_w(rng, K, N, p_zero=0.5):
    r = rng.random((K, N))
    w = np.zeros((K, N), np.int32)
    w[r >= p_zero] = -1
    w[r >= (p_zero + 1) / 2] = 1
    return w


@pytest.mark.parametrize("K,N", [(16, 16), (64, 24), (300, 70), (1, 5), (5, 1)])
def test_csc_equals_scipy(oracle, K, N):
    w = rand_w(np.random.default_rng(K * 131 + N), K, N)
    neg_row, neg_off, pos_row, pos_off = oracle.csc(w)
    for rows, offs, sign in ((pos_row, pos_off, 1), (neg_row, neg_off, -1)):
        c = sp.csc_matrix(w == sign)
        c.sort_indices()
        assert np.array_equal(c.indices, rows)
        assert np.array_equal(c.indptr, offs)


def test_csc_brute_force_tiny(oracle):
    w = np.array([[1, 0, -1], [0, -1, 1], [1, 1, 0], [-1, 0, 1]], np.int32)  # K=4, N=3
    neg_row, neg_off, pos_row, pos_off = oracle.csc(w)
    assert pos_row.tolist() == [0, 2, 2, 1, 3] and pos_off.tolist() == [0, 2, 3, 5]
    assert neg_row.tolist() == [3, 1, 0] and neg_off.tolist() == [0, 1, 2, 3]


@pytest.mark.parametrize("K,N,tk", [(16, 16, 8), (64, 24, 16), (512, 40, 64), (1024, 8, 256), (100, 7, 32)])
def test_tiled_csc_closed_form(oracle, K, N, tk):
    """row_local = row % TILE_K; start = exclusive cumsum of per-(column, tile) counts in (column, tile) order."""
    w = rand_w(np.random.default_rng(7 * K + N), K, N, 0.6)
    neg_row, neg_off, pos_row, pos_off = oracle.tiled_csc(w, tk)
    g_neg_row, _, g_pos_row, _ = oracle.csc(w)
    T = -(-K // tk)
    for rows_t, offs_t, rows_g, sign in ((pos_row, pos_off, g_pos_row, 1), (neg_row, neg_off, g_neg_row, -1)):
        assert np.array_equal(rows_t, rows_g % tk)
        wpad = np.zeros((T * tk, N), bool)
        wpad[:K] = w == sign
        cnt = wpad.reshape(T, tk, N).sum(1).T.reshape(-1)          # [column][tile]
        start = np.concatenate([[0], np.cumsum(cnt)[:-1]])
        assert np.array_equal(offs_t[0::2], start)
        assert np.array_equal(offs_t[1::2], start + cnt)
        # invariants: contiguous, ascending inside a tile, in range
        assert offs_t[-1] == (w == sign).sum()
        assert np.array_equal(offs_t[1:-1:2], offs_t[2::2])
        for c in range(N * T):
            seg = rows_t[offs_t[2 * c]:offs_t[2 * c + 1]]
            assert np.all(np.diff(seg) > 0) and (seg.size == 0 or (seg.min() >= 0 and seg.max() < tk))


def decode_tiled(neg_row, neg_off, pos_row, pos_off, K, N, tk):
    T = -(-K // tk)
    w = np.zeros((K, N), np.int32)
    for y in range(N):
        for t in range(T):
            c = y * T + t
            w[t * tk + pos_row[pos_off[2 * c]:pos_off[2 * c + 1]], y] = 1
            w[t * tk + neg_row[neg_off[2 * c]:neg_off[2 * c + 1]], y] = -1
    return w


def test_tiled_csc_round_trip(oracle):
    w = rand_w(np.random.default_rng(3), 200, 33, 0.7)
    assert np.array_equal(decode_tiled(*oracle.tiled_csc(w, 64), 200, 33, 64), w)


def one_tile(pos_rows, neg_rows, tk=16):
    w = np.zeros((tk, 1), np.int32)
    w[pos_rows, 0] = 1
    w[neg_rows, 0] = -1
    return w


def hand_cases():
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "mcsc_hand_cases.json")) as f:
        return json.load(f)["cases"]


def hand_case_weight(case):
    w = np.zeros((case["inners"], 1), np.int32)
    w[case["pos_rows"], 0] = 1
    w[case["neg_rows"], 0] = -1
    return w


@pytest.mark.parametrize("case", hand_cases(), ids=lambda c: c["name"][:40])
def test_mcsc_hand_worked_tiles(oracle, case):
    """tests/golden/mcsc_hand_cases.json: tiles worked out by hand from ter_spmm_wrapper.cu:156-315 (the
    4-alignment truncation :277-291, padding with overwrite :253-275, the truncated cursor :293-300)."""
    rows, off, tiles = oracle.tiled_mcsc(hand_case_weight(case), case["tile_k"], case["padding"], case["padding_size"])
    assert rows.tolist() == case["merged_row_idx"]
    assert off.tolist() == case["merged_off"]
    assert tiles.tolist() == case["col_tile_idx"]


@pytest.mark.parametrize("case", hand_cases(), ids=lambda c: c["name"][:40])
def test_mcsc_product_hand_worked(oracle, case):
    """orc_mcsc_product against the hand-worked sums of the fixture (ter_spmm_kernel.cuh:197-300): pairs,
    the same-sign part with its sign, the row offset of a second tile, dropped and mis-signed rows of the
    lossy tiles, a row named twice by padded arrays."""
    x = np.array(case["x"], np.float64)[None, :]
    assert case["x"] == [3 ** (k % 11) + k for k in range(case["inners"])]   # the fixture's activation row, as its note defines it
    assert sum(s * case["x"][r] for s, r in case["product_terms"]) == case["product"]
    rows = np.array(case["merged_row_idx"], np.int32)
    off = np.array(case["merged_off"], np.int32)
    assert oracle.mcsc_product(x, rows, off, 1, case["tile_k"])[0, 0] == case["product"]
    # under the kernels' UNIFORMED flag only the pair part counts: the terms whose position lies before off1
    o = off.reshape(-1, 4)
    n_pair_terms = int((o[:, 1] - o[:, 0]).sum())
    pairs_only = sum(s * case["x"][r] for s, r in case["product_terms"][:n_pair_terms])
    assert oracle.mcsc_product(x, rows, off, 1, case["tile_k"], uniformed=True)[0, 0] == pairs_only
    # a second activation row must not leak into the first, nor the first into the second
    x2 = np.vstack([x, 2.0 * x + 1.0])
    both = oracle.mcsc_product(x2, rows, off, 1, case["tile_k"])
    signs = sum(s for s, _ in case["product_terms"])
    assert both[0, 0] == case["product"] and both[1, 0] == 2 * case["product"] + signs


def test_mcsc_reduces_to_interleave_when_balanced(oracle):
    """Every tile with p == n and p even: the alignment rule is a no-op and the merged stream is the plain
    interleave of the tiled-CSC streams (the clean format of the reference's TernaryCSC.py:97-156)."""
    rng = np.random.default_rng(5)
    K, N, tk = 128, 12, 32
    w = np.zeros((K, N), np.int32)
    for y in range(N):
        for t in range(K // tk):
            pairs = 2 * rng.integers(0, 5)
            rows = rng.choice(tk, 2 * pairs, replace=False)
            w[t * tk + rows[:pairs], y] = 1
            w[t * tk + rows[pairs:], y] = -1
    neg_row, neg_off, pos_row, pos_off = oracle.tiled_csc(w, tk)
    rows, off, _ = oracle.tiled_mcsc(w, tk)
    expect = np.empty(rows.size, np.int32)
    expect[0::2] = pos_row
    expect[1::2] = neg_row
    assert np.array_equal(rows, expect)
    assert np.array_equal(off[0::4], 2 * pos_off[0::2]) and np.array_equal(off[1::4], 2 * pos_off[1::2])
    assert np.array_equal(off[2::4], off[1::4]) and np.all(off[3::4] == 1)
    # and the merged product equals the exact product there
    x = rng.standard_normal((3, K))
    assert np.allclose(oracle.mcsc_product(x, rows, off, N, tk), oracle.dense_product(x, w), atol=1e-12)


@pytest.mark.parametrize("padding", [False, True])
def test_mcsc_invariants(oracle, padding):
    w = ternary_weight(512, 40, 0.7, 9)
    rows, off, tiles = oracle.tiled_mcsc(w, 64, padding, 4)
    o = off.reshape(-1, 4)
    assert np.all((o[:, 1] - o[:, 0]) % 4 == 0) and np.all((o[:, 2] - o[:, 1]) % 4 == 0)
    assert np.all(np.isin(o[:, 3], (1, -1))) and np.all(o[:, 2] >= o[:, 1]) and np.all(o[:, 1] >= o[:, 0])
    if not padding:
        assert np.array_equal(o[1:, 0], o[:-1, 2])  # a tile starts where the previous one's kept entries end
    lengths = (o[:, 2] - o[:, 0]).reshape(40, 8)
    assert np.array_equal(tiles.reshape(40, 8), np.argsort(lengths, axis=1, kind="stable"))


def test_dense_product_against_numpy_and_special_cases(oracle):
    rng = np.random.default_rng(11)
    K, N, M = 90, 17, 4
    w = rand_w(rng, K, N)
    x = rng.standard_normal((M, K))
    assert np.allclose(oracle.dense_product(x, w), x @ w, rtol=0, atol=1e-12)
    assert np.array_equal(oracle.fast_product(x, w), x @ w.astype(np.float64))
    # not symmetric in its operands: a transposed W must change the answer
    wsq = rand_w(rng, K, K)
    assert not np.allclose(oracle.dense_product(x, wsq), x @ wsq.T)
    assert not oracle.dense_product(x, np.zeros((K, N), np.int32)).any()
    rows = rng.integers(0, K, N)
    signs = rng.choice([-1, 1], N)
    w1 = np.zeros((K, N), np.int32)
    w1[rows, np.arange(N)] = signs
    assert np.array_equal(oracle.dense_product(x, w1), x[:, rows] * signs[None, :])
    assert np.allclose(oracle.dense_product(x, np.ones((K, 1), np.int32))[:, 0], x.sum(1), atol=1e-12)
