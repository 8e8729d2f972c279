/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the ternary sparse GEMM path.
 *
 * Plain-C restatement of the reference algorithms of fpgasystems/ternaryLLM's
 * GPU extension.  Nothing in the shipped library links, loads or calls this
 * file: only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg
 * may use it, and only as the checker.
 *
 * Each function names the reference lines it restates.  All loops are the
 * naive scalar form on purpose: the oracle must be obviously right, not fast.
 *
 * Pinning status (what checks each function beyond "it was typed carefully"):
 *   orc_csc            -- scipy.sparse.csc_matrix(W == +-1) indices / indptr,
 *                         brute force on tiny W, round trip to dense.
 *   orc_tiled_csc      -- closed form (row % TILE_K, exclusive cumsum of the
 *                         per-(column, tile) counts), invariants, round trip.
 *   orc_tiled_mcsc     -- eight hand-worked cases (tests/golden/mcsc_hand_cases.json:
 *                         odd pair counts on either side, padding with
 *                         overwrite at padding sizes 4 and 8, the cursor
 *                         overwrite across two tiles, padded arrays, four
 *                         tiles of which three tie), the p == n / even case that
 *                         reduces to a plain interleave of orc_tiled_csc, the
 *                         alignment invariants of the offsets.  The reference
 *                         holds no fixture for it and its only other
 *                         implementation computes a different (untruncated)
 *                         format, so beyond those checks: parity unpinned.
 *   orc_tile_swizzle   -- numpy.argsort(kind="stable") per column and the hand case
 *                         with three tied tiles; equals the
 *                         reference's std::sort only while a column has at
 *                         most 16 tiles (libstdc++ then runs a pure insertion
 *                         sort); above that the tie order of the reference is
 *                         implementation-defined: parity unpinned for ties.
 *   orc_dense_product  -- textbook triple loop in double; checked against
 *                         numpy's float64 matmul and the special cases W = 0,
 *                         one +-1 per column, all-ones column.
 *   orc_mcsc_product   -- what the reference kernels' loop structure sums from
 *                         merged arrays (with the tile offset applied to every
 *                         gather; without the same-sign part when `uniformed`).
 *                         Pinned by the six hand cases: the terms of each sum
 *                         are written out by hand in the fixture, for an x
 *                         whose values (3^(k mod 11) + k) let no dropped term,
 *                         wrong sign or missing tile offset go unnoticed, and
 *                         the sums are asserted; also equals orc_dense_product
 *                         on inputs where the merged format is lossless.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------ */
/* ter_spmm_wrapper.cu:39-78  (convert_to_ter_csc)                           */
/* w is row-major int32 [inners][columns]; outputs are sized by the caller:  */
/* neg_row[cnt_neg], neg_off[columns+1], pos_row[cnt_pos], pos_off[cols+1].  */
/* Returns 0, or -1 when the counts handed in do not match W.                */
int orc_csc(const int32_t *w, int columns, int inners, int cnt_pos, int cnt_neg,
            int32_t *neg_row, int32_t *neg_off, int32_t *pos_row, int32_t *pos_off)
{
    int nb_neg = 0, nb_pos = 0;
    for (int y = 0; y < columns; y++) {
        neg_off[y] = nb_neg;
        pos_off[y] = nb_pos;
        for (int x = 0; x < inners; x++) {
            int32_t v = w[(size_t)x * columns + y];
            if (v == -1) {
                if (nb_neg >= cnt_neg) return -1;
                neg_row[nb_neg++] = x;
            } else if (v == 1) {
                if (nb_pos >= cnt_pos) return -1;
                pos_row[nb_pos++] = x;
            }
        }
    }
    neg_off[columns] = nb_neg;
    pos_off[columns] = nb_pos;
    return (nb_neg == cnt_neg && nb_pos == cnt_pos) ? 0 : -1;
}

static int ceil_div(int a, int b) { return (a + b - 1) / b; }

/* ------------------------------------------------------------------------ */
/* ter_spmm_wrapper.cu:92-152  (convert_to_ter_tiled_csc)                    */
/* neg_off_t / pos_off_t hold columns*T*2 entries, T = ceil(inners/tile_k).  */
/* Rows past `inners` in the last tile (the reference would read out of      */
/* bounds there) are taken as zero.                                          */
int orc_tiled_csc(const int32_t *w, int columns, int inners, int cnt_pos, int cnt_neg,
                  int tile_k, int32_t *neg_row, int32_t *neg_off_t,
                  int32_t *pos_row, int32_t *pos_off_t)
{
    int32_t *tmp_neg_off = (int32_t *)malloc(sizeof(int32_t) * (size_t)(columns + 1));
    int32_t *tmp_pos_off = (int32_t *)malloc(sizeof(int32_t) * (size_t)(columns + 1));
    if (!tmp_neg_off || !tmp_pos_off) { free(tmp_neg_off); free(tmp_pos_off); return -2; }
    int rc = orc_csc(w, columns, inners, cnt_pos, cnt_neg, neg_row, tmp_neg_off, pos_row, tmp_pos_off);
    free(tmp_neg_off);
    free(tmp_pos_off);
    if (rc) return rc;

    const int T = ceil_div(inners, tile_k);
    int nb_neg = 0, nb_pos = 0;
    for (int y = 0; y < columns; y++) {
        for (int t = 0; t < T; t++) {
            const int shift = t * tile_k;
            neg_off_t[(size_t)y * T * 2 + t * 2 + 0] = nb_neg;
            pos_off_t[(size_t)y * T * 2 + t * 2 + 0] = nb_pos;
            for (int x = 0; x < tile_k; x++) {
                const int row = shift + x;
                if (row >= inners) break;
                int32_t v = w[(size_t)row * columns + y];
                if (v == -1) { neg_row[nb_neg] -= shift; nb_neg++; }
                else if (v == 1) { pos_row[nb_pos] -= shift; nb_pos++; }
            }
            neg_off_t[(size_t)y * T * 2 + t * 2 + 1] = nb_neg;
            pos_off_t[(size_t)y * T * 2 + t * 2 + 1] = nb_pos;
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* ter_spmm_wrapper.cu:9-27  (inter_tile_swizzle)                            */
/* Per column: tile ids ordered by ascending stored length off[2]-off[0].    */
/* Stable insertion sort (see the header note about std::sort).              */
void orc_tile_swizzle(int columns, int T, const int32_t *merged_off, int32_t *tile_idx)
{
    for (int y = 0; y < columns; y++) {
        const int32_t *o = merged_off + (size_t)y * T * 4;
        int32_t *dst = tile_idx + (size_t)y * T;
        for (int t = 0; t < T; t++) {
            int len_t = (o[t * 4 + 1] - o[t * 4 + 0]) + (o[t * 4 + 2] - o[t * 4 + 1]);
            int j = t;
            while (j > 0) {
                int q = dst[j - 1];
                int len_q = (o[q * 4 + 1] - o[q * 4 + 0]) + (o[q * 4 + 2] - o[q * 4 + 1]);
                if (len_q <= len_t) break;
                dst[j] = q;
                j--;
            }
            dst[j] = t;
        }
    }
}

/* length of the merged index array: ter_spmm_wrapper.cu:180 and :198-230    */
int64_t orc_tiled_mcsc_len(const int32_t *neg_off_t, const int32_t *pos_off_t, int columns,
                           int T, int cnt_pos, int cnt_neg, int padding, int padding_size)
{
    if (!padding) return (int64_t)cnt_pos + cnt_neg;
    int64_t total = 0;
    for (int y = 0; y < columns; y++)
        for (int t = 0; t < T; t++) {
            size_t s = (size_t)y * T * 2 + 2 * t;
            int neg = neg_off_t[s + 1] - neg_off_t[s];
            int pos = pos_off_t[s + 1] - pos_off_t[s];
            int mn = neg <= pos ? neg : pos, mx = neg <= pos ? pos : neg;
            total += (int64_t)ceil_div(2 * mn, padding_size) * padding_size;
            total += (int64_t)ceil_div(mx - mn, padding_size) * padding_size;
        }
    return total;
}

/* ------------------------------------------------------------------------ */
/* ter_spmm_wrapper.cu:156-315  (convert_to_ter_tiled_mcsc)                  */
/* merged_row must hold orc_tiled_mcsc_len() entries and arrive zero-filled  */
/* (the reference value-initialises its vector, :180,229); merged_off holds  */
/* columns*T*4, tile_idx columns*T.                                          */
int orc_tiled_mcsc(const int32_t *w, int columns, int inners, int cnt_pos, int cnt_neg,
                   int tile_k, int padding, int padding_size,
                   int32_t *merged_row, int64_t merged_len, int32_t *merged_off, int32_t *tile_idx)
{
    const int T = ceil_div(inners, tile_k);
    int32_t *neg_row = (int32_t *)malloc(sizeof(int32_t) * (size_t)(cnt_neg + 1));
    int32_t *pos_row = (int32_t *)malloc(sizeof(int32_t) * (size_t)(cnt_pos + 1));
    int32_t *neg_off = (int32_t *)malloc(sizeof(int32_t) * (size_t)columns * T * 2 + 8);
    int32_t *pos_off = (int32_t *)malloc(sizeof(int32_t) * (size_t)columns * T * 2 + 8);
    int rc = -2;
    if (!neg_row || !pos_row || !neg_off || !pos_off) goto done;
    rc = orc_tiled_csc(w, columns, inners, cnt_pos, cnt_neg, tile_k, neg_row, neg_off, pos_row, pos_off);
    if (rc) goto done;
    if (merged_len != orc_tiled_mcsc_len(neg_off, pos_off, columns, T, cnt_pos, cnt_neg, padding, padding_size)) {
        rc = -3;
        goto done;
    }
    {
        int64_t cursor = 0; /* prev_cnt == prev_nnz after every tile (:299-300) */
        for (int y = 0; y < columns; y++) {
            for (int t = 0; t < T; t++) {
                size_t s = (size_t)y * T * 2 + 2 * t;
                int ns = neg_off[s], ne = neg_off[s + 1];
                int ps = pos_off[s], pe = pos_off[s + 1];
                int neg = ne - ns, pos = pe - ps;
                int neg_is_min = neg <= pos;
                int mn = neg_is_min ? neg : pos;
                int mx = neg_is_min ? pos : neg;

                int n_pair = 2 * mn;
                int n_pair_pad = padding ? ceil_div(n_pair, padding_size) * padding_size : n_pair;
                for (int k = 0; k < mn; k++) {               /* :253-256 */
                    merged_row[cursor + 2 * k + 0] = pos_row[ps + k];
                    merged_row[cursor + 2 * k + 1] = neg_row[ns + k];
                }
                for (int k = n_pair; k < n_pair_pad; k++)     /* :259-261 */
                    merged_row[cursor + k] = pos_row[ps];
                int n_rest = mx - mn;
                int n_rest_pad = padding ? ceil_div(n_rest, padding_size) * padding_size : n_rest;
                for (int k = mn; k < mx; k++)                 /* :266-275 */
                    merged_row[cursor + k + mn] = neg_is_min ? pos_row[ps + k] : neg_row[ns + k];

                if (n_rest % 2 == 1) n_rest--;                /* :279-291 */
                if (n_pair % 4 != 0) n_pair -= 2;
                if (n_rest % 4 != 0) n_rest -= 2;

                size_t o = (size_t)y * T * 4 + 4 * t;          /* :293-297 */
                merged_off[o + 0] = (int32_t)cursor;
                merged_off[o + 1] = (int32_t)(cursor + (padding ? n_pair_pad : n_pair));
                merged_off[o + 2] = merged_off[o + 1] + n_rest;
                merged_off[o + 3] = neg_is_min ? 1 : -1;
                cursor += padding ? (n_pair_pad + n_rest_pad) : (n_pair + n_rest); /* :299 */
            }
        }
    }
    orc_tile_swizzle(columns, T, merged_off, tile_idx);
    rc = 0;
done:
    free(neg_row); free(pos_row); free(neg_off); free(pos_off);
    return rc;
}

/* ------------------------------------------------------------------------ */
/* The exact product the path is judged against: Y = X * W in double.        */
/* It is the standard the reference's own CPU checks use                     */
/* (ternaryLLM_CPU/src/main.cpp:1485-1500, GEMM_CPU_FP32.cpp:8-18).          */
/* x: row-major double [M][K]; w: row-major int32 [K][N]; y: double [M][N].  */
void orc_dense_product(const double *x, const int32_t *w, double *y, int M, int N, int K)
{
    for (int m = 0; m < M; m++)
        for (int n = 0; n < N; n++) {
            double acc = 0.0;
            for (int k = 0; k < K; k++) {
                int32_t v = w[(size_t)k * N + n];
                if (v == 1) acc += x[(size_t)m * K + k];
                else if (v == -1) acc -= x[(size_t)m * K + k];
            }
            y[(size_t)m * N + n] = acc;
        }
}

/* ------------------------------------------------------------------------ */
/* What the merged arrays encode, summed the way the reference kernels walk  */
/* them (ter_spmm_kernel.cuh:197-300 and :44-68): per tile, pairs            */
/* (+x[p] - x[n]) over [off0, off1), then sign * sum x[c] over [off1, off2). */
/* Every gather uses the tile's row offset (the SpMV remainder loop at :63   */
/* omits it; that omission is a defect, not part of the format).             */
/* uniformed != 0: the [off1, off2) part is skipped, as both kernels do under */
/* their UNIFORMED template flag (ter_spmm_kernel.cuh:59, :249).              */
void orc_mcsc_product(const double *x, const int32_t *merged_row, const int32_t *merged_off,
                      double *y, int M, int N, int K, int tile_k, int uniformed)
{
    const int T = ceil_div(K, tile_k);
    for (int m = 0; m < M; m++)
        for (int n = 0; n < N; n++) {
            double acc = 0.0;
            for (int t = 0; t < T; t++) {
                const int32_t *o = merged_off + (size_t)n * T * 4 + 4 * t;
                const double *xt = x + (size_t)m * K + (size_t)t * tile_k;
                for (int i = o[0]; i < o[1]; i += 2)
                    acc += xt[merged_row[i]] - xt[merged_row[i + 1]];
                if (uniformed) continue;
                double part = 0.0;
                for (int i = o[1]; i < o[2]; i++) part += xt[merged_row[i]];
                acc += (double)o[3] * part;
            }
            y[(size_t)m * N + n] = acc;
        }
}
