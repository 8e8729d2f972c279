// Host packers: dense ternary matrix -> CSC / tiled CSC / merged tiled CSC.
//
// Outputs are bit-identical to the reference converters
// (ternaryLLM_GPU/csrc/ter_spmm_wrapper.cu:39-78, :92-152, :156-315, :9-27) but the
// work is organised for a row-major input: the matrix is swept row by row (unit
// stride) into per-(column, tile) counters, offsets come from one exclusive scan,
// and a second row-by-row sweep drops each index at its column's cursor.  The
// reference instead walks down every column of the row-major matrix three times.
#include <algorithm>
#include <cstring>
#include <numeric>
#include <vector>

#include "tl_common.h"

namespace tl {

thread_local char g_error[512] = "";

int fail(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

namespace {

struct TileCounts {
    int T = 0;
    std::vector<int32_t> pos;  // [columns][T]
    std::vector<int32_t> neg;
};

int check_dims(const void* w, int columns, int inners)
{
    if (!w) return fail(TL_ERR_ARG, "weight pointer is null");
    if (columns <= 0 || inners <= 0) return fail(TL_ERR_SHAPE, "columns=%d inners=%d must be positive", columns, inners);
    return TL_OK;
}

// One unit-stride sweep: counts of +1 / -1 per (column, tile).
int count_tiles(const int32_t* w, int columns, int inners, int tile_k, TileCounts* out)
{
    const int T = (int)ceil_div(inners, tile_k);
    out->T = T;
    out->pos.assign((size_t)columns * T, 0);
    out->neg.assign((size_t)columns * T, 0);
    for (int k = 0; k < inners; ++k) {
        const int t = k / tile_k;
        const int32_t* row = w + (size_t)k * columns;
        for (int y = 0; y < columns; ++y) {
            const int32_t v = row[y];
            if (v == 1) out->pos[(size_t)y * T + t]++;
            else if (v == -1) out->neg[(size_t)y * T + t]++;
            else if (v != 0) return fail(TL_ERR_VALUE, "weight[%d][%d] = %d is not ternary", k, y, v);
        }
    }
    return TL_OK;
}

}  // namespace
}  // namespace tl

using namespace tl;

extern "C" const char* tl_last_error(void) { return g_error; }
extern "C" int tl_version(void) { return 1; }

extern "C" int tl_count_nnz(const int32_t* w, int columns, int inners, int64_t* cnt_pos, int64_t* cnt_neg)
{
    if (int rc = check_dims(w, columns, inners)) return rc;
    if (!cnt_pos || !cnt_neg) return fail(TL_ERR_ARG, "count outputs are null");
    int64_t p = 0, n = 0;
    const size_t total = (size_t)columns * inners;
    for (size_t i = 0; i < total; ++i) {
        const int32_t v = w[i];
        if (v == 1) ++p;
        else if (v == -1) ++n;
        else if (v != 0) return fail(TL_ERR_VALUE, "weight element %zu = %d is not ternary", i, v);
    }
    *cnt_pos = p;
    *cnt_neg = n;
    return TL_OK;
}

extern "C" int tl_convert_to_ter_csc(const int32_t* w, int columns, int inners, int cnt_pos, int cnt_neg,
                                     int32_t* neg_row, int32_t* neg_off, int32_t* pos_row, int32_t* pos_off)
{
    if (int rc = check_dims(w, columns, inners)) return rc;
    if (!neg_off || !pos_off || (cnt_neg > 0 && !neg_row) || (cnt_pos > 0 && !pos_row))
        return fail(TL_ERR_ARG, "output pointer is null");
    if (cnt_pos < 0 || cnt_neg < 0) return fail(TL_ERR_ARG, "negative non-zero count");
    TileCounts c;
    if (int rc = count_tiles(w, columns, inners, inners, &c)) return rc;  // one tile == whole column
    int64_t p = 0, n = 0;
    for (int y = 0; y < columns; ++y) {
        pos_off[y] = (int32_t)p;
        neg_off[y] = (int32_t)n;
        p += c.pos[y];
        n += c.neg[y];
    }
    if (p != cnt_pos || n != cnt_neg)
        return fail(TL_ERR_VALUE, "counts given (+%d, -%d) differ from the matrix (+%lld, -%lld)", cnt_pos, cnt_neg,
                    (long long)p, (long long)n);
    pos_off[columns] = (int32_t)p;
    neg_off[columns] = (int32_t)n;
    std::vector<int32_t> pc(pos_off, pos_off + columns), nc(neg_off, neg_off + columns);
    for (int k = 0; k < inners; ++k) {
        const int32_t* row = w + (size_t)k * columns;
        for (int y = 0; y < columns; ++y) {
            const int32_t v = row[y];
            if (v == 1) pos_row[pc[y]++] = k;
            else if (v == -1) neg_row[nc[y]++] = k;
        }
    }
    return TL_OK;
}

extern "C" int tl_convert_to_ter_tiled_csc(const int32_t* w, int columns, int inners, int cnt_pos, int cnt_neg,
                                           int tile_k, int32_t* neg_row, int32_t* neg_off_tiled,
                                           int32_t* pos_row, int32_t* pos_off_tiled)
{
    if (int rc = check_dims(w, columns, inners)) return rc;
    if (tile_k <= 0) return fail(TL_ERR_ARG, "tile_k=%d must be positive", tile_k);
    if (!neg_off_tiled || !pos_off_tiled || (cnt_neg > 0 && !neg_row) || (cnt_pos > 0 && !pos_row))
        return fail(TL_ERR_ARG, "output pointer is null");
    TileCounts c;
    if (int rc = count_tiles(w, columns, inners, tile_k, &c)) return rc;
    const int T = c.T;
    const size_t cells = (size_t)columns * T;
    // [start, end) per cell: exclusive scan over cells in (column, tile) order.
    std::vector<int32_t> pcur(cells), ncur(cells);
    int64_t p = 0, n = 0;
    for (size_t i = 0; i < cells; ++i) {
        pcur[i] = (int32_t)p;
        ncur[i] = (int32_t)n;
        pos_off_tiled[2 * i] = (int32_t)p;
        neg_off_tiled[2 * i] = (int32_t)n;
        p += c.pos[i];
        n += c.neg[i];
        pos_off_tiled[2 * i + 1] = (int32_t)p;
        neg_off_tiled[2 * i + 1] = (int32_t)n;
    }
    if (p != cnt_pos || n != cnt_neg)
        return fail(TL_ERR_VALUE, "counts given (+%d, -%d) differ from the matrix (+%lld, -%lld)", cnt_pos, cnt_neg,
                    (long long)p, (long long)n);
    for (int k = 0; k < inners; ++k) {
        const int t = k / tile_k;
        const int32_t local = k - t * tile_k;
        const int32_t* row = w + (size_t)k * columns;
        for (int y = 0; y < columns; ++y) {
            const int32_t v = row[y];
            if (v == 1) pos_row[pcur[(size_t)y * T + t]++] = local;
            else if (v == -1) neg_row[ncur[(size_t)y * T + t]++] = local;
        }
    }
    return TL_OK;
}

namespace {

struct MergePlan {
    int pairs, pairs_pad, rest, rest_pad, kept_pairs, kept_rest;
    bool neg_is_min;
};

// Sizes of one merged tile.  kept_* are the counts the offsets advertise after the
// reference's alignment rule (ter_spmm_wrapper.cu:277-291): the leftover count is
// made even, then the pair-entry count and the leftover count are each lowered
// by 2 when they are not multiples of 4.
inline MergePlan plan_tile(int pos, int neg, bool padding, int padding_size)
{
    MergePlan m;
    m.neg_is_min = neg <= pos;
    const int mn = m.neg_is_min ? neg : pos;
    const int mx = m.neg_is_min ? pos : neg;
    m.pairs = 2 * mn;
    m.rest = mx - mn;
    m.pairs_pad = padding ? (int)round_up(m.pairs, padding_size) : m.pairs;
    m.rest_pad = padding ? (int)round_up(m.rest, padding_size) : m.rest;
    m.kept_rest = m.rest & ~1;
    m.kept_pairs = m.pairs;
    if (m.kept_pairs % 4 != 0) m.kept_pairs -= 2;
    if (m.kept_rest % 4 != 0) m.kept_rest -= 2;
    return m;
}

}  // namespace

extern "C" int tl_tiled_mcsc_size(const int32_t* w, int columns, int inners, int cnt_pos, int cnt_neg,
                                  int tile_k, int padding, int padding_size, int64_t* n_index)
{
    if (int rc = check_dims(w, columns, inners)) return rc;
    if (!n_index) return fail(TL_ERR_ARG, "n_index is null");
    if (tile_k <= 0) return fail(TL_ERR_ARG, "tile_k=%d must be positive", tile_k);
    if (!padding) {
        *n_index = (int64_t)cnt_pos + cnt_neg;
        return TL_OK;
    }
    if (padding_size <= 0) return fail(TL_ERR_ARG, "padding_size=%d must be positive", padding_size);
    TileCounts c;
    if (int rc = count_tiles(w, columns, inners, tile_k, &c)) return rc;
    int64_t total = 0;
    for (size_t i = 0; i < c.pos.size(); ++i) {
        MergePlan m = plan_tile(c.pos[i], c.neg[i], true, padding_size);
        total += m.pairs_pad + m.rest_pad;
    }
    *n_index = total;
    return TL_OK;
}

extern "C" int tl_convert_to_ter_tiled_mcsc(const int32_t* w, int columns, int inners, int cnt_pos, int cnt_neg,
                                            int tile_k, int padding, int padding_size,
                                            int32_t* merged_row, int64_t n_index,
                                            int32_t* merged_off, int32_t* col_tile_idx)
{
    if (int rc = check_dims(w, columns, inners)) return rc;
    if (!merged_off || !col_tile_idx || (n_index > 0 && !merged_row)) return fail(TL_ERR_ARG, "output pointer is null");
    if (padding && padding_size <= 0) return fail(TL_ERR_ARG, "padding_size=%d must be positive", padding_size);
    int64_t need = 0;
    if (int rc = tl_tiled_mcsc_size(w, columns, inners, cnt_pos, cnt_neg, tile_k, padding, padding_size, &need)) return rc;
    if (n_index != need)
        return fail(TL_ERR_SIZE, "merged index array has %lld entries, the format needs %lld", (long long)n_index,
                    (long long)need);

    const int T = (int)ceil_div(inners, tile_k);
    const size_t cells = (size_t)columns * T;
    std::vector<int32_t> neg_row((size_t)cnt_neg + 1), pos_row((size_t)cnt_pos + 1);
    std::vector<int32_t> neg_off(cells * 2), pos_off(cells * 2);
    if (int rc = tl_convert_to_ter_tiled_csc(w, columns, inners, cnt_pos, cnt_neg, tile_k, neg_row.data(),
                                             neg_off.data(), pos_row.data(), pos_off.data()))
        return rc;

    std::memset(merged_row, 0, sizeof(int32_t) * (size_t)n_index);
    int64_t cursor = 0;
    for (size_t cell = 0; cell < cells; ++cell) {
        const int32_t* P = pos_row.data() + pos_off[2 * cell];
        const int32_t* Q = neg_row.data() + neg_off[2 * cell];
        const int pos = pos_off[2 * cell + 1] - pos_off[2 * cell];
        const int neg = neg_off[2 * cell + 1] - neg_off[2 * cell];
        const MergePlan m = plan_tile(pos, neg, padding != 0, padding_size);
        int32_t* out = merged_row + cursor;
        const int mn = m.pairs / 2;
        for (int k = 0; k < mn; ++k) {
            out[2 * k] = P[k];
            out[2 * k + 1] = Q[k];
        }
        // Padding slots repeat the tile's first +1 row; the leftovers are written
        // after them and start right behind the real pairs, so they overwrite
        // padding slots where the two ranges overlap.
        for (int k = m.pairs; k < m.pairs_pad; ++k) out[k] = P[0];
        const int32_t* L = (m.neg_is_min ? P : Q) + mn;
        for (int k = 0; k < m.rest; ++k) out[m.pairs + k] = L[k];

        int32_t* o = merged_off + 4 * cell;
        o[0] = (int32_t)cursor;
        o[1] = (int32_t)(cursor + (padding ? m.pairs_pad : m.kept_pairs));
        o[2] = o[1] + m.kept_rest;
        o[3] = m.neg_is_min ? 1 : -1;
        cursor += padding ? (m.pairs_pad + m.rest_pad) : (m.kept_pairs + m.kept_rest);
    }

    // Per column: tile ids by ascending stored length (ter_spmm_wrapper.cu:9-27).
    // std::sort, like the reference, so equal lengths fall the same way under libstdc++.
    std::vector<int> order(T);
    for (int y = 0; y < columns; ++y) {
        const int32_t* o = merged_off + (size_t)y * T * 4;
        std::iota(order.begin(), order.end(), 0);
        std::sort(order.begin(), order.end(),
                  [o](int a, int b) { return (o[4 * a + 2] - o[4 * a]) < (o[4 * b + 2] - o[4 * b]); });
        std::copy(order.begin(), order.end(), col_tile_idx + (size_t)y * T);
    }
    return TL_OK;
}

extern "C" int tl_tiled_mcsc_to_dense(const void* merged_row, int index_width, int64_t n_index,
                                      const int32_t* merged_off, int columns, int inners, int tile_k,
                                      int32_t* w_out)
{
    if (!merged_off || !w_out || (n_index > 0 && !merged_row)) return fail(TL_ERR_ARG, "null pointer");
    if (columns <= 0 || inners <= 0 || tile_k <= 0) return fail(TL_ERR_SHAPE, "bad dimensions");
    if (index_width != 2 && index_width != 4) return fail(TL_ERR_DTYPE, "index_width=%d (2 or 4 expected)", index_width);
    const int T = (int)ceil_div(inners, tile_k);
    const int16_t* r16 = static_cast<const int16_t*>(merged_row);
    const int32_t* r32 = static_cast<const int32_t*>(merged_row);
    auto at = [&](int64_t i) -> int32_t { return index_width == 2 ? (int32_t)r16[i] : r32[i]; };
    std::memset(w_out, 0, sizeof(int32_t) * (size_t)columns * inners);
    for (int y = 0; y < columns; ++y)
        for (int t = 0; t < T; ++t) {
            const int32_t* o = merged_off + ((size_t)y * T + t) * 4;
            if (o[0] < 0 || o[1] < o[0] || o[2] < o[1] || o[2] > n_index || ((o[1] - o[0]) & 1) || (o[3] != 1 && o[3] != -1))
                return fail(TL_ERR_FORMAT, "column %d tile %d: offsets [%d,%d,%d,%d] are not a merged tile", y, t, o[0],
                            o[1], o[2], o[3]);
            for (int64_t i = o[0]; i < o[2]; ++i) {
                const int64_t row = (int64_t)t * tile_k + at(i);
                if (at(i) < 0 || at(i) >= tile_k || row >= inners)
                    return fail(TL_ERR_FORMAT, "column %d tile %d: row index %d out of range", y, t, at(i));
                int32_t s;
                if (i < o[1]) s = ((i - o[0]) & 1) ? -1 : 1;
                else s = o[3];
                w_out[(size_t)row * columns + y] += s;
            }
        }
    const size_t total = (size_t)columns * inners;
    for (size_t i = 0; i < total; ++i)
        if (w_out[i] < -1 || w_out[i] > 1)
            return fail(TL_ERR_VALUE, "decoded weight element %zu = %d is not ternary", i, w_out[i]);
    return TL_OK;
}
