// Builder / validator / decoder of the device weight format ("wave-tiled CSC").
//
// Input is the lossless tiled CSC of the reference API
// (ternaryLLM_GPU/csrc/ter_spmm_wrapper.cu:92-152: separate +1 / -1 row lists with
// tile-local indices and [start, end) offsets per (column, tile)).  The device
// format keeps the two separate streams but
//   - re-tiles K into tiles of at most 255 rows so that an index is one byte and
//     byte value 255 can act as a padding sentinel;
//   - pads every run to whole dwords so that a lane (or a broadcast word) always
//     carries four indices;
//   - groups columns in blocks of 16 and stores, block-major, one self-describing chunk per
//     (block, tile): 16 descriptors followed by the block's runs.  What a workgroup needs
//     for a range of tiles is then a single contiguous piece of memory.
#include <climits>
#include <cmath>
#include <cstring>
#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <thread>
#include <vector>

#include "tl_common.h"

using namespace tl;

namespace {

constexpr int kBlock = TL_BLOCK_COLUMNS;

struct Geometry {
    int tile_rows, n_tiles, n_blocks;
};

int pick_geometry(int columns, int inners, int tile_rows, Geometry* g)
{
    if (tile_rows < 0 || tile_rows > kMaxTileRows)
        return fail(TL_ERR_ARG, "tile_rows=%d must be in [1, %d] (0 = default)", tile_rows, kMaxTileRows);
    if (tile_rows == 0) {
        // the largest balanced height that is a multiple of 8: a tile's rows then start on a 16-byte
        // boundary of an fp16 (or fp32) activation row, which the decode kernel copies as whole vectors
        const int t = (int)ceil_div(inners, 248);
        tile_rows = std::min<int>(248, (int)round_up(ceil_div(inners, t), 8));
    }
    g->tile_rows = tile_rows;
    g->n_tiles = (int)ceil_div(inners, tile_rows);
    g->n_blocks = (int)ceil_div(columns, kBlock);
    return TL_OK;
}

// What kernels may read past the end of the stream: 192 dwords from the start of a wave's piece
// (the piece may be empty and start at the stream's last dword) or 63 dwords past a piece's end.
constexpr int kSparePrefetchDwords = 192;
constexpr int64_t kStreamSpareBytes = 1024;
static_assert(kStreamSpareBytes >= kSparePrefetchDwords * 4, "the spare must cover the index prefetch");

struct Sections {
    int64_t off_chunkstart, off_stream, total;
};

Sections place_sections(const Geometry& g, int64_t stream_bytes)
{
    Sections s;
    s.off_chunkstart = 256;
    s.off_stream = s.off_chunkstart + round_up(((int64_t)g.n_tiles * g.n_blocks + 1) * 4, 256);
    // Spare bytes behind the stream: the row kernel requests a wave's first kSparePrefetchDwords index
    // dwords from wherever its piece starts, also when the piece is the stream's last and shorter.
    s.total = s.off_stream + round_up(stream_bytes, 256) + kStreamSpareBytes;
    return s;
}

int64_t stream_upper_bound(int64_t nnz, int columns, const Geometry& g)
{
    // per (column, tile): two runs that each round up by at most 3 bytes; per chunk:
    // one descriptor dword per column of the block and up to 12 bytes of padding
    return round_up(nnz + (int64_t)6 * columns * g.n_tiles + (int64_t)g.n_tiles * g.n_blocks * (kBlock * 4 + 12), 16);
}

// Per (device tile, column) counts from the tiled-CSC offsets and local rows.
int count_device_tiles(const int32_t* row, const int32_t* off_tiled, int columns, int inners, int tile_k,
                       const Geometry& g, std::vector<uint16_t>* counts)
{
    const int Ta = (int)ceil_div(inners, tile_k);
    counts->assign((size_t)columns * g.n_tiles, 0);
    for (int y = 0; y < columns; ++y)
        for (int t = 0; t < Ta; ++t) {
            const int32_t b = off_tiled[((size_t)y * Ta + t) * 2], e = off_tiled[((size_t)y * Ta + t) * 2 + 1];
            if (b < 0 || e < b) return fail(TL_ERR_FORMAT, "column %d tile %d: offsets [%d, %d) are not ordered", y, t, b, e);
            for (int32_t i = b; i < e; ++i) {
                const int64_t k = (int64_t)t * tile_k + row[i];
                if (row[i] < 0 || row[i] >= tile_k || k >= inners)
                    return fail(TL_ERR_FORMAT, "column %d tile %d: local row %d out of range", y, t, row[i]);
                uint16_t& c = (*counts)[(size_t)(k / g.tile_rows) * columns + y];
                if (c == 0xffffu) return fail(TL_ERR_UNSUPPORTED, "column %d: more than 65535 entries in one tile", y);
                ++c;
            }
        }
    return TL_OK;
}

// Order of the rows inside runs.  The sum does not depend on it; the single-row kernel's speed does: a lane
// reads one activation per index from the LDS image of its tile, and the LDS serves half a wave, 32 lanes, at a
// time: reads of those 32 that fall on one LDS bank (of 32, four bytes wide) but on different words are served
// one after the other.  The plain single-row kernel (tl_spmv_tiles) gives a wave a whole tile: 16 columns, four
// lanes to a run (lane l on dwords l, l + 4, ... of the +1 run followed by the -1 run), lanes 0-31 on columns
// 0-7 of the block; all lanes read byte b of their k-th dword together.  So the rows of a group of 8
// neighbouring columns of a tile (32 lanes) are dealt out read by read: each lane takes from what is left of its
// run the row whose bank the read has used least so far (the padding bytes, which read the tile's zero slot, are
// counted first); then rows are swapped between the reads of a run while that lowers the number of lanes
// that share a bank.  tl_spmv_direct assigns its lanes the same way; kernels with another assignment (more
// lanes per run for long runs, the 8- and 16-row kernels) find an order that is no better than any other, and
// no worse.
struct RunRef {
    uint8_t* bytes;  // start of the +1 run (the -1 run follows its padded end)
    int n_pos, n_neg;
    int tile;
};

constexpr int kLanesPerRun = 4;
constexpr int kWeight16 = 4;  // a shared class of the 16-row kernel against a shared bank of the single-row kernel, in the deal
constexpr int kSpreadSweeps = 2;

// LDS bank of a row's activation in the single-row kernel: fp16 values, two to a bank word; the image of
// tile t starts kSpmvImageSkew bytes further round the banks than that of tile t - 1 (tl_common.h).
inline int bank_of(uint8_t row, int tile) { return ((row >> 1) + tile * (kSpmvImageSkew / 4)) & 31; }

void spread_over_banks(const RunRef* runs, int n_runs, int sweeps, int tile_rows)
{
    // read q = pass * 4 + byte; run r, lane l holds dword pass * 4 + l of the combined run
    int longest = 0;
    for (int r = 0; r < n_runs; ++r) longest = std::max(longest, (runs[r].n_pos + 3) / 4 + (runs[r].n_neg + 3) / 4);
    if (longest == 0) return;
    const int passes = (longest + kLanesPerRun - 1) / kLanesPerRun, reads = passes * 4;
    std::vector<int> load((size_t)reads * 32, 0);
    // 16-row kernel: at position e of the runs of one sign, the rows of the group's columns should differ modulo 8
    std::vector<uint8_t> load16((size_t)2 * 256 * 8, 0);
    std::vector<uint8_t> pool[2];
    {
        // Behind the end of its run a lane of the 16-row kernel gathers from a zero slot: slot 248 + (column % 8) when
        // the tile leaves all of 248 .. 255 free, else slot 255; the other columns' rows at those positions keep
        // out of that class.
        int longest16[2] = {0, 0};
        for (int r = 0; r < n_runs; ++r) {
            longest16[0] = std::max(longest16[0], (runs[r].n_pos + 3) / 4 * 4);
            longest16[1] = std::max(longest16[1], (runs[r].n_neg + 3) / 4 * 4);
        }
        for (int r = 0; r < n_runs; ++r)
            for (int sign = 0; sign < 2; ++sign) {
                const int n = sign ? runs[r].n_neg : runs[r].n_pos;
                const int zero_class = tile_rows <= kMaxTileRows - 7 ? (r & 7) : (kSentinel & 7);
                for (int e = (n + 3) / 4 * 4; e < longest16[sign]; ++e) ++load16[((size_t)sign * 256 + e) * 8 + zero_class];
            }
    }
    auto position = [&](const RunRef& run, int q, int l, bool* neg, int* e) {
        const int pd = (run.n_pos + 3) / 4;
        const int i = (q >> 2) * kLanesPerRun + l;
        *neg = i >= pd;
        *e = 4 * (*neg ? i - pd : i) + (q & 3);
        return *e < (*neg ? run.n_neg : run.n_pos);
    };
    for (int r = 0; r < n_runs; ++r) {
        const RunRef& run = runs[r];
        const int pd = (run.n_pos + 3) / 4;
        pool[0].assign(run.bytes, run.bytes + run.n_pos);
        pool[1].assign(run.bytes + 4 * pd, run.bytes + 4 * pd + run.n_neg);
        // the padding bytes of the two last dwords read the tile's zero slot: loads that are there whatever the order
        for (int sign = 0; sign < 2; ++sign) {
            const int n = sign ? run.n_neg : run.n_pos;
            for (int e = n; e < (n + 3) / 4 * 4; ++e) {
                ++load[(size_t)((((sign ? pd : 0) + e / 4) / kLanesPerRun) * 4 + (e & 3)) * 32 + bank_of(kSentinel, run.tile)];
                ++load16[((size_t)sign * 256 + e) * 8 + (kSentinel & 7)];
            }
        }
        for (int q = 0; q < reads; ++q)
            for (int l = 0; l < kLanesPerRun; ++l) {
                bool neg;
                int e;
                if (!position(run, q, l, &neg, &e)) continue;
                std::vector<uint8_t>& left = pool[neg ? 1 : 0];
                const int* ld = &load[(size_t)q * 32];
                uint8_t* l16 = &load16[((size_t)(neg ? 1 : 0) * 256 + e) * 8];
                auto key = [&](uint8_t row) { return (kWeight16 * l16[row & 7] + ld[bank_of(row, run.tile)]) * 256 + row; };
                size_t best = 0;
                int best_key = key(left[0]);
                for (size_t c = 1; c < left.size(); ++c) {
                    const int k = key(left[c]);
                    if (k < best_key) { best = c; best_key = k; }
                }
                const uint8_t row = left[best];
                left[best] = left.back();
                left.pop_back();
                ++load[(size_t)q * 32 + bank_of(row, run.tile)];
                ++l16[row & 7];
                run.bytes[(neg ? 4 * pd : 0) + e] = row;
            }
    }
    // Swaps inside a run, between two of its reads.  What a read costs is the largest number of different words that
    // any one bank has to deliver (lanes on the same word are served together), so a read with one shared bank
    // costs as much as a read with five: the swaps move shared banks out of the reads that have few of them and
    // into reads that have some already.  Potential of a read: sqrt(banks with two words or more) + 10 * (words
    // beyond two on a bank).
    struct ReadState {
        uint8_t words[128];  // lanes per word of the tile image (two fp16 rows to a word)
        uint8_t per_bank[32];
        int two, three;      // banks that deliver two or more different words; words beyond two, summed over the banks
    };
    std::vector<ReadState> state((size_t)reads);
    std::memset(state.data(), 0, state.size() * sizeof(ReadState));
    auto add = [&](int q, int word, int tile) {
        ReadState& s = state[(size_t)q];
        if (s.words[word]++ == 0) {
            const int n = ++s.per_bank[bank_of((uint8_t)(word * 2), tile)];
            s.two += n == 2;
            s.three += n >= 3;
        }
    };
    auto drop = [&](int q, int word, int tile) {
        ReadState& s = state[(size_t)q];
        if (--s.words[word] == 0) {
            const int n = s.per_bank[bank_of((uint8_t)(word * 2), tile)]--;
            s.two -= n == 2;
            s.three -= n >= 3;
        }
    };
    float root[33];
    for (int i = 0; i <= 32; ++i) root[i] = std::sqrt((float)i);
    auto potential = [&](int q) { return root[state[(size_t)q].two] + 10.0f * (float)state[(size_t)q].three; };
    for (int r = 0; r < n_runs; ++r) {
        const RunRef& run = runs[r];
        const int pd = (run.n_pos + 3) / 4, nd = (run.n_neg + 3) / 4;
        for (int e = 0; e < 4 * (pd + nd); ++e) add(((e / 4) / kLanesPerRun) * 4 + (e & 3), run.bytes[e] >> 1, run.tile);
    }
    // The 16-row kernel's side of a swap: what the positions e1 and e2 of one sign cost it before and after their rows
    // (classes c1, c2) change places.  A position costs the largest number of the group's rows in one class (its LDS
    // cycles), plus a little for every row beyond the first in a class.
    auto cost16 = [&](const uint8_t* cnt) {
        int most = 0, extra = 0;
        for (int c = 0; c < 8; ++c) {
            most = std::max(most, (int)cnt[c]);
            extra += cnt[c] > 1 ? cnt[c] - 1 : 0;
        }
        return (float)most + 0.25f * (float)extra;
    };
    auto swap16 = [&](int sign, int e1, int e2, int c1, int c2, bool apply) {
        if (c1 == c2) return 0.0f;
        uint8_t* a = &load16[((size_t)sign * 256 + e1) * 8];
        uint8_t* b = &load16[((size_t)sign * 256 + e2) * 8];
        const float before = cost16(a) + cost16(b);
        --a[c1]; ++a[c2]; --b[c2]; ++b[c1];
        const float after = cost16(a) + cost16(b);
        if (!apply) { ++a[c1]; --a[c2]; ++b[c2]; --b[c1]; }
        return before - after;  // what the swap gains
    };
    for (int sweep = 0; sweep < sweeps; ++sweep) {
        bool any = false;
        for (int r = 0; r < n_runs; ++r) {
            const RunRef& run = runs[r];
            const int pd = (run.n_pos + 3) / 4, tile = run.tile;
            for (int sign = 0; sign < 2; ++sign) {
                uint8_t* rows = run.bytes + (sign ? 4 * pd : 0);
                const int n = sign ? run.n_neg : run.n_pos;
                const int first_dword = sign ? pd : 0;
                auto read_of = [&](int e) { return ((first_dword + e / 4) / kLanesPerRun) * 4 + (e & 3); };
                for (int e1 = 0; e1 < n; ++e1) {
                    const int q1 = read_of(e1), w1 = rows[e1] >> 1, b1 = bank_of(rows[e1], tile), c1 = rows[e1] & 7;
                    // a row is worth moving when it is alone on its word, on a bank that delivers another word too
                    // (single-row kernel), or shares its class with a row of another column (16-row kernel)
                    const bool shared1 = state[(size_t)q1].words[w1] == 1 && state[(size_t)q1].per_bank[b1] >= 2;
                    const bool shared16 = load16[((size_t)sign * 256 + e1) * 8 + c1] >= 2;
                    if (!shared1 && !shared16) continue;
                    int best = -1;
                    float best_gain = 1e-6f;
                    for (int e2 = 0; e2 < n; ++e2) {
                        if (e2 == e1) continue;
                        const int q2 = read_of(e2), w2 = rows[e2] >> 1, c2 = rows[e2] & 7;
                        float gain = (float)kWeight16 * swap16(sign, e1, e2, c1, c2, false);
                        if (q2 != q1) {  // (inside one read of the single-row kernel nothing changes for it)
                            if (!shared1 && gain <= 0.f) continue;
                            const float before = potential(q1) + potential(q2);
                            drop(q1, w1, tile); add(q1, w2, tile); drop(q2, w2, tile); add(q2, w1, tile);
                            gain += before - potential(q1) - potential(q2);
                            drop(q2, w1, tile); add(q2, w2, tile); drop(q1, w2, tile); add(q1, w1, tile);
                        }
                        if (gain > best_gain) { best_gain = gain; best = e2; }
                    }
                    if (best >= 0) {
                        const int q2 = read_of(best), w2 = rows[best] >> 1;
                        if (q2 != q1) { drop(q1, w1, tile); add(q1, w2, tile); drop(q2, w2, tile); add(q2, w1, tile); }
                        swap16(sign, e1, best, c1, rows[best] & 7, true);
                        std::swap(rows[e1], rows[best]);
                        any = true;
                    }
                }
            }
        }
        if (!any) break;
    }
}

// FNV-1a, 64-bit, one step per dword, over the chunk table (with its end entry) and the stream.
uint64_t content_checksum(const uint32_t* chunkstart, size_t n_table, const uint32_t* stream, size_t n_stream)
{
    uint64_t h = 0xcbf29ce484222325ull;
    for (size_t i = 0; i < n_table; ++i) h = (h ^ chunkstart[i]) * 0x100000001b3ull;
    for (size_t i = 0; i < n_stream; ++i) h = (h ^ stream[i]) * 0x100000001b3ull;
    return h;
}

// Threads for the row-ordering pass of one tl_layout_build call: TL_PACK_THREADS if set, else the machine's hardware
// threads up to 8, shared among the calls that are in that pass at the moment (callers that pack many weights on
// threads of their own then get one each).  The caller gives its count back when its pass is over.
std::atomic<int> g_builds_running{0};

int pack_workers(int n_blocks)
{
    int cap = 0;
    if (const char* e = std::getenv("TL_PACK_THREADS")) cap = std::atoi(e);
    if (cap <= 0) cap = (int)std::min(8u, std::max(1u, std::thread::hardware_concurrency()));
    const int running = g_builds_running.fetch_add(1) + 1;
    return std::max(1, std::min(cap / running, n_blocks));
}

// Last "end" entry of a tiled-CSC offset array = number of stored rows of that sign.
int64_t stream_length(const int32_t* off_tiled, int columns, int inners, int tile_k)
{
    const int Ta = (int)ceil_div(inners, tile_k);
    return off_tiled[((size_t)columns * Ta - 1) * 2 + 1];
}

}  // namespace

extern "C" int tl_layout_size(const int32_t* neg_off_tiled, const int32_t* pos_off_tiled,
                              int columns, int inners, int tile_k, int tile_rows, int64_t* blob_bytes)
{
    if (!neg_off_tiled || !pos_off_tiled || !blob_bytes) return fail(TL_ERR_ARG, "null pointer");
    if (columns <= 0 || inners <= 0 || tile_k <= 0) return fail(TL_ERR_SHAPE, "bad dimensions");
    Geometry g;
    if (int rc = pick_geometry(columns, inners, tile_rows, &g)) return rc;
    const int64_t nnz = stream_length(neg_off_tiled, columns, inners, tile_k) + stream_length(pos_off_tiled, columns, inners, tile_k);
    *blob_bytes = place_sections(g, stream_upper_bound(nnz, columns, g)).total;
    return TL_OK;
}

extern "C" int tl_layout_build(const int32_t* neg_row, const int32_t* neg_off_tiled,
                               const int32_t* pos_row, const int32_t* pos_off_tiled,
                               int columns, int inners, int tile_k, int tile_rows,
                               void* blob, int64_t blob_bytes)
{
    if (!neg_off_tiled || !pos_off_tiled || !blob) return fail(TL_ERR_ARG, "null pointer");
    if (columns <= 0 || inners <= 0 || tile_k <= 0) return fail(TL_ERR_SHAPE, "bad dimensions");
    Geometry g;
    if (int rc = pick_geometry(columns, inners, tile_rows, &g)) return rc;
    int64_t budget = 0;
    if (int rc = tl_layout_size(neg_off_tiled, pos_off_tiled, columns, inners, tile_k, tile_rows, &budget)) return rc;
    if (blob_bytes < budget) return fail(TL_ERR_SIZE, "blob has %lld bytes, %lld needed", (long long)blob_bytes, (long long)budget);
    const int64_t n_pos = stream_length(pos_off_tiled, columns, inners, tile_k);
    const int64_t n_neg = stream_length(neg_off_tiled, columns, inners, tile_k);
    if ((n_pos > 0 && !pos_row) || (n_neg > 0 && !neg_row)) return fail(TL_ERR_ARG, "row array is null");

    std::vector<uint16_t> cp, cn;  // [tile][column]
    if (int rc = count_device_tiles(pos_row, pos_off_tiled, columns, inners, tile_k, g, &cp)) return rc;
    if (int rc = count_device_tiles(neg_row, neg_off_tiled, columns, inners, tile_k, g, &cn)) return rc;

    const int T = g.n_tiles, NB = g.n_blocks;
    const int Ta = (int)ceil_div(inners, tile_k);
    const int64_t reserve = stream_upper_bound(n_pos + n_neg, columns, g);
    const Sections s = place_sections(g, reserve);
    std::memset(blob, 0, (size_t)blob_bytes);
    uint8_t* base = static_cast<uint8_t*>(blob);
    uint32_t* chunkstart = reinterpret_cast<uint32_t*>(base + s.off_chunkstart);
    uint32_t* stream = reinterpret_cast<uint32_t*>(base + s.off_stream);

    // Pass 1: chunk starts and descriptors, block-major.
    uint64_t dwords = 0, run_sum = 0;
    uint32_t run_max = 0, chunk_max = 0;
    for (int nb = 0; nb < NB; ++nb)
        for (int t = 0; t < T; ++t) {
            chunkstart[(size_t)nb * T + t] = (uint32_t)dwords;
            if (dwords > 0xffffffffull - 16384) return fail(TL_ERR_UNSUPPORTED, "index stream does not fit 32-bit dword offsets");
            uint32_t* desc = stream + dwords;
            uint32_t in_chunk = kBlock;  // runs start behind the descriptors
            for (int j = 0; j < kBlock; ++j) {
                const int y = nb * kBlock + j;
                uint32_t p = 0, n = 0;
                if (y < columns) {
                    p = cp[(size_t)t * columns + y];
                    n = cn[(size_t)t * columns + y];
                }
                if (p > 255 || n > 255)
                    return fail(TL_ERR_UNSUPPORTED, "column %d tile %d names %u/%u rows of one sign (255 at most)", y, t, p, n);
                if ((dwords + j) * 4 >= (uint64_t)reserve) return fail(TL_ERR_SIZE, "stream reserve exceeded");
                desc[j] = make_desc(p, n, in_chunk);
                const uint32_t run = (p + 3) / 4 + (n + 3) / 4;
                in_chunk += run;  // at most 16 + 16 * 128 dwords: always fits 16 bits
                if (y < columns) {
                    run_sum += run;
                    if (run > run_max) run_max = run;
                }
            }
            in_chunk = (uint32_t)round_up(in_chunk, 4);
            if (in_chunk > chunk_max) chunk_max = in_chunk;
            dwords += in_chunk;
            if (dwords * 4 > (uint64_t)reserve) return fail(TL_ERR_SIZE, "stream reserve exceeded");
        }
    chunkstart[(size_t)NB * T] = (uint32_t)dwords;

    // Pass 2: sentinel-fill the runs, then scatter the rows.  Rows arrive ascending per
    // column, so one cursor per (device tile, sign) of the current column fills every run in order.
    for (int nb = 0; nb < NB; ++nb)
        for (int t = 0; t < T; ++t) {
            const uint64_t c0 = chunkstart[(size_t)nb * T + t], c1 = chunkstart[(size_t)nb * T + t + 1];
            std::memset(stream + c0 + kBlock, kSentinel, (size_t)(c1 - c0 - kBlock) * 4);
        }
    std::vector<uint64_t> cursor((size_t)T * 2);
    uint8_t* bytes = reinterpret_cast<uint8_t*>(stream);
    for (int y = 0; y < columns; ++y) {
        const int nb = y / kBlock, j = y % kBlock;
        for (int t = 0; t < T; ++t) {
            const uint64_t c0 = chunkstart[(size_t)nb * T + t];
            const uint32_t d = stream[c0 + j];
            const uint64_t start = (c0 + (d >> 16)) * 4;
            cursor[2 * t] = start;
            cursor[2 * t + 1] = start + (((d & 0xff) + 3) / 4) * 4;
        }
        for (int sign = 0; sign < 2; ++sign) {
            const int32_t* row = sign == 0 ? pos_row : neg_row;
            const int32_t* off = sign == 0 ? pos_off_tiled : neg_off_tiled;
            for (int t = 0; t < Ta; ++t)
                for (int32_t i = off[((size_t)y * Ta + t) * 2]; i < off[((size_t)y * Ta + t) * 2 + 1]; ++i) {
                    const int k = t * tile_k + row[i];
                    bytes[cursor[2 * (k / g.tile_rows) + sign]++] = (uint8_t)(k % g.tile_rows);
                }
        }
    }

    // Pass 3: order the rows inside every group of 8 neighbouring columns of a tile (the single-row kernel puts 32
    // lanes, half a wave, on them: four per column, and the LDS serves half a wave at a time).  Blocks are
    // independent of each other and the order found depends on the block alone, so worker threads take blocks in
    // turn: the blob does not depend on how many there are.
    auto order_block = [&](int nb) {
        RunRef runs[8];
        const int cols = std::min(kBlock, columns - nb * kBlock);
        for (int t = 0; t < T; ++t) {
            const uint64_t c0 = chunkstart[(size_t)nb * T + t];
            for (int j0 = 0; j0 < cols; j0 += 8) {
                const int gsz = std::min(8, cols - j0);
                for (int i = 0; i < gsz; ++i) {
                    const uint32_t d = stream[c0 + j0 + i];
                    runs[i] = RunRef{bytes + (c0 + (d >> 16)) * 4, (int)(d & 0xff), (int)((d >> 8) & 0xff), t};
                }
                spread_over_banks(runs, gsz, kSpreadSweeps, g.tile_rows);
            }
        }
    };
    {
        const int workers = pack_workers(NB);
        std::atomic<int> next{0};
        auto work = [&]() {
            for (int nb = next.fetch_add(1); nb < NB; nb = next.fetch_add(1)) order_block(nb);
        };
        std::vector<std::thread> pool;
        for (int i = 1; i < workers; ++i) pool.emplace_back(work);
        work();
        for (auto& th : pool) th.join();
        g_builds_running.fetch_sub(1);
    }

    tl_layout_header h;
    std::memset(&h, 0, sizeof(h));
    static_assert(sizeof(tl_layout_header) == 256, "header must stay 256 bytes");
    h.magic = TL_LAYOUT_MAGIC;
    h.version = TL_LAYOUT_VERSION;
    h.inners = (uint32_t)inners;
    h.columns = (uint32_t)columns;
    h.tile_rows = (uint32_t)g.tile_rows;
    h.n_tiles = (uint32_t)T;
    h.n_blocks = (uint32_t)NB;
    h.max_chunk_dwords = chunk_max;
    h.nnz_pos = (uint64_t)n_pos;
    h.nnz_neg = (uint64_t)n_neg;
    h.off_chunkstart = (uint64_t)s.off_chunkstart;
    h.off_stream = (uint64_t)s.off_stream;
    h.stream_bytes = dwords * 4;
    // The blob handed in is sized by an upper bound; what the format occupies is smaller.
    h.total_bytes = (uint64_t)place_sections(g, (int64_t)dwords * 4).total;
    h.max_run_dwords = run_max;
    h.mean_run_dwords_x16 = (uint32_t)ceil_div((int64_t)run_sum * 16, (int64_t)columns * T);
    h.checksum = content_checksum(chunkstart, (size_t)NB * T + 1, stream, (size_t)dwords);
    std::memcpy(blob, &h, sizeof(h));
    return TL_OK;
}

extern "C" int tl_layout_from_dense(const int32_t* w, int columns, int inners, int tile_rows,
                                    void* blob, int64_t* blob_bytes)
{
    if (!w || !blob_bytes) return fail(TL_ERR_ARG, "null pointer");
    if (columns <= 0 || inners <= 0) return fail(TL_ERR_SHAPE, "bad dimensions");
    int64_t p = 0, n = 0;
    if (int rc = tl_count_nnz(w, columns, inners, &p, &n)) return rc;
    if (p > INT32_MAX || n > INT32_MAX) return fail(TL_ERR_UNSUPPORTED, "more than 2^31 non-zeros of one sign");
    Geometry g;
    if (int rc = pick_geometry(columns, inners, tile_rows, &g)) return rc;
    // Pack with the device tile height directly: the API-level tiles then coincide with device tiles.
    const int T = g.n_tiles;
    std::vector<int32_t> neg_row((size_t)n + 1), pos_row((size_t)p + 1), neg_off((size_t)columns * T * 2),
        pos_off((size_t)columns * T * 2);
    if (int rc = tl_convert_to_ter_tiled_csc(w, columns, inners, (int)p, (int)n, g.tile_rows, neg_row.data(),
                                             neg_off.data(), pos_row.data(), pos_off.data()))
        return rc;
    int64_t need = 0;
    if (int rc = tl_layout_size(neg_off.data(), pos_off.data(), columns, inners, g.tile_rows, g.tile_rows, &need)) return rc;
    if (!blob) {
        *blob_bytes = need;
        return TL_OK;
    }
    if (*blob_bytes < need) return fail(TL_ERR_SIZE, "blob has %lld bytes, %lld needed", (long long)*blob_bytes, (long long)need);
    return tl_layout_build(neg_row.data(), neg_off.data(), pos_row.data(), pos_off.data(), columns, inners, g.tile_rows,
                           g.tile_rows, blob, *blob_bytes);
}

extern "C" int tl_layout_from_mcsc(const void* merged_row, int index_width, int64_t n_index,
                                   const int32_t* merged_off, int columns, int inners, int tile_k,
                                   int uniformed, int tile_rows, void* blob, int64_t* blob_bytes)
{
    if (!merged_off || !blob_bytes || (n_index > 0 && !merged_row)) return fail(TL_ERR_ARG, "null pointer");
    if (columns <= 0 || inners <= 0 || tile_k <= 0) return fail(TL_ERR_SHAPE, "bad dimensions");
    if (index_width != 2 && index_width != 4) return fail(TL_ERR_DTYPE, "index_width=%d (2 or 4 expected)", index_width);
    const int T = (int)ceil_div(inners, tile_k);
    const int16_t* r16 = static_cast<const int16_t*>(merged_row);
    const int32_t* r32 = static_cast<const int32_t*>(merged_row);
    auto at = [&](int64_t i) -> int32_t { return index_width == 2 ? (int32_t)r16[i] : r32[i]; };
    // The walk of the reference kernels, turned into the two row lists of every (column, tile):
    // tiled CSC whose rows may repeat and come in the order the merged stream names them.
    std::vector<int32_t> pos_off((size_t)columns * T * 2), neg_off((size_t)columns * T * 2);
    std::vector<int32_t> pos_row, neg_row;
    for (int y = 0; y < columns; ++y)
        for (int t = 0; t < T; ++t) {
            const int32_t* o = merged_off + ((size_t)y * T + t) * 4;
            if (o[0] < 0 || o[1] < o[0] || o[2] < o[1] || o[2] > n_index || ((o[1] - o[0]) & 1) || (o[3] != 1 && o[3] != -1))
                return fail(TL_ERR_FORMAT, "column %d tile %d: offsets [%d,%d,%d,%d] are not a merged tile", y, t, o[0],
                            o[1], o[2], o[3]);
            const size_t c = ((size_t)y * T + t) * 2;
            pos_off[c] = (int32_t)pos_row.size();
            neg_off[c] = (int32_t)neg_row.size();
            const int64_t end = uniformed ? o[1] : o[2];
            for (int64_t i = o[0]; i < end; ++i) {
                const int32_t r = at(i);
                if (r < 0 || r >= tile_k || (int64_t)t * tile_k + r >= inners)
                    return fail(TL_ERR_FORMAT, "column %d tile %d: row index %d out of range", y, t, r);
                const bool plus = i < o[1] ? ((i - o[0]) & 1) == 0 : o[3] > 0;
                (plus ? pos_row : neg_row).push_back(r);
            }
            if (pos_row.size() > (size_t)INT32_MAX || neg_row.size() > (size_t)INT32_MAX)
                return fail(TL_ERR_UNSUPPORTED, "more than 2^31 entries of one sign");
            pos_off[c + 1] = (int32_t)pos_row.size();
            neg_off[c + 1] = (int32_t)neg_row.size();
        }
    int64_t need = 0;
    if (int rc = tl_layout_size(neg_off.data(), pos_off.data(), columns, inners, tile_k, tile_rows, &need)) return rc;
    if (!blob) {
        *blob_bytes = need;
        return TL_OK;
    }
    if (*blob_bytes < need) return fail(TL_ERR_SIZE, "blob has %lld bytes, %lld needed", (long long)*blob_bytes, (long long)need);
    pos_row.push_back(0);  // never read; keeps data() non-null for an all-zero weight
    neg_row.push_back(0);
    return tl_layout_build(neg_row.data(), neg_off.data(), pos_row.data(), pos_off.data(), columns, inners, tile_k, tile_rows,
                           blob, *blob_bytes);
}

extern "C" int tl_layout_validate(const void* blob, int64_t blob_bytes)
{
    if (!blob) return fail(TL_ERR_ARG, "null blob");
    if (blob_bytes < (int64_t)sizeof(tl_layout_header)) return fail(TL_ERR_FORMAT, "blob shorter than its header");
    tl_layout_header h;
    std::memcpy(&h, blob, sizeof(h));
    if (h.magic != TL_LAYOUT_MAGIC || h.version != TL_LAYOUT_VERSION) return fail(TL_ERR_FORMAT, "bad magic/version %08x/%u", h.magic, h.version);
    if (h.tile_rows == 0 || h.tile_rows > (uint32_t)kMaxTileRows || h.columns == 0 || h.inners == 0 ||
        h.n_tiles != (uint32_t)ceil_div(h.inners, h.tile_rows) || h.n_blocks != (uint32_t)ceil_div(h.columns, kBlock))
        return fail(TL_ERR_FORMAT, "inconsistent geometry K=%u N=%u rows=%u tiles=%u blocks=%u", h.inners, h.columns,
                    h.tile_rows, h.n_tiles, h.n_blocks);
    Geometry g{(int)h.tile_rows, (int)h.n_tiles, (int)h.n_blocks};
    const Sections s = place_sections(g, (int64_t)h.stream_bytes);
    if (h.off_chunkstart != (uint64_t)s.off_chunkstart || h.off_stream != (uint64_t)s.off_stream ||
        h.total_bytes != (uint64_t)s.total || h.total_bytes > (uint64_t)blob_bytes || (h.stream_bytes & 15))
        return fail(TL_ERR_FORMAT, "section table does not match the geometry");
    const uint8_t* base = static_cast<const uint8_t*>(blob);
    const uint32_t* chunkstart = reinterpret_cast<const uint32_t*>(base + h.off_chunkstart);
    const uint32_t* stream = reinterpret_cast<const uint32_t*>(base + h.off_stream);
    const uint32_t T = h.n_tiles, NB = h.n_blocks;
    uint64_t np = 0, nn = 0, expect_start = 0;
    uint32_t run_max = 0, chunk_max = 0;
    for (uint32_t nb = 0; nb < NB; ++nb)
        for (uint32_t t = 0; t < T; ++t) {
            const uint32_t rows_here = (t + 1 == T) ? h.inners - t * h.tile_rows : h.tile_rows;
            if (chunkstart[(size_t)nb * T + t] != expect_start)
                return fail(TL_ERR_FORMAT, "block %u tile %u: start %u, expected %llu", nb, t, chunkstart[(size_t)nb * T + t],
                            (unsigned long long)expect_start);
            if ((expect_start + kBlock) * 4 > h.stream_bytes) return fail(TL_ERR_FORMAT, "block %u tile %u: chunk leaves the stream", nb, t);
            const uint32_t* desc = stream + expect_start;
            uint32_t expect = kBlock;
            for (uint32_t j = 0; j < (uint32_t)kBlock; ++j) {
                const uint32_t y = nb * kBlock + j;
                const uint32_t d = desc[j], p = d & 0xff, n = (d >> 8) & 0xff, off = d >> 16;
                if (off != expect) return fail(TL_ERR_FORMAT, "tile %u column %u: run offset %u, expected %u", t, y, off, expect);
                if (y >= h.columns && (p || n)) return fail(TL_ERR_FORMAT, "tile %u: padding column %u is not empty", t, y);
                const uint32_t pd = (p + 3) / 4, nd = (n + 3) / 4;
                if ((expect_start + off + pd + nd) * 4 > h.stream_bytes) return fail(TL_ERR_FORMAT, "tile %u column %u: run leaves the stream", t, y);
                const uint8_t* run = reinterpret_cast<const uint8_t*>(stream + expect_start + off);
                for (int sign = 0; sign < 2; ++sign) {
                    const uint8_t* r = sign ? run + 4 * pd : run;
                    const uint32_t cnt = sign ? n : p, padded = sign ? 4 * nd : 4 * pd;
                    for (uint32_t i = 0; i < padded; ++i) {
                        if (i < cnt) {
                            if (r[i] >= rows_here) return fail(TL_ERR_FORMAT, "tile %u column %u: row out of range", t, y);
                        } else if (r[i] != kSentinel) {
                            return fail(TL_ERR_FORMAT, "tile %u column %u: padding byte is not the sentinel", t, y);
                        }
                    }
                }
                np += p;
                nn += n;
                expect += pd + nd;
                if (pd + nd > run_max) run_max = pd + nd;
            }
            const uint32_t padded_chunk = (uint32_t)round_up(expect, 4);
            for (uint32_t i = expect; i < padded_chunk; ++i)
                if (stream[expect_start + i] != 0xffffffffu) return fail(TL_ERR_FORMAT, "block %u tile %u: chunk padding is not the sentinel", nb, t);
            if (padded_chunk > chunk_max) chunk_max = padded_chunk;
            expect_start += padded_chunk;
        }
    if (chunkstart[(size_t)T * NB] != expect_start || expect_start * 4 != h.stream_bytes)
        return fail(TL_ERR_FORMAT, "stream length does not match the chunk table");
    if (np != h.nnz_pos || nn != h.nnz_neg || run_max != h.max_run_dwords || chunk_max != h.max_chunk_dwords)
        return fail(TL_ERR_FORMAT, "header totals do not match the streams");
    if (content_checksum(chunkstart, (size_t)T * NB + 1, stream, (size_t)expect_start) != h.checksum)
        return fail(TL_ERR_FORMAT, "checksum of the chunk table and the stream does not match the header");
    return TL_OK;
}

extern "C" int tl_layout_to_dense(const void* blob, int64_t blob_bytes, int32_t* w_out)
{
    if (!w_out) return fail(TL_ERR_ARG, "null output");
    if (int rc = tl_layout_validate(blob, blob_bytes)) return rc;
    tl_layout_header h;
    std::memcpy(&h, blob, sizeof(h));
    const uint8_t* base = static_cast<const uint8_t*>(blob);
    const uint32_t* chunkstart = reinterpret_cast<const uint32_t*>(base + h.off_chunkstart);
    const uint32_t* stream = reinterpret_cast<const uint32_t*>(base + h.off_stream);
    std::memset(w_out, 0, sizeof(int32_t) * (size_t)h.inners * h.columns);
    for (uint32_t y = 0; y < h.columns; ++y)
        for (uint32_t t = 0; t < h.n_tiles; ++t) {
            const uint32_t* chunk = stream + chunkstart[(size_t)(y / kBlock) * h.n_tiles + t];
            const uint32_t d = chunk[y % kBlock], p = d & 0xff, n = (d >> 8) & 0xff;
            const uint8_t* run = reinterpret_cast<const uint8_t*>(chunk + (d >> 16));
            for (uint32_t i = 0; i < p; ++i) w_out[((size_t)t * h.tile_rows + run[i]) * h.columns + y] += 1;
            run += ((p + 3) / 4) * 4;
            for (uint32_t i = 0; i < n; ++i) w_out[((size_t)t * h.tile_rows + run[i]) * h.columns + y] -= 1;
        }
    return TL_OK;
}
