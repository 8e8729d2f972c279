// gfx950 kernels of libternary_spmm for more than 48 activation rows (prefill), and their launchers.
//
//   tl_spmm_rows   Lanes own activation rows, a wave owns C output columns, so an index is wave-uniform: it is
//                  broadcast once and serves 64 * R rows; the activation tile is staged in LDS as [slot][row] so the
//                  gather of a wave is one contiguous, conflict-free LDS read.  Output tiles go one per workgroup, or
//                  their K tiles are shared out evenly among one workgroup per compute unit, with tl_rows_fixup adding
//                  up the partial sums.  tl_relayout_rows_h / tl_relayout_x bring activations into its layout.
//
// Only additions and subtractions touch the data; fp32 accumulation throughout.
#include "tl_device.h"

using namespace tl;

namespace {

// ---------------------------------------------------------------------------
// Activation re-layout for the row-parallel kernel: XT[k][m] (m contiguous, padded
// with zeros to ldm columns) from row-major X[m][k] or K-major X[k][m].
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void tl_relayout_x(const T* __restrict__ X, long long ldx, int kmajor, T* __restrict__ XT,
                                                     long long ldm, int M, int K)
{
    __shared__ T tile[64][65];
    const int k0 = blockIdx.x * 64, m0 = blockIdx.y * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;  // 64 x 4
    if (kmajor) {
        for (int j = ty; j < 64; j += 4) {
            const int k = k0 + j, m = m0 + tx;
            if (k < K) XT[(long long)k * ldm + m] = (m < M) ? X[(long long)k * ldx + m] : T(0.0f);
        }
        return;
    }
    for (int j = ty; j < 64; j += 4) {
        const int m = m0 + j, k = k0 + tx;
        tile[j][tx] = (m < M && k < K) ? X[(long long)m * ldx + k] : T(0.0f);
    }
    __syncthreads();
    for (int j = ty; j < 64; j += 4) {
        const int k = k0 + j, m = m0 + tx;
        if (k < K) XT[(long long)k * ldm + m] = tile[tx][j];
    }
}

// The same image from row-major fp16 rows whose 16-byte pieces are whole and aligned (K and ldx multiples of 8):
// 16 bytes per lane on both sides.  A workgroup turns 128 rows x 64 inner positions; a thread loads the same
// piece of two neighbouring rows and writes them to LDS as (row 2p, row 2p + 1) pairs, one dword per position.
__global__ __launch_bounds__(256) void tl_relayout_rows_h(const __half* __restrict__ X, long long ldx, __half* __restrict__ XT,
                                                          long long ldm, int M, int K)
{
    constexpr int TM = 128, TK = 64, PITCH = TM + 8;  // halves; a row of the turned tile is 272 bytes, whole 16-byte pieces
    __shared__ __align__(16) __half tile[TK][PITCH];
    const int k0 = blockIdx.x * TK, m0 = blockIdx.y * TM, tid = threadIdx.x;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int e = tid + 256 * i, p = e >> 3, c = e & 7;  // row pair p of 64, piece c of 8
        const int m = m0 + 2 * p, k = k0 + 8 * c;
        u32x4 lo = {0u, 0u, 0u, 0u}, hi = {0u, 0u, 0u, 0u};
        if (k < K) {
            if (m < M) lo = *reinterpret_cast<const u32x4*>(X + (long long)m * ldx + k);
            if (m + 1 < M) hi = *reinterpret_cast<const u32x4*>(X + (long long)(m + 1) * ldx + k);
        }
        const uint32_t* l = reinterpret_cast<const uint32_t*>(&lo);
        const uint32_t* h = reinterpret_cast<const uint32_t*>(&hi);
#pragma unroll
        for (int j = 0; j < 4; ++j) {  // dword j holds positions 2j, 2j + 1 of both rows
            *reinterpret_cast<uint32_t*>(&tile[8 * c + 2 * j][2 * p]) = (l[j] & 0xffffu) | (h[j] << 16);
            *reinterpret_cast<uint32_t*>(&tile[8 * c + 2 * j + 1][2 * p]) = (l[j] >> 16) | (h[j] & 0xffff0000u);
        }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int e = tid + 256 * i, k = e >> 4, mc = e & 15;  // position k of 64, piece mc of 16
        if (k0 + k < K)
            *reinterpret_cast<u32x4*>(XT + (long long)(k0 + k) * ldm + m0 + 8 * mc) = *reinterpret_cast<const u32x4*>(&tile[k][8 * mc]);
    }
}

// ---------------------------------------------------------------------------
// Row-parallel kernel.
// ---------------------------------------------------------------------------
// The runs of one wave (C neighbouring columns) for one tile: descriptors, the
// dword where the wave's piece of the stream starts, and its first NPRE * 64 dwords
// (one per lane and chunk), fetched one tile ahead of their use.
constexpr int NPRE = 3;
template <int C>
struct WaveRuns {
    uint32_t d[C];
    uint32_t base;
    uint32_t pre[NPRE];
};

// The three dependent reads behind a wave's runs (chunk offset -> descriptors -> index dwords) are
// spread over three tiles, so that none of them is waited for in the tile that issues it: while tile t
// is consumed, the index dwords of tile t + 1, the descriptors of tile t + 2 and the chunk offset of
// tile t + 3 are in flight.
template <int C>
struct RunFetcher {
    WaveRuns<C> cur, nxt;   // runs of the tile being consumed / of the next one
    uint32_t d1[C];         // descriptors one tile further on
    uint32_t chunk1;        // chunk offset that goes with d1
    uint32_t chunk2;        // chunk offset one tile further still
    const_u32_ptr chunkstart, stream_c;
    const uint32_t* stream;
    int sub, lane;

    __device__ __forceinline__ void descriptors(uint32_t (&d)[C], uint32_t chunk) const
    {
        const_u32_ptr dp = stream_c + chunk + sub;
#pragma unroll
        for (int c = 0; c < C; ++c) d[c] = dp[c];
    }
    // NPRE * 64 dwords from the start of the wave's piece, whatever its length: what lies past the piece is
    // never used, and past the stream's end the blob keeps as many spare bytes (tl_layout.cpp, kStreamSpareBytes).
    __device__ __forceinline__ void indices(WaveRuns<C>& r, uint32_t chunk) const
    {
        r.base = chunk + (r.d[0] >> 16);
#pragma unroll
        for (int ch = 0; ch < NPRE; ++ch) r.pre[ch] = stream[r.base + ch * 64 + lane];
    }
    // Makes tile t0 the next one advance() hands out.
    __device__ __forceinline__ void prime(const WeightPtrs& w, int T, int n0, int lane_, int t0)
    {
        chunkstart = as_const(w.chunkstart) + (size_t)(n0 / TL_BLOCK_COLUMNS) * T;
        stream_c = as_const(w.stream);
        stream = w.stream;
        sub = n0 % TL_BLOCK_COLUMNS;
        lane = lane_;
        const uint32_t chunk0 = chunkstart[t0];
        descriptors(nxt.d, chunk0);
        indices(nxt, chunk0);
        chunk1 = chunk2 = 0;
#pragma unroll
        for (int c = 0; c < C; ++c) d1[c] = 0;
        if (t0 + 1 < T) {
            chunk1 = chunkstart[t0 + 1];
            descriptors(d1, chunk1);
        }
        if (t0 + 2 < T) chunk2 = chunkstart[t0 + 2];
    }
    // Call at the start of tile t: afterwards `cur` holds tile t's runs.
    __device__ __forceinline__ void advance(int t, int T)
    {
        cur = nxt;
        if (t + 1 < T) {
#pragma unroll
            for (int c = 0; c < C; ++c) nxt.d[c] = d1[c];
            indices(nxt, chunk1);
        }
        if (t + 2 < T) {
            descriptors(d1, chunk2);
            chunk1 = chunk2;
        }
        if (t + 3 < T) chunk2 = chunkstart[t + 3];
    }
};

// The inner loop of the row-parallel kernel, written out in assembly.
//
// A slot of the staged tile is 512 bytes for both activation types (256 fp16 rows / 128 fp32 rows), and a lane
// reads its 8 bytes of a slot with one ds_read_b64: rows 4l .. 4l + 3 (fp16) or 2l, 2l + 1 (fp32) of the row
// tile.  An 8-byte read moves twice the bytes of a 4-byte one in nearly the same LDS time (1.47 against
// 1.31 ns per wave instruction and compute unit, measured), which is what makes the vector ALU and not the
// LDS the unit this loop keeps busy.  Per dword of four indices: one v_readlane (the dword sits in a lane of
// the chunk vector), four scalar byte extractions, four v_lshl_or (address = slot * 512 | 8 * lane, written
// into the low register of the pair the read then fills), four LDS reads, and 16 (fp16) or 8 (fp32)
// accumulating vector ops.  Two register sets alternate so that the reads of dword i + 1 are in flight while
// dword i is accumulated; LDS reads complete in issue order, so "lgkmcnt(4)" means everything but the four
// reads issued last has arrived.
// The register pairs are named outright (the halves of a 64-bit asm operand cannot be named), and listed as
// clobbered so that the compiler keeps them free around the loop.
#define TL_RUN_CLOBBERS "v112", "v113", "v114", "v115", "v116", "v117", "v118", "v119", "v120", "v121", "v122", "v123", "v124", "v125", "v126", "v127"

#define TL_ISSUE(L0, H0, L1, H1, L2, H2, L3, H3)                     \
    "s_bfe_u32 %[t], %[w], 0x80000\n\t"                              \
    "s_bfe_u32 %[u], %[w], 0x80008\n\t"                              \
    "v_lshl_or_b32 v" L0 ", %[t], 9, %[l8]\n\t"                      \
    "s_bfe_u32 %[t], %[w], 0x80010\n\t"                              \
    "v_lshl_or_b32 v" L1 ", %[u], 9, %[l8]\n\t"                      \
    "s_lshr_b32 %[u], %[w], 24\n\t"                                  \
    "ds_read_b64 v[" L0 ":" H0 "], v" L0 "\n\t"                      \
    "v_lshl_or_b32 v" L2 ", %[t], 9, %[l8]\n\t"                      \
    "ds_read_b64 v[" L1 ":" H1 "], v" L1 "\n\t"                      \
    "v_lshl_or_b32 v" L3 ", %[u], 9, %[l8]\n\t"                      \
    "s_add_u32 %[i], %[i], 1\n\t"                                    \
    "ds_read_b64 v[" L2 ":" H2 "], v" L2 "\n\t"                      \
    "ds_read_b64 v[" L3 ":" H3 "], v" L3 "\n\t"

// fp16: a dword holds two rows; the mixed-precision fma converts and accumulates in one op
#define TL_FMA_H(L, H)                                                                      \
    "v_fma_mix_f32 %[c0], v" L ", %[sg], %[c0] op_sel_hi:[1,0,0]\n\t"                        \
    "v_fma_mix_f32 %[c1], v" L ", %[sg], %[c1] op_sel:[1,0,0] op_sel_hi:[1,0,0]\n\t"         \
    "v_fma_mix_f32 %[c2], v" H ", %[sg], %[c2] op_sel_hi:[1,0,0]\n\t"                        \
    "v_fma_mix_f32 %[c3], v" H ", %[sg], %[c3] op_sel:[1,0,0] op_sel_hi:[1,0,0]\n\t"
#define TL_FMA_F(L, H)                                  \
    "v_fma_f32 %[c0], v" L ", %[sg], %[c0]\n\t"          \
    "v_fma_f32 %[c1], v" H ", %[sg], %[c1]\n\t"

#define TL_ISSUE_A TL_ISSUE("112", "113", "114", "115", "116", "117", "118", "119")
#define TL_ISSUE_B TL_ISSUE("120", "121", "122", "123", "124", "125", "126", "127")
#define TL_ACC_A(F) F("112", "113") F("114", "115") F("116", "117") F("118", "119")
#define TL_ACC_B(F) F("120", "121") F("122", "123") F("124", "125") F("126", "127")

#define TL_RUN_LOOP(F)                                   \
    "v_readlane_b32 %[w], %[v], %[i]\n\t"                \
    TL_ISSUE_A                                           \
    "Ltl_loop%=:\n\t"                                    \
    "s_cmp_lt_u32 %[i], %[hi]\n\t"                       \
    "s_cbranch_scc0 Ltl_lastA%=\n\t"                     \
    "v_readlane_b32 %[w], %[v], %[i]\n\t"                \
    TL_ISSUE_B                                           \
    "s_waitcnt lgkmcnt(4)\n\t"                           \
    TL_ACC_A(F)                                          \
    "s_cmp_lt_u32 %[i], %[hi]\n\t"                       \
    "s_cbranch_scc0 Ltl_lastB%=\n\t"                     \
    "v_readlane_b32 %[w], %[v], %[i]\n\t"                \
    TL_ISSUE_A                                           \
    "s_waitcnt lgkmcnt(4)\n\t"                           \
    TL_ACC_B(F)                                          \
    "s_branch Ltl_loop%=\n\t"                            \
    "Ltl_lastA%=:\n\t"                                   \
    "s_waitcnt lgkmcnt(0)\n\t"                           \
    TL_ACC_A(F)                                          \
    "s_branch Ltl_end%=\n\t"                             \
    "Ltl_lastB%=:\n\t"                                   \
    "s_waitcnt lgkmcnt(0)\n\t"                           \
    TL_ACC_B(F)                                          \
    "Ltl_end%=:"

// The dwords [lo, hi) of the chunk vector `v` (dword i sits in lane i), all of one column and one
// sign: acc += sgn * (rows of the tile at each index).  lo < hi.  lane8 = 8 * lane.
template <typename XT, int R>
__device__ __forceinline__ void rows_run(float (&acc)[R], uint32_t v, int lo, int hi, float sgn_one, uint32_t lane8)
{
    uint32_t w, t, u;
    uint32_t i = (uint32_t)lo;
    if constexpr (sizeof(XT) == 2) {
        static_assert(R == 4, "fp16 row tiles hold 4 rows per lane");
        asm volatile(TL_RUN_LOOP(TL_FMA_H)
                     : [c0] "+v"(acc[0]), [c1] "+v"(acc[1]), [c2] "+v"(acc[2]), [c3] "+v"(acc[3]), [i] "+s"(i),
                       [w] "=&s"(w), [t] "=&s"(t), [u] "=&s"(u)
                     : [v] "v"(v), [hi] "s"((uint32_t)hi), [sg] "s"(sgn_one), [l8] "v"(lane8)
                     : TL_RUN_CLOBBERS, "scc", "memory");
    } else {
        static_assert(R == 2, "fp32 row tiles hold 2 rows per lane");
        asm volatile(TL_RUN_LOOP(TL_FMA_F)
                     : [c0] "+v"(acc[0]), [c1] "+v"(acc[1]), [i] "+s"(i), [w] "=&s"(w), [t] "=&s"(t), [u] "=&s"(u)
                     : [v] "v"(v), [hi] "s"((uint32_t)hi), [sg] "s"(sgn_one), [l8] "v"(lane8)
                     : TL_RUN_CLOBBERS, "scc", "memory");
    }
}

// Wave priority for run `r` of the `total` runs a wave works through per tile.  The issue arbiter serves the
// oldest wave of a SIMD first, so left alone the four waves of a SIMD drift far apart inside a tile and the
// early ones idle at the tile's barrier (a quarter of the kernel's time, measured).  Priority that falls with
// progress holds back the waves that are ahead; the steps shrink towards the end of the tile, because what the
// waves differ by when they arrive is at most the last step.
template <int r, int total>
__device__ __forceinline__ void progress_priority()
{
    if constexpr (r * 16 < 7 * total) __builtin_amdgcn_s_setprio(3);
    else if constexpr (r * 16 < 12 * total) __builtin_amdgcn_s_setprio(2);
    else if constexpr (r * 16 < 15 * total) __builtin_amdgcn_s_setprio(1);
    else __builtin_amdgcn_s_setprio(0);
}

// Column c (of C, counted from compile-time index) of one 64-dword chunk of the wave's piece.
template <typename XT, int R, int C, int RUN0, int RUNS, int c>
__device__ __forceinline__ void rows_chunk_column(float (&acc)[C][R], const int (&pb)[C], const int (&pe)[C], const int (&ne)[C],
                                                  uint32_t v, int cb, float one, uint32_t lane8)
{
    int lo = max(pb[c], cb) - cb, hi = min(pe[c], cb + 64) - cb;
    if (lo < hi) {
        progress_priority<RUN0 + 2 * c, RUNS>();
        rows_run<XT, R>(acc[c], v, lo, hi, one, lane8);
    }
    lo = max(pe[c], cb) - cb;
    hi = min(ne[c], cb + 64) - cb;
    if (lo < hi) {
        progress_priority<RUN0 + 2 * c + 1, RUNS>();
        rows_run<XT, R>(acc[c], v, lo, hi, -one, lane8);
    }
    if constexpr (c + 1 < C) rows_chunk_column<XT, R, C, RUN0, RUNS, c + 1>(acc, pb, pe, ne, v, cb, one, lane8);
}

// One 64-dword chunk of the wave's piece: dword i of the piece sits in lane i - cb of `v`
// and is broadcast from there, so its four row indices are wave-uniform.  The wave's runs are numbered
// RUN0 ... of RUNS per tile (two per column; the fused kernel walks two weights).
template <typename XT, int R, int C, int RUN0, int RUNS>
__device__ __forceinline__ void rows_chunk(float (&acc)[C][R], const int (&pb)[C], const int (&pe)[C], const int (&ne)[C],
                                           uint32_t v, int cb, float one, uint32_t lane8)
{
    rows_chunk_column<XT, R, C, RUN0, RUNS, 0>(acc, pb, pe, ne, v, cb, one, lane8);
}

template <typename XT, int R, int C, int RUN0, int RUNS>
__device__ __forceinline__ void rows_consume(float (&acc)[C][R], const WaveRuns<C>& r, const uint32_t* __restrict__ idx,
                                             int lane, float one)
{
    int pb[C], pe[C], ne[C];
    const uint32_t lane8 = (uint32_t)lane * 8u;
#pragma unroll
    for (int c = 0; c < C; ++c) {
        pb[c] = (int)((r.d[c] >> 16) - (r.d[0] >> 16));
        pe[c] = pb[c] + run_pos_dwords(r.d[c]);
        ne[c] = pe[c] + run_neg_dwords(r.d[c]);
    }
    const int total = ne[C - 1];
#pragma unroll
    for (int ch = 0; ch < NPRE; ++ch)
        if (ch * 64 < total) rows_chunk<XT, R, C, RUN0, RUNS>(acc, pb, pe, ne, r.pre[ch], ch * 64, one, lane8);
    for (int cb = NPRE * 64; cb < total; cb += 64)  // pieces longer than the prefetch window: fetched on demand
        rows_chunk<XT, R, C, RUN0, RUNS>(acc, pb, pe, ne, idx[r.base + cb + lane], cb, one, lane8);
}

// Staging of one activation tile: global -> registers (issued a tile ahead), registers -> LDS.
// A thread owns the 16-byte chunks threadIdx.x + i * NT of the tile.  Their byte offsets from the tile's first
// row are the same for every full tile, so they are computed once (stage_offsets) and a tile's loads
// take only a wave-uniform base on top; the last tile, when it is shorter, gets offsets of its own.
template <typename XT, int CHUNKS, int NT, int PER>
__device__ __forceinline__ void stage_offsets(uint32_t (&voff)[PER], const KernelArgs& a, int rows)
{
    const int n_chunks = rows * CHUNKS;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        // Chunks past the tile's end re-read its last chunk (never stored): the load stays unconditional.
        const int e = min((int)threadIdx.x + i * NT, n_chunks - 1);
        const int r = e / CHUNKS, ch = e % CHUNKS;
        voff[i] = (uint32_t)r * (uint32_t)a.ldx * (uint32_t)sizeof(XT) + (uint32_t)ch * 16u;
    }
}

template <int PER>
__device__ __forceinline__ void tile_to_regs(u32x4 (&pf)[PER], const unsigned char* __restrict__ tile_base, const uint32_t (&voff)[PER])
{
#pragma unroll
    for (int i = 0; i < PER; ++i) pf[i] = *reinterpret_cast<const u32x4*>(tile_base + voff[i]);
}

template <int CHUNKS, int NT, int PER>
__device__ __forceinline__ void regs_to_lds(const u32x4 (&pf)[PER], unsigned char* smem, const KernelArgs& a, int t)
{
    const int n_chunks = min(a.tile_rows, a.K - t * a.tile_rows) * CHUNKS;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int e = (int)threadIdx.x + i * NT;
        if (e < n_chunks) *reinterpret_cast<u32x4*>(smem + (size_t)e * 16) = pf[i];
    }
}

// Scale, optional SiLU gate, and store of one workgroup's output tile.  Row of accumulator j of a lane:
// row R * l + j of the row tile.
// A lane holds C neighbouring columns of R scattered rows, so storing from the accumulators would write
// 2- or 4-byte pieces a row apart.  The tile therefore goes through LDS (the activation tile's space,
// free by now): lanes write their C columns of a row side by side, then the workgroup stores whole
// rows of WAVES * C columns, 8 or 16 bytes per lane.  Output tiles that the matrix edge cuts, or whose
// rows are not aligned for that, are stored value by value.
template <typename XT, int R, int C, int WAVES, bool GATED, bool PAIRS>
__device__ __forceinline__ void rows_store(const KernelArgs& a, int m0, int n_wg, int wave, int lane, const float (&acc)[C][R],
                                           const float (&acc2)[GATED ? C : 1][R], unsigned char* smem)
{
    constexpr int MTILE = 64 * R;
    constexpr int COLS = WAVES * C;
    static_assert(C % 4 == 0, "the staged store moves groups of four columns per lane");
    // The store's addresses are worked out here: left to the compiler they are computed at the top of the kernel and
    // spilled across the tile loop (a dozen dwords per thread of scratch traffic, written and read back).
    int tid = (int)threadIdx.x;
    asm volatile("" : "+v"(tid), "+v"(lane));
    const int n0 = n_wg + wave * C;
    if constexpr (PAIRS) {
        // One weight whose columns are (gate, up) pairs: a wave's C columns are C / 2 whole pairs, and column n / 2 of
        // the output is silu(y[n]) * y[n + 1], both rounded to the output type first, as the product followed by
        // the pairs form of the SiLU kernel rounds.  The tile that goes out is half as wide.
        static_assert(!GATED && C % 8 == 0, "pairs of the plain kernel's columns, four outputs per lane and staged piece");
        constexpr int HC = C / 2, HCOLS = COLS / 2;
        float h[HC][R];
#pragma unroll
        for (int p = 0; p < HC; ++p) {
            const int n = min(n0 + 2 * p, a.N - 1), nu = min(n0 + 2 * p + 1, a.N - 1);
            const float sg = load_scale(a.w0.scale, a.scale_f16, n), su = load_scale(a.w0.scale, a.scale_f16, nu);
#pragma unroll
            for (int j = 0; j < R; ++j)
                h[p][j] = gate_pair(as_output(acc[2 * p][j] * sg, a.y_f16), as_output(acc[2 * p + 1][j] * su, a.y_f16), a.y_f16);
        }
        const int es = a.y_f16 ? 2 : 4;
        const int stride = HCOLS * es + 4 * es;
        const bool whole = n_wg + COLS <= a.N && (a.ldy * es) % (4 * es) == 0 &&
                           (reinterpret_cast<uintptr_t>(a.Y) + (size_t)(n_wg / 2) * es) % (4 * es) == 0 &&
                           (size_t)MTILE * stride <= (size_t)kSentinel * MTILE * sizeof(XT);
        if (!whole) {
#pragma unroll
            for (int p = 0; p < HC; ++p) {
                const int n = n0 + 2 * p;
                if (n + 1 >= a.N) continue;
#pragma unroll
                for (int j = 0; j < R; ++j) {
                    const int m = m0 + R * lane + j;
                    if (m < a.M) store_out(a.Y, a.y_f16, (long long)m * a.ldy + n / 2, h[p][j]);
                }
            }
            return;
        }
        __syncthreads();  // every wave is done reading the activation tile
#pragma unroll
        for (int j = 0; j < R; ++j) {
            const int r = R * lane + j;
#pragma unroll
            for (int g = 0; g < HC; g += 4) {
                unsigned char* dst = smem + (size_t)r * stride + (size_t)(wave * HC + g) * es;
                if (a.y_f16) {
                    const __half2 lo = __floats2half2_rn(settled(h[g][j]), settled(h[g + 1][j])), hi = __floats2half2_rn(settled(h[g + 2][j]), settled(h[g + 3][j]));
                    *reinterpret_cast<uint2*>(dst) = make_uint2(*reinterpret_cast<const uint32_t*>(&lo), *reinterpret_cast<const uint32_t*>(&hi));
                } else {
                    *reinterpret_cast<float4*>(dst) = make_float4(h[g][j], h[g + 1][j], h[g + 2][j], h[g + 3][j]);
                }
            }
        }
        __syncthreads();
        constexpr int LANES_PER_ROW = HCOLS / 4;
        constexpr int ROWS_PER_PASS = WAVES * 64 / LANES_PER_ROW;
        const int q = tid % LANES_PER_ROW, r0 = tid / LANES_PER_ROW;
#pragma unroll
        for (int r = r0; r < MTILE; r += ROWS_PER_PASS) {
            const int m = m0 + r;
            if (m >= a.M) continue;
            const unsigned char* src = smem + (size_t)r * stride + (size_t)q * 4 * es;
            unsigned char* out = static_cast<unsigned char*>(a.Y) + ((size_t)m * a.ldy + n_wg / 2 + q * 4) * es;
            if (a.y_f16) *reinterpret_cast<uint2*>(out) = *reinterpret_cast<const uint2*>(src);
            else *reinterpret_cast<float4*>(out) = *reinterpret_cast<const float4*>(src);
        }
        return;
    }
    float v[C][R];
#pragma unroll
    for (int c = 0; c < C; ++c) {
        const int n = min(n0 + c, a.N - 1);
        const float s = load_scale(a.w0.scale, a.scale_f16, n);
        const float s2 = GATED ? load_scale(a.w1.scale, a.scale_f16, n) : 1.0f;
#pragma unroll
        for (int j = 0; j < R; ++j) {
            v[c][j] = acc[c][j] * s;
            if constexpr (GATED) v[c][j] = silu(v[c][j]) * (acc2[GATED ? c : 0][j] * s2);
        }
    }
    const int es = a.y_f16 ? 2 : 4;
    const int stride = COLS * es + 4 * es;  // bytes per staged row: the pad keeps the lanes' writes off one bank
    // uniform over the workgroup; the staged tile must stay below the sentinel slot at the end of the activation tile
    const bool whole = n_wg + COLS <= a.N && (a.ldy * es) % (4 * es) == 0 &&
                       (reinterpret_cast<uintptr_t>(a.Y) + (size_t)n_wg * es) % (4 * es) == 0 &&
                       (size_t)MTILE * stride <= (size_t)kSentinel * MTILE * sizeof(XT);
    if (!whole) {
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const int n = n0 + c;
            if (n >= a.N) continue;
#pragma unroll
            for (int j = 0; j < R; ++j) {
                const int m = m0 + R * lane + j;
                if (m < a.M) store_out(a.Y, a.y_f16, (long long)m * a.ldy + n, v[c][j]);
            }
        }
        return;
    }
    __syncthreads();  // every wave is done reading the activation tile
#pragma unroll
    for (int j = 0; j < R; ++j) {
        const int r = R * lane + j;
#pragma unroll
        for (int g = 0; g < C; g += 4) {
            unsigned char* dst = smem + (size_t)r * stride + (size_t)(wave * C + g) * es;
            if (a.y_f16) {
                const __half2 lo = __floats2half2_rn(v[g][j], v[g + 1][j]), hi = __floats2half2_rn(v[g + 2][j], v[g + 3][j]);
                *reinterpret_cast<uint2*>(dst) = make_uint2(*reinterpret_cast<const uint32_t*>(&lo), *reinterpret_cast<const uint32_t*>(&hi));
            } else {
                *reinterpret_cast<float4*>(dst) = make_float4(v[g][j], v[g + 1][j], v[g + 2][j], v[g + 3][j]);
            }
        }
    }
    __syncthreads();
    constexpr int LANES_PER_ROW = COLS / 4;             // each lane moves four columns
    constexpr int ROWS_PER_PASS = WAVES * 64 / LANES_PER_ROW;
    const int q = tid % LANES_PER_ROW, r0 = tid / LANES_PER_ROW;
#pragma unroll
    for (int r = r0; r < MTILE; r += ROWS_PER_PASS) {
        const int m = m0 + r;
        if (m >= a.M) continue;
        const unsigned char* src = smem + (size_t)r * stride + (size_t)q * 4 * es;
        unsigned char* out = static_cast<unsigned char*>(a.Y) + ((size_t)m * a.ldy + n_wg + q * 4) * es;
        if (a.y_f16) *reinterpret_cast<uint2*>(out) = *reinterpret_cast<const uint2*>(src);
        else *reinterpret_cast<float4*>(out) = *reinterpret_cast<const float4*>(src);
    }
}

// Where the partial sums of a workgroup that owns only some tiles of an output tile go: slot
// (workgroup, which) of the partial area, one float per (wave, column, accumulator, lane), the gate's
// set first and the up projection's after it.
template <int R, int C, int WAVES, bool GATED>
__device__ __forceinline__ float* partial_slot(float* base, int lin, int which)
{
    constexpr size_t kSet = (size_t)WAVES * C * R * 64;
    return base + ((size_t)lin * 2 + which) * kSet * (GATED ? 2 : 1);
}

// The step list is (output tile, K tile) in output-tile-major order; workgroup `lin` of G owns steps
// [lin * S / G, (lin + 1) * S / G).
__device__ __host__ inline long long split_begin(long long lin, long long S, long long G) { return lin * S / G; }
__device__ __host__ inline long long split_owner(long long step, long long S, long long G) { return ((step + 1) * G - 1) / S; }

template <typename XT, int R, int C, int WAVES, bool GATED, bool PAIRS = false>
__global__ __launch_bounds__(WAVES * 64) void tl_spmm_rows(KernelArgs a)
{
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int MTILE = 64 * R;
    constexpr int NT = WAVES * 64;
    constexpr int CHUNKS = MTILE * (int)sizeof(XT) / 16;                 // 16-byte chunks per staged row
    constexpr int PER = (kMaxTileRows * CHUNKS + NT - 1) / NT;           // chunks one thread stages per tile
    static_assert(TL_BLOCK_COLUMNS % C == 0, "a wave's columns must not straddle column blocks");
    XT* tile = reinterpret_cast<XT*>(smem);                              // [256 slots][MTILE]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // Workgroups are dealt to the 8 XCDs round-robin by linear id, and every XCD has its own L2.
    // The id is therefore re-read so that XCD x works through one contiguous eighth of the
    // (row tile, column tile) list, row tile major: the workgroups that share an L2 then share
    // the same few row tiles of the activations instead of all of them.
    const int n_col_tiles = (a.N + WAVES * C - 1) / (WAVES * C);
    const int total = (int)gridDim.x;
    int lin = (int)blockIdx.x;
    const int per_xcd = total / 8;
    if (lin < per_xcd * 8) lin = (lin & 7) * per_xcd + (lin >> 3);
    // A workgroup first works through a.whole_units output tiles of its own.  With a.split_steps != 0 the
    // output tiles from a.split_first_unit on are left over, and each workgroup takes an equal share of
    // their (output tile, K tile) steps: it may then own only the last tiles of one output tile and only
    // the first tiles of the next, and leaves partial sums for tl_rows_fixup to add up.
    int own = 0;
    long long step = a.split_steps ? split_begin(lin, a.split_steps, total) : 0;
    const long long step_end = a.split_steps ? split_begin(lin + 1, a.split_steps, total) : 0;
    const unsigned char* __restrict__ XTr = static_cast<const unsigned char*>(a.X);  // [K][ldx] of XT, m contiguous
    const int last_rows = a.K - (a.T - 1) * a.tile_rows;
    const size_t tile_stride = (size_t)a.tile_rows * a.ldx * sizeof(XT);  // bytes between the first rows of two tiles

    // Slot 255 is what padding bytes address: zero it once, staging never writes it.
    for (int e = threadIdx.x; e < MTILE; e += NT) tile[kSentinel * MTILE + e] = XT(0.0f);

    while (own < a.whole_units || step < step_end) {
        int unit, t0, t1;
        if (own < a.whole_units) {
            unit = lin * a.whole_units + own;
            t0 = 0;
            t1 = a.T;
            ++own;
        } else {
            const int shared = (int)(step / a.T);
            unit = a.split_first_unit + shared;
            t0 = (int)(step - (long long)shared * a.T);
            t1 = (int)min((long long)a.T, t0 + (step_end - step));
            step += t1 - t0;
        }
        const int m0 = (unit / n_col_tiles) * MTILE;
        const int n0 = (unit % n_col_tiles) * (WAVES * C) + wave * C;
        const bool wave_live = n0 < a.N;                                   // uniform; then n0 lies inside a stored column block

        float acc[C][R];
        float acc2[GATED ? C : 1][R];
#pragma unroll
        for (int c = 0; c < C; ++c)
#pragma unroll
            for (int j = 0; j < R; ++j) {
                acc[c][j] = 0.f;
                if (GATED) acc2[GATED ? c : 0][j] = 0.f;
            }

        // The next activation tile travels global -> registers while the current one is consumed.
        u32x4 pf[PER];
        RunFetcher<C> f0, f1;
        if (wave_live) {
            f0.prime(a.w0, a.T, n0, lane, t0);
            if constexpr (GATED) f1.prime(a.w1, a.T, n0, lane, t0);
        }
        uint32_t voff[PER];
        const unsigned char* __restrict__ col0 = XTr + (size_t)m0 * sizeof(XT);
        stage_offsets<XT, CHUNKS, NT, PER>(voff, a, t0 + 1 < a.T ? a.tile_rows : last_rows);
        tile_to_regs<PER>(pf, col0 + (size_t)t0 * tile_stride, voff);
        for (int t = t0; t < t1; ++t) {
            __syncthreads();  // every wave is done with the previous tile
            regs_to_lds<CHUNKS, NT, PER>(pf, smem, a, t);
            __syncthreads();
            if (t + 1 < t1) {
                if (t + 2 == a.T && last_rows != a.tile_rows) stage_offsets<XT, CHUNKS, NT, PER>(voff, a, last_rows);
                tile_to_regs<PER>(pf, col0 + (size_t)(t + 1) * tile_stride, voff);
            }
            if (wave_live) {
                f0.advance(t, a.T);
                if constexpr (GATED) f1.advance(t, a.T);
                constexpr int RUNS = (GATED ? 4 : 2) * C;  // runs of a wave per tile
                rows_consume<XT, R, C, 0, RUNS>(acc, f0.cur, a.w0.stream, lane, a.one);
                if constexpr (GATED) rows_consume<XT, R, C, 2 * C, RUNS>(acc2, f1.cur, a.w1.stream, lane, a.one);
            }
        }

        if (t0 == 0 && t1 == a.T) {
            rows_store<XT, R, C, WAVES, GATED, PAIRS>(a, m0, (unit % n_col_tiles) * (WAVES * C), wave, lane, acc, acc2, smem);
        } else {
            float* part = partial_slot<R, C, WAVES, GATED>(a.partial, lin, t0 > 0 ? 0 : 1);
#pragma unroll
            for (int c = 0; c < C; ++c)
#pragma unroll
                for (int j = 0; j < R; ++j) {
                    part[((size_t)(wave * C + c) * R + j) * 64 + lane] = acc[c][j];
                    if constexpr (GATED) part[((size_t)(WAVES * C + wave * C + c) * R + j) * 64 + lane] = acc2[GATED ? c : 0][j];
                }
        }
    }
}

// One workgroup per shared-out output tile: adds up the partial sums its workgroups left and finishes
// the tile (nothing to do when the whole tile fell into one workgroup's share).
template <typename XT, int R, int C, int WAVES, bool GATED, bool PAIRS = false>
__global__ __launch_bounds__(WAVES * 64) void tl_rows_fixup(KernelArgs a, int G)
{
    constexpr int MTILE = 64 * R;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int n_col_tiles = (a.N + WAVES * C - 1) / (WAVES * C);
    const int unit = a.split_first_unit + (int)blockIdx.x;
    const long long first = (long long)blockIdx.x * a.T, last = first + a.T - 1;  // in the list of shared-out steps
    const int lin_a = (int)split_owner(first, a.split_steps, G), lin_b = (int)split_owner(last, a.split_steps, G);
    if (lin_a == lin_b) return;  // one workgroup had all of it and has stored it
    const int m0 = (unit / n_col_tiles) * MTILE;
    float acc[C][R];
    float acc2[GATED ? C : 1][R];
#pragma unroll
    for (int c = 0; c < C; ++c)
#pragma unroll
        for (int j = 0; j < R; ++j) {
            acc[c][j] = 0.f;
            if (GATED) acc2[GATED ? c : 0][j] = 0.f;
        }
    for (int lin = lin_a; lin <= lin_b; ++lin) {
        const long long begin = split_begin(lin, a.split_steps, G);
        if (split_begin(lin + 1, a.split_steps, G) == begin) continue;  // fewer steps than workgroups: this one had none
        // a workgroup whose share starts inside this tile left its sums in slot 0, one that started earlier in slot 1
        const float* part = partial_slot<R, C, WAVES, GATED>(a.partial, lin, begin > first ? 0 : 1);
#pragma unroll
        for (int c = 0; c < C; ++c)
#pragma unroll
            for (int j = 0; j < R; ++j) {
                acc[c][j] += part[((size_t)(wave * C + c) * R + j) * 64 + lane];
                if constexpr (GATED) acc2[GATED ? c : 0][j] += part[((size_t)(WAVES * C + wave * C + c) * R + j) * 64 + lane];
            }
    }
    extern __shared__ __align__(16) unsigned char smem[];
    rows_store<XT, R, C, WAVES, GATED, PAIRS>(a, m0, (unit % n_col_tiles) * (WAVES * C), wave, lane, acc, acc2, smem);
}

static_assert(kRowsColsPlain == 2 * kRowsCols, "one accumulator set of the plain kernel is as large as the fused kernel's two");

template <typename XT, int R, bool GATED, bool PAIRS = false>
int launch_rows_t(KernelArgs a, void* partial, int64_t partial_bytes, hipStream_t st)
{
    constexpr int MTILE = 64 * R;
    const size_t lds = (size_t)kTileSlots * MTILE * sizeof(XT);
    constexpr int COLS = GATED ? kRowsCols : kRowsColsPlain;
    auto kernel = tl_spmm_rows<XT, R, COLS, kRowsWaves, GATED, PAIRS>;
    static bool raised = false;  // per instantiation; a repeated call is harmless
    if (!raised) {
        // the kernel addresses its activation tile from LDS offset 0: it must own no static LDS
        hipFuncAttributes attr;
        if (hipFuncGetAttributes(&attr, reinterpret_cast<const void*>(kernel)) != hipSuccess || attr.sharedSizeBytes != 0)
            return fail(TL_ERR_LAUNCH, "row kernel was built with static LDS; its tile would not start at offset 0");
        if (int rc = raise_lds_limit(kernel, lds)) return rc;
        raised = true;
    }
    const int64_t units = ceil_div(a.N, kRowsWaves * COLS) * ceil_div(a.M, MTILE);
    // One workgroup per output tile leaves compute units idle in the last round (or all along, with
    // fewer tiles than units).  When that costs more than a few percent, one workgroup per compute
    // unit is launched instead: each works through an equal number of whole output tiles, the tiles
    // left over are shared out by (output tile, K tile) steps, and a second small launch adds up the
    // partial sums of those.
    const int G = std::min(compute_units(), kMaxComputeUnits);  // workgroups of a one-per-compute-unit launch
    const int64_t rounds = ceil_div(units, G);
    const bool uneven = (double)rounds * G > 1.06 * (double)units;
    const bool want = knob(TL_ROWS_SPLIT, uneven && units * a.T >= 4 * G ? 1 : 0) != 0;
    const int64_t leftover = units % G;  // output tiles beyond an equal number of whole ones per workgroup
    if (want && leftover && partial && partial_bytes >= kRowsPartialBytes && reinterpret_cast<uintptr_t>(partial) % 16 == 0 && a.T >= 2) {
        a.whole_units = (int)(units / G);
        a.split_first_unit = a.whole_units * G;
        a.split_steps = leftover * a.T;
        a.partial = static_cast<float*>(partial);
        hipLaunchKernelGGL(kernel, dim3((unsigned)G), dim3(kRowsWaves * 64), lds, st, a);
        // LDS of the fix-up: the staged output tile (fp32 at most, padded rows)
        const size_t fix_lds = (size_t)MTILE * (kRowsWaves * COLS * 4 + 16);
        auto fixup = tl_rows_fixup<XT, R, COLS, kRowsWaves, GATED, PAIRS>;
        static bool fix_raised = false;
        if (!fix_raised) {
            if (int rc = raise_lds_limit(fixup, fix_lds)) return rc;
            fix_raised = true;
        }
        hipLaunchKernelGGL(fixup, dim3((unsigned)leftover), dim3(kRowsWaves * 64), fix_lds, st, a, G);
        return TL_OK;
    }
    a.split_steps = 0;
    a.whole_units = 1;
    a.split_first_unit = 0;
    hipLaunchKernelGGL(kernel, dim3((unsigned)units), dim3(kRowsWaves * 64), lds, st, a);  // 1-D: the kernel maps ids to tiles
    return TL_OK;
}

// K-major activations whose leading dimension is a whole number of row tiles (and 16-byte aligned)
// are what the row-parallel kernel reads directly; anything else goes through the re-layout pre-pass.
inline bool rows_needs_relayout(const void* X, int x_dtype, int x_layout, int64_t ldx, int64_t M)
{
    const int mtile = rows_mtile(x_dtype);
    return x_layout != TL_X_K_MAJOR || ldx % mtile != 0 || ldx < round_up(M, mtile) || reinterpret_cast<uintptr_t>(X) % 16 != 0;
}

// Runs the re-layout pre-pass into `workspace` when needed, then the row-parallel kernel.  The
// workspace holds the K-major image of the activations first, the partial sums behind it.
int rows_launch(KernelArgs a, int x_dtype, void* workspace, int64_t workspace_bytes, bool gated, hipStream_t st)
{
    const int64_t image = rows_relayout_bytes(a.K, a.M, x_dtype);
    if (rows_needs_relayout(a.X, x_dtype, a.x_kmajor ? TL_X_K_MAJOR : TL_X_ROW_MAJOR, a.ldx, a.M)) {
        const int mtile = rows_mtile(x_dtype);
        const int64_t ldm = round_up(a.M, mtile);
        const int64_t need = (int64_t)a.K * ldm * (x_dtype == TL_F16 ? 2 : 4);
        if (!workspace || workspace_bytes < need)
            return fail(TL_ERR_SIZE, "workspace has %lld bytes, %lld needed", (long long)workspace_bytes, (long long)need);
        if (reinterpret_cast<uintptr_t>(workspace) % 16) return fail(TL_ERR_ALIGN, "workspace must be 16-byte aligned");
        dim3 tgrid((unsigned)ceil_div(a.K, 64), (unsigned)(ldm / 64));
        if (x_dtype == TL_F16 && !a.x_kmajor && a.K % 8 == 0 && a.ldx % 8 == 0 && reinterpret_cast<uintptr_t>(a.X) % 16 == 0)
            hipLaunchKernelGGL(tl_relayout_rows_h, dim3((unsigned)ceil_div(a.K, 64), (unsigned)(ldm / 128)), dim3(256), 0, st,
                               static_cast<const __half*>(a.X), a.ldx, static_cast<__half*>(workspace), ldm, a.M, a.K);
        else if (x_dtype == TL_F16)
            hipLaunchKernelGGL(tl_relayout_x<__half>, tgrid, dim3(256), 0, st, static_cast<const __half*>(a.X), a.ldx, a.x_kmajor,
                               static_cast<__half*>(workspace), ldm, a.M, a.K);
        else
            hipLaunchKernelGGL(tl_relayout_x<float>, tgrid, dim3(256), 0, st, static_cast<const float*>(a.X), a.ldx, a.x_kmajor,
                               static_cast<float*>(workspace), ldm, a.M, a.K);
        a.X = workspace;
        a.ldx = ldm;
        a.x_kmajor = 1;
    }
    // the kernel keeps a thread's byte offsets inside one activation tile in 32 bits
    if ((int64_t)kTileSlots * a.ldx * (x_dtype == TL_F16 ? 2 : 4) >= (int64_t)1 << 32)
        return fail(TL_ERR_ARG, "activation leading dimension %lld is too large for one call; split the rows", (long long)a.ldx);
    // room for partial sums, if the caller's workspace reaches that far (without it every output tile
    // simply gets a workgroup of its own)
    void* partial = nullptr;
    int64_t partial_bytes = 0;
    if (workspace && workspace_bytes >= image + kRowsPartialBytes) {
        partial = static_cast<unsigned char*>(workspace) + image;
        partial_bytes = workspace_bytes - image;
    }
    if (a.gated) {  // one weight with (gate, up) column pairs: the plain kernel with the pair epilogue
        if (gated) return fail(TL_ERR_ARG, "the two-weight kernel has its own gate");
        return x_dtype == TL_F16 ? launch_rows_t<__half, 4, false, true>(a, partial, partial_bytes, st)
                                 : launch_rows_t<float, 2, false, true>(a, partial, partial_bytes, st);
    }
    if (x_dtype == TL_F16)
        return gated ? launch_rows_t<__half, 4, true>(a, partial, partial_bytes, st) : launch_rows_t<__half, 4, false>(a, partial, partial_bytes, st);
    return gated ? launch_rows_t<float, 2, true>(a, partial, partial_bytes, st) : launch_rows_t<float, 2, false>(a, partial, partial_bytes, st);
}

}  // namespace

int tl::launch_rows(KernelArgs a, int x_dtype, void* workspace, int64_t workspace_bytes, bool gated, hipStream_t st)
{
    return rows_launch(a, x_dtype, workspace, workspace_bytes, gated, st);
}

extern "C" int tl_mlp_gate_up(const tl_layout_header* gate_header, const void* gate_blob_dev,
                              const tl_layout_header* up_header, const void* up_blob_dev,
                              const void* X, int x_dtype, int x_layout, int64_t ldx, int64_t M,
                              void* H, int h_dtype, int64_t ldh,
                              const void* gate_scale, const void* up_scale, int scale_dtype,
                              int activation,
                              void* workspace, int64_t workspace_bytes, void* stream)
{
    if (int rc = check_header(gate_header)) return rc;
    if (int rc = check_header(up_header)) return rc;
    if (gate_header->inners != up_header->inners || gate_header->columns != up_header->columns ||
        gate_header->tile_rows != up_header->tile_rows)
        return fail(TL_ERR_SHAPE, "gate and up weights must share K, N and tile height");
    if (activation != TL_ACT_SILU_GATE) return fail(TL_ERR_UNSUPPORTED, "activation code %d (only TL_ACT_SILU_GATE)", activation);
    if (!up_blob_dev || reinterpret_cast<uintptr_t>(up_blob_dev) % 256) return fail(TL_ERR_ALIGN, "up blob null or not 256-byte aligned");
    if (int rc = check_io(gate_blob_dev, X, H, x_dtype, x_layout, ldx, M, h_dtype, ldh, gate_scale, scale_dtype, gate_header)) return rc;
    if ((gate_scale == nullptr) != (up_scale == nullptr)) return fail(TL_ERR_ARG, "pass both scales or neither");
    if (M <= kSmallMaxM) return fail(TL_ERR_UNSUPPORTED, "fused gate/up needs M > %d; use two tl_spmm calls below that", kSmallMaxM);
    KernelArgs a;
    std::memset(&a, 0, sizeof(a));
    a.w0 = weight_ptrs(gate_header, gate_blob_dev, gate_scale);
    a.w1 = weight_ptrs(up_header, up_blob_dev, up_scale);
    a.X = X; a.Y = H;
    a.ldx = ldx; a.ldy = ldh;
    a.NB = (int)gate_header->n_blocks;
    a.M = (int)M; a.N = (int)gate_header->columns; a.K = (int)gate_header->inners; a.T = (int)gate_header->n_tiles;
    a.tile_rows = (int)gate_header->tile_rows;
    a.x_f16 = x_dtype == TL_F16; a.x_kmajor = x_layout == TL_X_K_MAJOR; a.y_f16 = h_dtype == TL_F16; a.scale_f16 = scale_dtype == TL_F16;
    a.one = 1.0f;
    if (int rc = launch_rows(a, x_dtype, workspace, workspace_bytes, true, static_cast<hipStream_t>(stream))) return rc;
    return finish_launch();
}

