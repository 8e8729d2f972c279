// gfx950 kernels and launchers of libternary_spmm: Y = (X * W) * scale for a ternary W
// held in the wave-tiled CSC blob (see tl_layout.cpp for the format).
//
// Two kernels replace the reference's pair
// (ternaryLLM_GPU/csrc/ter_spmm_kernel.cuh:24-78 SpMV, :106-308 SpMM):
//
//   tl_spmm_block  M <= 48 (decode and small batches).  A workgroup owns a block of 16
//                  columns over all of K and streams its chunks and the matching
//                  activation rows through LDS; LPC lanes share a column and split
//                  each run, four dwords = sixteen 8-bit row indices per lane; every
//                  index is one LDS gather and one fp32 add per activation row; the
//                  LPC partial sums are folded with cross-lane shuffles.
//   tl_spmm_rows   larger M (prefill).  Lanes own activation rows, a wave owns C
//                  output columns, so an index is wave-uniform: it is read through
//                  the scalar path once and serves 64*R rows; the activation tile
//                  is staged in LDS as [slot][row] so the gather of a wave is one
//                  contiguous, conflict-free LDS read.
//
// Only additions and subtractions touch the data; fp32 accumulation throughout.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <cstring>

#include "tl_common.h"

using namespace tl;

namespace {

// Loads through this pointer type may use the scalar (constant) path when the address is wave-uniform.
typedef const __attribute__((address_space(4))) uint32_t* const_u32_ptr;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));  // one 16-byte chunk in registers
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wold-style-cast"
__device__ __forceinline__ const_u32_ptr as_const(const uint32_t* p) { return (const_u32_ptr)p; }
#pragma clang diagnostic pop

struct WeightPtrs {
    const uint32_t* chunkstart;  // [NB * T + 1], dword offsets into stream
    const uint32_t* stream;      // chunks: 64 descriptors + runs of four 8-bit rows per dword
    const void* scale;           // per-column factor or null
};

struct KernelArgs {
    WeightPtrs w0;
    WeightPtrs w1;  // second weight set of the fused gate/up kernel
    const void* X;
    void* Y;
    long long ldx, ldy;
    int M, N, K, T, tile_rows, NB;
    int x_f16, x_kmajor, y_f16, scale_f16;
    int tiles_per_group;  // small-M kernel: activation tiles staged per pass
    unsigned tile_magic;  // ceil(2^32 / tile_rows): k / tile_rows == (k * tile_magic) >> 32 for every k < 2^24
    float one;  // 1.0f, passed in so that the fp16 -> fp32 accumulate stays a single mixed-precision fma
};

__device__ __forceinline__ float load_scale(const void* scale, int is_f16, int n)
{
    if (!scale) return 1.0f;
    return is_f16 ? __half2float(static_cast<const __half*>(scale)[n]) : static_cast<const float*>(scale)[n];
}

__device__ __forceinline__ void store_out(void* Y, int is_f16, long long off, float v)
{
    if (is_f16) static_cast<__half*>(Y)[off] = __float2half(v);
    else static_cast<float*>(Y)[off] = v;
}

__device__ __forceinline__ float silu(float g) { return g / (1.0f + __expf(-g)); }

__device__ __forceinline__ int run_pos_dwords(uint32_t d) { return (int)(((d & 0xffu) + 3u) >> 2); }
__device__ __forceinline__ int run_neg_dwords(uint32_t d) { return (int)((((d >> 8) & 0xffu) + 3u) >> 2); }

// ---------------------------------------------------------------------------
// Small-M kernel: one workgroup per (column block, range of tiles, block of rows).
// ---------------------------------------------------------------------------
template <int MT>
__device__ __forceinline__ void gather_add(float (&acc)[MT], const float* __restrict__ xt, uint32_t word, float sign)
{
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        const uint32_t r = (word >> (8 * b)) & 0xffu;
        const float* row = xt + r * MT;
        if constexpr (MT % 4 == 0) {
#pragma unroll
            for (int m = 0; m < MT; m += 4) {
                const float4 v = *reinterpret_cast<const float4*>(row + m);
                acc[m + 0] = fmaf(v.x, sign, acc[m + 0]);
                acc[m + 1] = fmaf(v.y, sign, acc[m + 1]);
                acc[m + 2] = fmaf(v.z, sign, acc[m + 2]);
                acc[m + 3] = fmaf(v.w, sign, acc[m + 3]);
            }
        } else if constexpr (MT == 2) {
            const float2 v = *reinterpret_cast<const float2*>(row);
            acc[0] = fmaf(v.x, sign, acc[0]);
            acc[1] = fmaf(v.y, sign, acc[1]);
        } else {
            acc[0] = fmaf(row[0], sign, acc[0]);
        }
    }
}

constexpr int kSmallStreamBytes = 32 * 1024;  // LDS for the chunks of one group of tiles
constexpr int kSmallXBytes = 32 * 1024;       // LDS for the activation rows of one group of tiles
constexpr int kBlockThreads = 512;            // workgroup of the small-M kernel: 32 lanes for each of its 16 columns
constexpr int kMaxChunkBytes = (TL_BLOCK_COLUMNS + TL_BLOCK_COLUMNS * 128) * 4;  // a chunk of all-non-zero columns

// Sizes of one group of tiles for a workgroup of NT threads with MT activation rows: what one
// thread keeps in registers while a group is in flight is bounded (256 bytes of stream and a
// few 16-byte activation vectors), and the whole group fits the two LDS areas.
template <int MT, int NT>
struct BlockShape {
    static constexpr int kStreamCap = (NT * 256 < kMaxChunkBytes ? kMaxChunkBytes + 240
                                       : (NT * 256 > kSmallStreamBytes ? kSmallStreamBytes : NT * 256)) / 16 * 16;
    static constexpr int kVectors = (kStreamCap / 16 + NT - 1) / NT;
    static constexpr int kByLds = kSmallXBytes / (kTileSlots * MT * 4);
    static constexpr int kTiles = kByLds < 32 ? kByLds : 32;                         // tiles per group at most
    // 16-byte activation vectors per row of a group (fp32: 4 values each; +2 for the ragged ends)
    static constexpr int kRowVectors = (kTiles * kMaxTileRows + 3) / 4 + 2;
    static constexpr int kXVectors = MT * ((kRowVectors + NT - 1) / NT);             // per thread
};

// One workgroup owns one block of 16 columns (and MT activation rows) over all of K.
// K is walked in groups of tiles.  For a group, the chunks are one contiguous piece of the
// stream; it and the activation rows of the same tiles (contiguous in K) travel
// global -> registers one group ahead as 16-byte vectors, all in flight before anything
// waits, then registers -> LDS (activations as fp32 [slot][row]).
// From LDS, 32 lanes share a column: TP tiles are worked on side by side, LW lanes per run,
// one dword (four row indices) per lane and pass; an index is one LDS gather and one fp32
// add per activation row.  The 32 partial sums of a column are folded with cross-lane
// shuffles.  No workgroup depends on another.
// X must be row-major with 16-byte aligned rows (the launcher repacks anything else).
template <int MT, int LW, bool XF16>
__global__ __launch_bounds__(kBlockThreads) void tl_spmm_block(KernelArgs a)
{
    extern __shared__ __align__(16) unsigned char lds[];
    constexpr int NT = kBlockThreads;
    constexpr int LPC = NT / TL_BLOCK_COLUMNS;  // lanes per column: TP tiles in parallel x LW lanes per run
    constexpr int TP = LPC / LW;
    using Shape = BlockShape<MT, NT>;
    constexpr int NV = Shape::kVectors;    // 16-byte stream vectors per thread and group
    constexpr int NXV = Shape::kXVectors;  // 16-byte activation vectors per thread and group
    constexpr int VE = XF16 ? 8 : 4;       // activation values per vector
    constexpr int XPR = NXV / MT;          // vectors per thread and row
    const int tid = threadIdx.x;
    const int nb = blockIdx.x, m0 = blockIdx.y * MT;
    const int TG = a.tiles_per_group;  // <= Shape::kTiles, and TG chunks fit Shape::kStreamCap
    float* xs = reinterpret_cast<float*>(lds);                                   // [TG * 256 slots][MT]
    uint32_t* buf = reinterpret_cast<uint32_t*>(lds + kSmallXBytes);             // chunk copy
    uint32_t* cst = reinterpret_cast<uint32_t*>(lds + kSmallXBytes + kSmallStreamBytes);  // chunk starts inside buf
    const_u32_ptr cs = as_const(a.w0.chunkstart) + (size_t)nb * a.T;
    const unsigned char* Xb = static_cast<const unsigned char*>(a.X);
    constexpr int ES = XF16 ? 2 : 4;

    // Slots that staging never writes (rows past the tile height, the sentinel slot) must read as zero.
    for (int e = tid; e < kSmallXBytes / 16; e += NT) reinterpret_cast<u32x4*>(xs)[e] = u32x4{0u, 0u, 0u, 0u};

    u32x4 cv[NV];
    u32x4 xv[NXV];
    // global -> registers for the tiles [t, t + nt)
    auto prefetch = [&](int t, int nt) {
        const uint32_t s_lo = cs[t];
        const int nvec = (int)(cs[t + nt] - s_lo) / 4;
        const u32x4* src = reinterpret_cast<const u32x4*>(a.w0.stream + s_lo);
#pragma unroll
        for (int i = 0; i < NV; ++i) cv[i] = src[min(tid + i * NT, nvec - 1)];  // past the end: last vector again, never stored
        const int k_lo = t * a.tile_rows, k_hi = min(a.K, (t + nt) * a.tile_rows);
        const int v_lo = k_lo / VE, v_hi = (k_hi + VE - 1) / VE;  // vectors [v_lo, v_hi) of a row cover the group
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const int row = min(m0 + m, a.M - 1);  // rows past M re-read the last row; they are never stored to Y
#pragma unroll
            for (int i = 0; i < XPR; ++i) {
                const int v = min(v_lo + tid + i * NT, v_hi - 1);
                xv[m * XPR + i] = *reinterpret_cast<const u32x4*>(Xb + ((size_t)row * a.ldx + (size_t)v * VE) * ES);
            }
        }
    };
    // registers -> LDS
    auto commit = [&](int t, int nt) {
        const uint32_t s_lo = cs[t];
        const int nvec = (int)(cs[t + nt] - s_lo) / 4;
#pragma unroll
        for (int i = 0; i < NV; ++i)
            if (tid + i * NT < nvec) reinterpret_cast<u32x4*>(buf)[tid + i * NT] = cv[i];
        const int k_lo = t * a.tile_rows, k_hi = min(a.K, (t + nt) * a.tile_rows);
        const int v_lo = k_lo / VE, v_hi = (k_hi + VE - 1) / VE;
#pragma unroll
        for (int i = 0; i < XPR; ++i) {
            const int v = v_lo + tid + i * NT;
            if (v < v_hi) {
                int k = v * VE;
                int tile = (int)(((unsigned long long)(unsigned)k * a.tile_magic) >> 32);  // k / tile_rows
                int r = k - tile * a.tile_rows;
#pragma unroll
                for (int e = 0; e < VE; ++e) {
                    if (k >= k_lo && k < k_hi) {
                        float* dst = xs + (size_t)((tile - t) * kTileSlots + r) * MT;
#pragma unroll
                        for (int m = 0; m < MT; ++m) {
                            const uint32_t word = xv[m * XPR + i][XF16 ? e / 2 : e];
                            dst[m] = XF16 ? __half2float(__ushort_as_half((unsigned short)(e % 2 ? word >> 16 : word & 0xffffu)))
                                          : __uint_as_float(word);
                        }
                    }
                    ++k;
                    if (++r == a.tile_rows) { r = 0; ++tile; }
                }
            }
        }
        if (tid <= nt) cst[tid] = cs[t + tid] - s_lo;
    };

    const int col = tid / LPC, lig = tid % LPC;
    const int tp = lig / LW, lw = lig % LW;
    float acc[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[m] = 0.f;

    constexpr int TU = MT <= 2 ? 4 : (MT <= 8 ? 2 : 1);  // tiles of one lane whose LDS reads are issued together
    prefetch(0, min(TG, a.T));
    for (int t = 0; t < a.T; t += TG) {
        const int nt = min(TG, a.T - t);
        __syncthreads();  // the previous group has been consumed
        commit(t, nt);
        __syncthreads();
        if (t + TG < a.T) prefetch(t + TG, min(TG, a.T - t - TG));
        for (int tl0 = tp; tl0 < nt; tl0 += TP * TU) {
            uint32_t d[TU], w[TU];
            const uint32_t* run[TU];
#pragma unroll
            for (int u = 0; u < TU; ++u) {
                const int tl = tl0 + u * TP;
                const uint32_t* chunk = buf + cst[min(tl, nt - 1)];
                d[u] = tl < nt ? chunk[col] : 0u;  // tiles past the group: empty run
                run[u] = chunk + (d[u] >> 16);
            }
#pragma unroll
            for (int u = 0; u < TU; ++u)  // lanes past the run's end take an all-sentinel word: four gathers of zero
                w[u] = lw < run_pos_dwords(d[u]) + run_neg_dwords(d[u]) ? run[u][lw] : 0xffffffffu;
#pragma unroll
            for (int u = 0; u < TU; ++u) {
                const int pd = run_pos_dwords(d[u]), tot = pd + run_neg_dwords(d[u]);
                const float* xt = xs + (size_t)min(tl0 + u * TP, nt - 1) * kTileSlots * MT;
                gather_add<MT>(acc, xt, w[u], lw < pd ? 1.0f : -1.0f);
                for (int i = lw + LW; i < tot; i += LW)  // runs longer than the lane group
                    gather_add<MT>(acc, xt, run[u][i], i < pd ? 1.0f : -1.0f);
            }
        }
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) {
#pragma unroll
        for (int off = LPC / 2; off > 0; off >>= 1) acc[m] += __shfl_xor(acc[m], off, 64);
    }
    const int n = nb * TL_BLOCK_COLUMNS + col;
    if (lig == 0 && n < a.N) {
        const float s = load_scale(a.w0.scale, a.scale_f16, n);
#pragma unroll
        for (int m = 0; m < MT; ++m)
            if (m0 + m < a.M) store_out(a.Y, a.y_f16, (long long)(m0 + m) * a.ldy + n, acc[m] * s);
    }
}

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
    // Reads past the wave's piece stay inside the blob (it ends with spare bytes) and are never used.
    __device__ __forceinline__ void indices(WaveRuns<C>& r, uint32_t chunk) const
    {
        r.base = chunk + (r.d[0] >> 16);
#pragma unroll
        for (int ch = 0; ch < NPRE; ++ch) r.pre[ch] = stream[r.base + ch * 64 + lane];
    }
    __device__ __forceinline__ void prime(const WeightPtrs& w, int T, int n0, int lane_)
    {
        chunkstart = as_const(w.chunkstart) + (size_t)(n0 / TL_BLOCK_COLUMNS) * T;
        stream_c = as_const(w.stream);
        stream = w.stream;
        sub = n0 % TL_BLOCK_COLUMNS;
        lane = lane_;
        const uint32_t chunk0 = chunkstart[0];
        descriptors(nxt.d, chunk0);
        indices(nxt, chunk0);
        chunk1 = chunk2 = 0;
#pragma unroll
        for (int c = 0; c < C; ++c) d1[c] = 0;
        if (T > 1) {
            chunk1 = chunkstart[1];
            descriptors(d1, chunk1);
        }
        if (T > 2) chunk2 = chunkstart[2];
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
// A slot of the staged tile is 512 bytes for both activation types (256 fp16 rows / 128 fp32 rows).
// Its two halves are fetched with LDS "add-TID" reads: address = M0 + offset + 4 * lane, with
// M0 = slot * 512 set on the scalar unit, so no vector instruction is spent on addressing.  Lane l thus holds, for fp16, rows {2l, 2l+1} and {128+2l, 129+2l} of the row tile;
// for fp32, rows l and 64+l.  Per dword of four indices: one v_readlane (the dword sits in a lane of
// the chunk vector), scalar byte extraction, eight LDS reads, and 16 (fp16) or 8 (fp32) accumulating
// vector ops.  Two register sets alternate so that the reads of dword i + 1 are in flight while
// dword i is accumulated; LDS reads complete in issue order, so "lgkmcnt(8)" means everything but
// the eight reads issued last has arrived.
// The tile starts at LDS address 0 (the kernel has no other LDS; the launcher checks it), so
// M0 = slot * 512 = the index byte moved to bits 9..16: one shift and one mask per index.  The scalar
// op that prepares the next index sits between each write of M0 and the reads that use it (one wait
// state is required there); the last gap is filled by the loop counter's increment.
#define TL_ISSUE(W, X0, Y0, X1, Y1, X2, Y2, X3, Y3)                 \
    "s_lshl_b32 %[t], " W ", 9\n\t"                                  \
    "s_and_b32 m0, %[t], %[mk]\n\t"                                  \
    "s_lshl_b32 %[t], " W ", 1\n\t"                                  \
    "ds_read_addtid_b32 " X0 " offset:0\n\t"                         \
    "ds_read_addtid_b32 " Y0 " offset:256\n\t"                       \
    "s_and_b32 m0, %[t], %[mk]\n\t"                                  \
    "s_lshr_b32 %[t], " W ", 7\n\t"                                  \
    "ds_read_addtid_b32 " X1 " offset:0\n\t"                         \
    "ds_read_addtid_b32 " Y1 " offset:256\n\t"                       \
    "s_and_b32 m0, %[t], %[mk]\n\t"                                  \
    "s_lshr_b32 %[t], " W ", 15\n\t"                                 \
    "ds_read_addtid_b32 " X2 " offset:0\n\t"                         \
    "ds_read_addtid_b32 " Y2 " offset:256\n\t"                       \
    "s_and_b32 m0, %[t], %[mk]\n\t"                                  \
    "s_add_u32 %[i], %[i], 1\n\t"                                    \
    "ds_read_addtid_b32 " X3 " offset:0\n\t"                         \
    "ds_read_addtid_b32 " Y3 " offset:256\n\t"

// fp16: a dword holds two rows; the mixed-precision fma converts and accumulates in one op
#define TL_FMA_H(X, Y)                                                                   \
    "v_fma_mix_f32 %[c0], " X ", %[sg], %[c0] op_sel_hi:[1,0,0]\n\t"                      \
    "v_fma_mix_f32 %[c1], " X ", %[sg], %[c1] op_sel:[1,0,0] op_sel_hi:[1,0,0]\n\t"       \
    "v_fma_mix_f32 %[c2], " Y ", %[sg], %[c2] op_sel_hi:[1,0,0]\n\t"                      \
    "v_fma_mix_f32 %[c3], " Y ", %[sg], %[c3] op_sel:[1,0,0] op_sel_hi:[1,0,0]\n\t"
#define TL_FMA_F(X, Y)                              \
    "v_fma_f32 %[c0], " X ", %[sg], %[c0]\n\t"       \
    "v_fma_f32 %[c1], " Y ", %[sg], %[c1]\n\t"

#define TL_SET_A "%[a0]", "%[b0]", "%[a1]", "%[b1]", "%[a2]", "%[b2]", "%[a3]", "%[b3]"
#define TL_SET_B "%[p0]", "%[q0]", "%[p1]", "%[q1]", "%[p2]", "%[q2]", "%[p3]", "%[q3]"
#define TL_ISSUE_SET(W, ...) TL_ISSUE(W, __VA_ARGS__)
#define TL_ACC_A(F) F("%[a0]", "%[b0]") F("%[a1]", "%[b1]") F("%[a2]", "%[b2]") F("%[a3]", "%[b3]")
#define TL_ACC_B(F) F("%[p0]", "%[q0]") F("%[p1]", "%[q1]") F("%[p2]", "%[q2]") F("%[p3]", "%[q3]")

#define TL_RUN_LOOP(F)                                   \
    "v_readlane_b32 %[w], %[v], %[i]\n\t"                \
    TL_ISSUE_SET("%[w]", TL_SET_A)                       \
    "Ltl_loop%=:\n\t"                                    \
    "s_cmp_lt_u32 %[i], %[hi]\n\t"                       \
    "s_cbranch_scc0 Ltl_lastA%=\n\t"                     \
    "v_readlane_b32 %[w], %[v], %[i]\n\t"                \
    TL_ISSUE_SET("%[w]", TL_SET_B)                       \
    "s_waitcnt lgkmcnt(8)\n\t"                           \
    TL_ACC_A(F)                                          \
    "s_cmp_lt_u32 %[i], %[hi]\n\t"                       \
    "s_cbranch_scc0 Ltl_lastB%=\n\t"                     \
    "v_readlane_b32 %[w], %[v], %[i]\n\t"                \
    TL_ISSUE_SET("%[w]", TL_SET_A)                       \
    "s_waitcnt lgkmcnt(8)\n\t"                           \
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
// sign: acc += sgn * (rows of the tile at each index).  lo < hi.
template <typename XT, int R>
__device__ __forceinline__ void rows_run(float (&acc)[R], uint32_t v, int lo, int hi, float sgn_one)
{
    uint32_t a0, b0, a1, b1, a2, b2, a3, b3, p0, q0, p1, q1, p2, q2, p3, q3, w, t;
    uint32_t i = (uint32_t)lo;
    if constexpr (sizeof(XT) == 2) {
        static_assert(R == 4, "fp16 row tiles hold 4 rows per lane");
        asm volatile(TL_RUN_LOOP(TL_FMA_H)
                     : [c0] "+v"(acc[0]), [c1] "+v"(acc[1]), [c2] "+v"(acc[2]), [c3] "+v"(acc[3]), [i] "+s"(i),
                       [a0] "=&v"(a0), [b0] "=&v"(b0), [a1] "=&v"(a1), [b1] "=&v"(b1), [a2] "=&v"(a2), [b2] "=&v"(b2),
                       [a3] "=&v"(a3), [b3] "=&v"(b3), [p0] "=&v"(p0), [q0] "=&v"(q0), [p1] "=&v"(p1), [q1] "=&v"(q1),
                       [p2] "=&v"(p2), [q2] "=&v"(q2), [p3] "=&v"(p3), [q3] "=&v"(q3), [w] "=&s"(w), [t] "=&s"(t)
                     : [v] "v"(v), [hi] "s"((uint32_t)hi), [mk] "s"(0x1fe00u), [sg] "s"(sgn_one)
                     : "m0", "scc", "memory");
    } else {
        static_assert(R == 2, "fp32 row tiles hold 2 rows per lane");
        asm volatile(TL_RUN_LOOP(TL_FMA_F)
                     : [c0] "+v"(acc[0]), [c1] "+v"(acc[1]), [i] "+s"(i),
                       [a0] "=&v"(a0), [b0] "=&v"(b0), [a1] "=&v"(a1), [b1] "=&v"(b1), [a2] "=&v"(a2), [b2] "=&v"(b2),
                       [a3] "=&v"(a3), [b3] "=&v"(b3), [p0] "=&v"(p0), [q0] "=&v"(q0), [p1] "=&v"(p1), [q1] "=&v"(q1),
                       [p2] "=&v"(p2), [q2] "=&v"(q2), [p3] "=&v"(p3), [q3] "=&v"(q3), [w] "=&s"(w), [t] "=&s"(t)
                     : [v] "v"(v), [hi] "s"((uint32_t)hi), [mk] "s"(0x1fe00u), [sg] "s"(sgn_one)
                     : "m0", "scc", "memory");
    }
}

// One 64-dword chunk of the wave's piece: dword i of the piece sits in lane i - cb of `v`
// and is broadcast from there, so its four row indices are wave-uniform.
template <typename XT, int R, int C>
__device__ __forceinline__ void rows_chunk(float (&acc)[C][R], const int (&pb)[C], const int (&pe)[C], const int (&ne)[C],
                                           uint32_t v, int cb, float one)
{
#pragma unroll
    for (int c = 0; c < C; ++c) {
        int lo = max(pb[c], cb) - cb, hi = min(pe[c], cb + 64) - cb;
        if (lo < hi) rows_run<XT, R>(acc[c], v, lo, hi, one);
        lo = max(pe[c], cb) - cb;
        hi = min(ne[c], cb + 64) - cb;
        if (lo < hi) rows_run<XT, R>(acc[c], v, lo, hi, -one);
    }
}

template <typename XT, int R, int C>
__device__ __forceinline__ void rows_consume(float (&acc)[C][R], const WaveRuns<C>& r, const uint32_t* __restrict__ idx,
                                             int lane, float one)
{
    int pb[C], pe[C], ne[C];
#pragma unroll
    for (int c = 0; c < C; ++c) {
        pb[c] = (int)((r.d[c] >> 16) - (r.d[0] >> 16));
        pe[c] = pb[c] + run_pos_dwords(r.d[c]);
        ne[c] = pe[c] + run_neg_dwords(r.d[c]);
    }
    const int total = ne[C - 1];
#pragma unroll
    for (int ch = 0; ch < NPRE; ++ch)
        if (ch * 64 < total) rows_chunk<XT, R, C>(acc, pb, pe, ne, r.pre[ch], ch * 64, one);
    for (int cb = NPRE * 64; cb < total; cb += 64)  // pieces longer than the prefetch window: fetched on demand
        rows_chunk<XT, R, C>(acc, pb, pe, ne, idx[r.base + cb + lane], cb, one);
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

template <typename XT, int R, int C, int WAVES, bool GATED>
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
    int id = (int)blockIdx.x;
    const int per_xcd = total / 8;
    if (id < per_xcd * 8) id = (id & 7) * per_xcd + (id >> 3);
    const int m0 = (id / n_col_tiles) * MTILE;
    const int n0 = (id % n_col_tiles) * (WAVES * C) + wave * C;
    const bool wave_live = n0 < a.N;                                       // uniform; then n0 lies inside a stored column block
    const unsigned char* __restrict__ XTr = static_cast<const unsigned char*>(a.X);  // [K][ldx] of XT, m contiguous

    float acc[C][R];
    float acc2[GATED ? C : 1][R];
#pragma unroll
    for (int c = 0; c < C; ++c)
#pragma unroll
        for (int j = 0; j < R; ++j) {
            acc[c][j] = 0.f;
            if (GATED) acc2[GATED ? c : 0][j] = 0.f;
        }

    // Slot 255 is what padding bytes address: zero it once, staging never writes it.
    for (int e = threadIdx.x; e < MTILE; e += NT) tile[kSentinel * MTILE + e] = XT(0.0f);

    // The next activation tile travels global -> registers while the current one is consumed.
    u32x4 pf[PER];
    RunFetcher<C> f0, f1;
    if (wave_live) {
        f0.prime(a.w0, a.T, n0, lane);
        if constexpr (GATED) f1.prime(a.w1, a.T, n0, lane);
    }
    uint32_t voff[PER];
    const int last_rows = a.K - (a.T - 1) * a.tile_rows;
    const size_t tile_stride = (size_t)a.tile_rows * a.ldx * sizeof(XT);  // bytes between the first rows of two tiles
    const unsigned char* __restrict__ col0 = XTr + (size_t)m0 * sizeof(XT);
    stage_offsets<XT, CHUNKS, NT, PER>(voff, a, a.T > 1 ? a.tile_rows : last_rows);
    tile_to_regs<PER>(pf, col0, voff);
    for (int t = 0; t < a.T; ++t) {
        __syncthreads();  // every wave is done with the previous tile
        regs_to_lds<CHUNKS, NT, PER>(pf, smem, a, t);
        __syncthreads();
        if (t + 1 < a.T) {
            if (t + 2 == a.T && last_rows != a.tile_rows) stage_offsets<XT, CHUNKS, NT, PER>(voff, a, last_rows);
            tile_to_regs<PER>(pf, col0 + (size_t)(t + 1) * tile_stride, voff);
        }
        if (wave_live) {
            f0.advance(t, a.T);
            if constexpr (GATED) f1.advance(t, a.T);
            rows_consume<XT, R, C>(acc, f0.cur, a.w0.stream, lane, a.one);
            if constexpr (GATED) rows_consume<XT, R, C>(acc2, f1.cur, a.w1.stream, lane, a.one);
        }
    }

#pragma unroll
    for (int c = 0; c < C; ++c) {
        const int n = n0 + c;
        if (n >= a.N) continue;
        const float s = load_scale(a.w0.scale, a.scale_f16, n);
        const float s2 = GATED ? load_scale(a.w1.scale, a.scale_f16, n) : 1.0f;
#pragma unroll
        for (int j = 0; j < R; ++j) {
            // rows of a lane: see rows_add4
            const int m = m0 + (sizeof(XT) == 2 ? (j >> 1) * 128 + 2 * lane + (j & 1) : j * 64 + lane);
            if (m >= a.M) continue;
            float v = acc[c][j] * s;
            if constexpr (GATED) v = silu(v) * (acc2[GATED ? c : 0][j] * s2);
            store_out(a.Y, a.y_f16, (long long)m * a.ldy + n, v);
        }
    }
}

// ---------------------------------------------------------------------------
// Host side.
// ---------------------------------------------------------------------------
int check_header(const tl_layout_header* h)
{
    if (!h) return fail(TL_ERR_ARG, "layout header is null");
    if (h->magic != TL_LAYOUT_MAGIC || h->version != TL_LAYOUT_VERSION) return fail(TL_ERR_FORMAT, "bad layout magic/version");
    if (h->tile_rows == 0 || h->tile_rows > (uint32_t)kMaxTileRows || h->n_tiles != (uint32_t)ceil_div(h->inners, h->tile_rows) ||
        h->n_blocks != (uint32_t)ceil_div(h->columns, TL_BLOCK_COLUMNS) || h->max_chunk_dwords < TL_BLOCK_COLUMNS ||
        (int64_t)h->max_chunk_dwords * 4 > kMaxChunkBytes + 16)
        return fail(TL_ERR_FORMAT, "layout header geometry is inconsistent");
    return TL_OK;
}

int check_dtype(int d, const char* what)
{
    if (d != TL_F32 && d != TL_F16) return fail(TL_ERR_DTYPE, "%s dtype code %d unknown", what, d);
    return TL_OK;
}

constexpr int kSmallMaxM = 48;       // above this the row-parallel kernel takes over
constexpr int kRowsWaves = 16;
constexpr int kRowsCols = 4;

inline int rows_mtile(int x_dtype) { return x_dtype == TL_F16 ? 256 : 128; }

int env_int(const char* name, int fallback)
{
    const char* v = std::getenv(name);
    return v && *v ? std::atoi(v) : fallback;
}

WeightPtrs weight_ptrs(const tl_layout_header* h, const void* blob_dev, const void* scale)
{
    const unsigned char* b = static_cast<const unsigned char*>(blob_dev);
    WeightPtrs w;
    w.chunkstart = reinterpret_cast<const uint32_t*>(b + h->off_chunkstart);
    w.stream = reinterpret_cast<const uint32_t*>(b + h->off_stream);
    w.scale = scale;
    return w;
}

template <typename KernelT>
int raise_lds_limit(KernelT kernel, size_t bytes)
{
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e != hipSuccess) return fail(TL_ERR_LAUNCH, "hipFuncSetAttribute(%zu bytes of LDS): %s", bytes, hipGetErrorString(e));
    return TL_OK;
}

template <int MT, int LW, bool XF16>
int launch_block_kernel(KernelArgs a, const tl_layout_header* h, hipStream_t st)
{
    using Shape = BlockShape<MT, kBlockThreads>;
    const int by_stream = (int)(Shape::kStreamCap / ((int64_t)h->max_chunk_dwords * 4));
    a.tiles_per_group = std::max(1, std::min(std::min(Shape::kTiles, by_stream), 255));
    a.tile_magic = (unsigned)(((1ull << 32) + h->tile_rows - 1) / h->tile_rows);
    const size_t lds = kSmallXBytes + kSmallStreamBytes + 1024;
    auto kernel = tl_spmm_block<MT, LW, XF16>;
    static bool raised = false;  // per instantiation; a repeated or racing call is harmless
    if (!raised) {
        if (int rc = raise_lds_limit(kernel, lds)) return rc;
        raised = true;
    }
    dim3 grid((unsigned)a.NB, (unsigned)ceil_div(a.M, MT));
    hipLaunchKernelGGL(kernel, grid, dim3(kBlockThreads), lds, st, a);
    return TL_OK;
}

template <int MT>
int launch_small_lpc(const KernelArgs& a, const tl_layout_header* h, int lpc, hipStream_t st)
{
    if (a.x_f16) {
        switch (lpc) {
            case 8: return launch_block_kernel<MT, 8, true>(a, h, st);
            case 16: return launch_block_kernel<MT, 16, true>(a, h, st);
            default: return launch_block_kernel<MT, 32, true>(a, h, st);
        }
    }
    switch (lpc) {
        case 8: return launch_block_kernel<MT, 8, false>(a, h, st);
        case 16: return launch_block_kernel<MT, 16, false>(a, h, st);
        default: return launch_block_kernel<MT, 32, false>(a, h, st);
    }
}

// Row-major activations with 16-byte aligned rows are read in place; anything else
// (K-major, odd leading dimension, odd base address) is first repacked into the workspace.
inline bool small_needs_repack(const void* X, int x_dtype, int x_layout, int64_t ldx, int64_t K)
{
    const int es = x_dtype == TL_F16 ? 2 : 4;
    // K must be whole vectors too: the kernel reads 16 bytes at a time and must not run past a row's end
    return x_layout != TL_X_ROW_MAJOR || (ldx * es) % 16 != 0 || (K * es) % 16 != 0 || reinterpret_cast<uintptr_t>(X) % 16 != 0;
}
inline int64_t small_repack_bytes(const tl_layout_header* h, int64_t M, int x_dtype)
{
    // rows padded to a multiple of 8 values plus one spare vector: the kernel reads whole vectors
    return M * (round_up(h->inners, 8) + 8) * (x_dtype == TL_F16 ? 2 : 4);
}

template <typename T>
__global__ __launch_bounds__(256) void tl_repack_rows(const T* __restrict__ X, long long ldx, int kmajor, T* __restrict__ out,
                                                      long long ldo, int M, int K)
{
    const long long i = blockIdx.x * 256ll + threadIdx.x;
    if (i >= (long long)M * ldo) return;
    const int m = (int)(i / ldo), k = (int)(i % ldo);
    out[i] = k < K ? (kmajor ? X[(long long)k * ldx + m] : X[(long long)m * ldx + k]) : T(0.0f);
}

int launch_small(KernelArgs a, const tl_layout_header* h, int x_dtype, void* workspace, int64_t workspace_bytes, hipStream_t st)
{
    int mt = 1;
    while (mt < a.M && mt < 32) mt *= 2;
    // lanes per run: one dword per lane should cover a typical run in one pass
    const double mean_run = h->mean_run_dwords_x16 / 16.0;
    int lpc = 8;
    while (lpc < 32 && lpc < mean_run) lpc *= 2;
    lpc = env_int("TL_LPC", lpc);
    if (lpc != 8 && lpc != 16 && lpc != 32) return fail(TL_ERR_ARG, "TL_LPC=%d (8, 16 or 32 expected)", lpc);
    if (small_needs_repack(a.X, x_dtype, a.x_kmajor ? TL_X_K_MAJOR : TL_X_ROW_MAJOR, a.ldx, a.K)) {
        const int64_t need = small_repack_bytes(h, a.M, x_dtype);
        if (!workspace || workspace_bytes < need)
            return fail(TL_ERR_SIZE, "workspace has %lld bytes, %lld needed", (long long)workspace_bytes, (long long)need);
        if (reinterpret_cast<uintptr_t>(workspace) % 16) return fail(TL_ERR_ALIGN, "workspace must be 16-byte aligned");
        const long long ldo = round_up(a.K, 8) + 8;
        const unsigned blocks = (unsigned)ceil_div((int64_t)a.M * ldo, 256);
        if (x_dtype == TL_F16)
            hipLaunchKernelGGL(tl_repack_rows<__half>, dim3(blocks), dim3(256), 0, st, static_cast<const __half*>(a.X), a.ldx,
                               a.x_kmajor, static_cast<__half*>(workspace), ldo, a.M, a.K);
        else
            hipLaunchKernelGGL(tl_repack_rows<float>, dim3(blocks), dim3(256), 0, st, static_cast<const float*>(a.X), a.ldx,
                               a.x_kmajor, static_cast<float*>(workspace), ldo, a.M, a.K);
        a.X = workspace;
        a.ldx = ldo;
        a.x_kmajor = 0;
    }
    switch (mt) {
        case 1: return launch_small_lpc<1>(a, h, lpc, st);
        case 2: return launch_small_lpc<2>(a, h, lpc, st);
        case 4: return launch_small_lpc<4>(a, h, lpc, st);
        case 8: return launch_small_lpc<8>(a, h, lpc, st);
        case 16: return launch_small_lpc<16>(a, h, lpc, st);
        default: return launch_small_lpc<32>(a, h, lpc, st);
    }
}

template <typename XT, int R, bool GATED>
int launch_rows_t(const KernelArgs& a, hipStream_t st)
{
    constexpr int MTILE = 64 * R;
    const size_t lds = (size_t)kTileSlots * MTILE * sizeof(XT);
    auto kernel = tl_spmm_rows<XT, R, kRowsCols, kRowsWaves, GATED>;
    static bool raised = false;  // per instantiation; a repeated call is harmless
    if (!raised) {
        // the kernel addresses its activation tile from LDS offset 0: it must own no static LDS
        hipFuncAttributes attr;
        if (hipFuncGetAttributes(&attr, reinterpret_cast<const void*>(kernel)) != hipSuccess || attr.sharedSizeBytes != 0)
            return fail(TL_ERR_LAUNCH, "row kernel was built with static LDS; its tile would not start at offset 0");
        if (int rc = raise_lds_limit(kernel, lds)) return rc;
        raised = true;
    }
    dim3 grid((unsigned)(ceil_div(a.N, kRowsWaves * kRowsCols) * ceil_div(a.M, MTILE)));  // 1-D: the kernel maps ids to tiles
    hipLaunchKernelGGL(kernel, grid, dim3(kRowsWaves * 64), lds, st, a);
    return TL_OK;
}

// K-major activations whose leading dimension is a whole number of row tiles (and 16-byte aligned)
// are what the row-parallel kernel reads directly; anything else goes through the re-layout pre-pass.
inline bool rows_needs_relayout(const void* X, int x_dtype, int x_layout, int64_t ldx, int64_t M)
{
    const int mtile = rows_mtile(x_dtype);
    return x_layout != TL_X_K_MAJOR || ldx % mtile != 0 || ldx < round_up(M, mtile) || reinterpret_cast<uintptr_t>(X) % 16 != 0;
}

// Runs the re-layout pre-pass into `workspace` when needed, then the row-parallel kernel.
int launch_rows(KernelArgs a, int x_dtype, void* workspace, int64_t workspace_bytes, bool gated, hipStream_t st)
{
    if (rows_needs_relayout(a.X, x_dtype, a.x_kmajor ? TL_X_K_MAJOR : TL_X_ROW_MAJOR, a.ldx, a.M)) {
        const int mtile = rows_mtile(x_dtype);
        const int64_t ldm = round_up(a.M, mtile);
        const int64_t need = (int64_t)a.K * ldm * (x_dtype == TL_F16 ? 2 : 4);
        if (!workspace || workspace_bytes < need)
            return fail(TL_ERR_SIZE, "workspace has %lld bytes, %lld needed", (long long)workspace_bytes, (long long)need);
        if (reinterpret_cast<uintptr_t>(workspace) % 16) return fail(TL_ERR_ALIGN, "workspace must be 16-byte aligned");
        dim3 tgrid((unsigned)ceil_div(a.K, 64), (unsigned)(ldm / 64));
        if (x_dtype == TL_F16)
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
    if (x_dtype == TL_F16) return gated ? launch_rows_t<__half, 4, true>(a, st) : launch_rows_t<__half, 4, false>(a, st);
    return gated ? launch_rows_t<float, 2, true>(a, st) : launch_rows_t<float, 2, false>(a, st);
}

int finish_launch()
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(TL_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString(e));
    return TL_OK;
}

int check_io(const void* blob_dev, const void* X, void* Y, int x_dtype, int x_layout, int64_t ldx, int64_t M, int y_dtype,
             int64_t ldy, const void* scale, int scale_dtype, const tl_layout_header* h)
{
    if (!blob_dev || !X || !Y) return fail(TL_ERR_ARG, "device pointer is null");
    if (reinterpret_cast<uintptr_t>(blob_dev) % 256) return fail(TL_ERR_ALIGN, "weight blob must be 256-byte aligned");
    if (int rc = check_dtype(x_dtype, "x")) return rc;
    if (int rc = check_dtype(y_dtype, "y")) return rc;
    if (scale)
        if (int rc = check_dtype(scale_dtype, "scale")) return rc;
    if (x_layout != TL_X_ROW_MAJOR && x_layout != TL_X_K_MAJOR) return fail(TL_ERR_ARG, "x_layout=%d unknown", x_layout);
    if (M <= 0 || M > (1 << 30)) return fail(TL_ERR_SHAPE, "M=%lld out of range", (long long)M);
    const int64_t min_ldx = x_layout == TL_X_ROW_MAJOR ? h->inners : M;
    if (ldx < min_ldx) return fail(TL_ERR_SHAPE, "ldx=%lld smaller than the %lld elements of a row", (long long)ldx, (long long)min_ldx);
    if (ldy < (int64_t)h->columns) return fail(TL_ERR_SHAPE, "ldy=%lld smaller than N=%u", (long long)ldy, h->columns);
    return TL_OK;
}

}  // namespace

extern "C" int tl_spmm_workspace(const tl_layout_header* header, int64_t M, int x_dtype, int x_layout, int64_t* workspace_bytes)
{
    if (int rc = check_header(header)) return rc;
    if (int rc = check_dtype(x_dtype, "x")) return rc;
    if (!workspace_bytes) return fail(TL_ERR_ARG, "workspace_bytes is null");
    if (M <= 0) return fail(TL_ERR_SHAPE, "M=%lld must be positive", (long long)M);
    if (M <= kSmallMaxM) {
        // needed only when the activations have to be repacked (K-major or unaligned rows); whether the
        // base address is aligned is not known here, so the room is always asked for
        *workspace_bytes = small_repack_bytes(header, M, x_dtype);
        (void)x_layout;
        return TL_OK;
    }
    *workspace_bytes = (int64_t)header->inners * round_up(M, rows_mtile(x_dtype)) * (x_dtype == TL_F16 ? 2 : 4);
    return TL_OK;
}

extern "C" int tl_spmm(const tl_layout_header* header, const void* blob_dev,
                       const void* X, int x_dtype, int x_layout, int64_t ldx, int64_t M,
                       void* Y, int y_dtype, int64_t ldy,
                       const void* scale, int scale_dtype,
                       void* workspace, int64_t workspace_bytes, void* stream)
{
    if (int rc = check_header(header)) return rc;
    if (int rc = check_io(blob_dev, X, Y, x_dtype, x_layout, ldx, M, y_dtype, ldy, scale, scale_dtype, header)) return rc;
    KernelArgs a;
    std::memset(&a, 0, sizeof(a));
    a.w0 = weight_ptrs(header, blob_dev, scale);
    a.X = X; a.Y = Y;
    a.ldx = ldx; a.ldy = ldy;
    a.M = (int)M; a.N = (int)header->columns; a.K = (int)header->inners; a.T = (int)header->n_tiles; a.tile_rows = (int)header->tile_rows;
    a.NB = (int)header->n_blocks;
    a.x_f16 = x_dtype == TL_F16; a.x_kmajor = x_layout == TL_X_K_MAJOR; a.y_f16 = y_dtype == TL_F16; a.scale_f16 = scale_dtype == TL_F16;
    a.one = 1.0f;
    hipStream_t st = static_cast<hipStream_t>(stream);
    int rc = (M <= kSmallMaxM) ? launch_small(a, header, x_dtype, workspace, workspace_bytes, st)
                               : launch_rows(a, x_dtype, workspace, workspace_bytes, false, st);
    if (rc) return rc;
    return finish_launch();
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

extern "C" int tl_spmm_time(const tl_layout_header* header, const void* blob_dev,
                            const void* X, int x_dtype, int x_layout, int64_t ldx, int64_t M,
                            void* Y, int y_dtype, int64_t ldy,
                            const void* scale, int scale_dtype,
                            void* workspace, int64_t workspace_bytes, void* stream,
                            int iters, float* mean_ms)
{
    if (iters <= 0 || !mean_ms) return fail(TL_ERR_ARG, "iters must be positive and mean_ms non-null");
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return fail(TL_ERR_LAUNCH, "hipEventCreate failed");
    int rc = TL_OK;
    (void)hipEventRecord(e0, st);
    for (int i = 0; i < iters && rc == TL_OK; ++i)
        rc = tl_spmm(header, blob_dev, X, x_dtype, x_layout, ldx, M, Y, y_dtype, ldy, scale, scale_dtype, workspace, workspace_bytes, stream);
    (void)hipEventRecord(e1, st);
    if (rc == TL_OK) {
        hipError_t e = hipEventSynchronize(e1);
        float ms = 0.f;
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
        if (e != hipSuccess) rc = fail(TL_ERR_LAUNCH, "event timing failed: %s", hipGetErrorString(e));
        *mean_ms = ms / iters;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return rc;
}
