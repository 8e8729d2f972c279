// gfx950 kernels of libternary_spmm for 1 to 48 activation rows, and their launchers.
//
//   tl_spmv_tiles  M = 1 (decode), the plain product of a contiguous aligned row: a wave owns whole tiles, loads their
//                  chunks and its pieces of the row itself and gathers a tile as soon as that tile's loads have landed.
//   tl_spmv_direct M = 1 with a producer of the row in front (RMSNorm, SiLU gate, attention pieces), or a block that
//                  does not fit the former: a workgroup owns a block of 16 columns over all of K, chunks and row
//                  copied straight into LDS by direct global -> LDS loads.
//   tl_spmm_block  M = 2 ... 4, and single rows that are strided or unaligned.  Owns 1, 2 or 4 blocks; chunks and
//                  activations travel through registers into LDS; partial sums folded with cross-lane shuffles.
//   tl_spmm_quad   M = 5 ... 48, slots of 8 or 16 rows from an aligned K-major image, staged by direct loads; a lane
//                  owns four rows of a column, so a gather reads 16 slots as whole pieces.  tl_spmm_octet: eight rows
//                  per lane, two blocks per wave, for wide outputs at 16 fp16 rows.
//   tl_spmm_res    up to 16 rows, outputs wider than the chip has compute units: the activation image of all of K
//                  resident in LDS, the index stream straight into registers, one workgroup per compute unit.
//
// Only additions and subtractions touch the data; fp32 accumulation throughout.
#include "tl_device.h"

using namespace tl;

namespace {

// ---------------------------------------------------------------------------
// Small-M kernel: one workgroup per (set of column blocks, block of MT rows).
// ---------------------------------------------------------------------------
// acc[m] += sign * x[slot][m] for the four slots named by the bytes of `word`.  `xt` is the staged
// tile, [slot][MT] in the activations' own type; a slot's MT values are fetched with the widest
// LDS reads that fit, fp16 values are widened inside the accumulating fma.
template <int MT, typename XT>
__device__ __forceinline__ void gather_add(float (&acc)[MT], const XT* __restrict__ xt, uint32_t word, float sign)
{
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        const uint32_t r = (word >> (8 * b)) & 0xffu;
        const XT* row = xt + r * MT;
        if constexpr (sizeof(XT) == 4) {
            if constexpr (MT == 4) {
                const float4 v = *reinterpret_cast<const float4*>(row);
                acc[0] = fmaf(v.x, sign, acc[0]);
                acc[1] = fmaf(v.y, sign, acc[1]);
                acc[2] = fmaf(v.z, sign, acc[2]);
                acc[3] = fmaf(v.w, sign, acc[3]);
            } else if constexpr (MT == 2) {
                const float2 v = *reinterpret_cast<const float2*>(row);
                acc[0] = fmaf(v.x, sign, acc[0]);
                acc[1] = fmaf(v.y, sign, acc[1]);
            } else {
                acc[0] = fmaf(row[0], sign, acc[0]);
            }
        } else {
            if constexpr (MT == 4) {
                const uint2 v = *reinterpret_cast<const uint2*>(row);
                acc[0] = fmaf(__half2float(__ushort_as_half((unsigned short)(v.x & 0xffffu))), sign, acc[0]);
                acc[1] = fmaf(__half2float(__ushort_as_half((unsigned short)(v.x >> 16))), sign, acc[1]);
                acc[2] = fmaf(__half2float(__ushort_as_half((unsigned short)(v.y & 0xffffu))), sign, acc[2]);
                acc[3] = fmaf(__half2float(__ushort_as_half((unsigned short)(v.y >> 16))), sign, acc[3]);
            } else if constexpr (MT == 2) {
                const uint32_t v = *reinterpret_cast<const uint32_t*>(row);
                acc[0] = fmaf(__half2float(__ushort_as_half((unsigned short)(v & 0xffffu))), sign, acc[0]);
                acc[1] = fmaf(__half2float(__ushort_as_half((unsigned short)(v >> 16))), sign, acc[1]);
            } else {
                acc[0] = fmaf(__half2float(row[0]), sign, acc[0]);
            }
        }
    }
}

// The same for a lane that owns four neighbouring rows of the slot (`xq` already points at them):
// one 8- or 16-byte LDS read and four accumulating ops per index.
template <int MT, typename XT>
__device__ __forceinline__ void gather_add_quad(float (&acc)[4], const XT* __restrict__ xq, uint32_t word, float sign)
{
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        const uint32_t r = (word >> (8 * b)) & 0xffu;
        const XT* row = xq + r * MT;
        if constexpr (sizeof(XT) == 4) {
            const float4 v = *reinterpret_cast<const float4*>(row);
            acc[0] = fmaf(v.x, sign, acc[0]);
            acc[1] = fmaf(v.y, sign, acc[1]);
            acc[2] = fmaf(v.z, sign, acc[2]);
            acc[3] = fmaf(v.w, sign, acc[3]);
        } else {
            const uint2 v = *reinterpret_cast<const uint2*>(row);
            acc[0] = fmaf(__half2float(__ushort_as_half((unsigned short)(v.x & 0xffffu))), sign, acc[0]);
            acc[1] = fmaf(__half2float(__ushort_as_half((unsigned short)(v.x >> 16))), sign, acc[1]);
            acc[2] = fmaf(__half2float(__ushort_as_half((unsigned short)(v.y & 0xffffu))), sign, acc[2]);
            acc[3] = fmaf(__half2float(__ushort_as_half((unsigned short)(v.y >> 16))), sign, acc[3]);
        }
    }
}

// The quad gather in two steps, so that a lane has the reads of several indices in flight at once (left to
// the compiler, every read is waited for before the next is issued, and a wave spends most of its time on LDS
// latency).  The reads are issued from assembly, which the compiler neither reorders nor tracks; the results
// may be used only after quad_wait<N> has named them, N being the number of reads issued after them.
template <typename XT>
struct QuadRead {
    typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
    typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
    using type = typename std::conditional<sizeof(XT) == 2, u32x2_t, u32x4_t>::type;  // four rows of a slot
};

template <int MT, typename XT>
__device__ __forceinline__ void quad_issue(typename QuadRead<XT>::type (&v)[4], const XT* __restrict__ xq, uint32_t word)
{
    using lds_ptr = const __attribute__((address_space(3))) void*;
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        const uint32_t r = (word >> (8 * b)) & 0xffu;
        const uint32_t addr = (uint32_t)reinterpret_cast<uintptr_t>((lds_ptr)(xq + r * MT));
        if constexpr (sizeof(XT) == 2) asm volatile("ds_read_b64 %0, %1" : "=v"(v[b]) : "v"(addr) : "memory");
        else asm volatile("ds_read_b128 %0, %1" : "=v"(v[b]) : "v"(addr) : "memory");
    }
}

template <int N, typename V>
__device__ __forceinline__ void quad_wait(V (&v)[4])
{
    static_assert(N == 0 || N == 4, "reads are issued four at a time");
    if constexpr (N == 0) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]) : : "memory");
    else asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]) : : "memory");
}

template <typename XT>
__device__ __forceinline__ void quad_accumulate(float (&acc)[4], const typename QuadRead<XT>::type (&v)[4], float sign)
{
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        if constexpr (sizeof(XT) == 4) {
            acc[0] = fmaf(__uint_as_float(v[b].x), sign, acc[0]);
            acc[1] = fmaf(__uint_as_float(v[b].y), sign, acc[1]);
            acc[2] = fmaf(__uint_as_float(v[b].z), sign, acc[2]);
            acc[3] = fmaf(__uint_as_float(v[b].w), sign, acc[3]);
        } else {
            acc[0] = fmaf(__half2float(__ushort_as_half((unsigned short)(v[b].x & 0xffffu))), sign, acc[0]);
            acc[1] = fmaf(__half2float(__ushort_as_half((unsigned short)(v[b].x >> 16))), sign, acc[1]);
            acc[2] = fmaf(__half2float(__ushort_as_half((unsigned short)(v[b].y & 0xffffu))), sign, acc[2]);
            acc[3] = fmaf(__half2float(__ushort_as_half((unsigned short)(v[b].y >> 16))), sign, acc[3]);
        }
    }
}

constexpr int kBlockThreads = 512;            // workgroup of the small-M kernel
// Staging of the activations by the small-M kernel:
constexpr int kStageElements = 0;     // a thread owns slots and reads their MT values one by one (any layout)
constexpr int kStageSlotVectors = 1;  // K-major, aligned: a thread owns slots and reads each as 16-byte vectors
constexpr int kStageRowVectors = 2;   // row-major, aligned, MT <= 4: a thread owns 16-byte pieces of the rows
constexpr int kStageRowCopy = 3;      // one row, aligned, tile height a whole number of vectors: tiles are copied vector by vector
constexpr int kMaxBlockSet = 4;               // column blocks one workgroup may own
constexpr int kSmallStreamBytes = 32 * 1024;  // LDS for the chunks of one group of tiles

// What one thread keeps in registers while a group of tiles is in flight: kVectors 16-byte pieces of
// the stream and, for kSlots slots of the staged tiles, kSlotRegs dwords of activations each.
// (One dword per value: slots are staged element by element or as vectors, as the layout allows.)
template <int MT, int ES, int NT>
struct BlockShape {
    static constexpr int kStreamCap = (NT * 256 < kMaxChunkBytes ? kMaxChunkBytes + 240
                                       : (NT * 256 > kSmallStreamBytes ? kSmallStreamBytes : NT * 256)) / 16 * 16;
    static constexpr int kVectors = (kStreamCap / 16 + NT - 1) / NT;
    static constexpr int kSlotRegs = MT;
    static constexpr int kSlots = 16;  // per thread
    static constexpr int kTiles = kSlots * NT / kTileSlots;                   // tiles per group at most
};

// A workgroup owns BS neighbouring blocks of 16 columns and MT activation rows over all of K.
// K is walked in groups of tiles.  For a group, the chunks of each block are one contiguous piece
// of the stream: the pieces travel global -> registers as 16-byte vectors one group ahead, all in
// flight before anything waits, then registers -> LDS.  The activation rows of the same tiles are
// staged by slot: a thread owns slots of the [tile][slot][MT] LDS image, reads the slot's MT values
// (strided element reads from row-major activations, whole vectors from K-major ones), and
// writes them side by side, so that the gather of an index is one contiguous LDS read of MT values.
// Slots past a tile's height, the sentinel slot among them, are written as zeros.
// From LDS, LPC = 32 / BS lanes share a column: TP tiles are worked on side by side, LW lanes per run,
// one dword (four row indices) per lane and pass; an index is one LDS read and MT accumulating
// ops.  The LPC partial sums of a column are folded with cross-lane shuffles.  No workgroup depends
// on another.
// Four waves per SIMD (two workgroups per compute unit) is what the LDS budget plans for: the register
// allocation is held to that.  MT is 1, 2 or 4; taller slots go to tl_spmm_quad.
template <int MT, bool XF16>
__global__ __launch_bounds__(kBlockThreads) __attribute__((amdgpu_waves_per_eu(4, 4)))
void tl_spmm_block(KernelArgs a)
{
    extern __shared__ __align__(16) unsigned char lds[];
    using XT = typename std::conditional<XF16, __half, float>::type;
    constexpr int NT = kBlockThreads;
    constexpr int ES = (int)sizeof(XT);
    using Shape = BlockShape<MT, ES, NT>;
    constexpr int NV = Shape::kVectors;  // 16-byte stream vectors per thread and group
    constexpr int SPT = Shape::kSlots;   // staged slots per thread and group
    constexpr int RPS = Shape::kSlotRegs;
    constexpr int VPS = MT * ES / 16;    // 16-byte vectors per slot (0: slots are never read as vectors)
    constexpr int VE = 16 / ES;          // activation values per 16-byte vector
    // row-vector staging: vectors per thread and row that cover a group of Shape::kTiles tiles (+2 for the ragged ends)
    constexpr int XPR = ((Shape::kTiles * kMaxTileRows + VE - 1) / VE + 2 + NT - 1) / NT;
    static_assert(MT <= 4, "slots of 8 and 16 rows are tl_spmm_quad's");
    static_assert(MT * XPR * 4 <= SPT * RPS, "row vectors must fit the staging registers");
    const int tid = threadIdx.x;
    const int BS = a.block_set, TG = a.tiles_per_group;
    const int nb0 = blockIdx.x * BS, m0 = blockIdx.y * MT;
    const int bs = min(BS, a.NB - nb0);  // blocks this workgroup really has
    XT* xs = reinterpret_cast<XT*>(lds);                                           // [TG][256 slots][MT]
    uint32_t* buf = reinterpret_cast<uint32_t*>(lds + a.xs_bytes);                 // chunk copies, block after block
    uint32_t* cst = reinterpret_cast<uint32_t*>(lds + a.xs_bytes + a.buf_bytes);   // [BS][TG + 1] chunk starts inside buf
    const_u32_ptr cs = as_const(a.w0.chunkstart) + (size_t)nb0 * a.T;
    const unsigned char* Xb = static_cast<const unsigned char*>(a.X);

    u32x4 cv[NV];
    uint32_t xr[SPT][RPS];  // raw bits: one value per entry (element staging) or whole vectors
    // global -> registers for the tiles [t, t + nt)
    auto prefetch = [&](int t, int nt) {
        uint32_t lo[kMaxBlockSet], pre[kMaxBlockSet + 1];
        pre[0] = 0;
#pragma unroll
        for (int j = 0; j < kMaxBlockSet; ++j) {
            const bool live = j < bs;
            lo[j] = live ? cs[(size_t)j * a.T + t] : 0u;
            pre[j + 1] = pre[j] + (live ? (cs[(size_t)j * a.T + t + nt] - lo[j]) / 4 : 0u);
        }
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const uint32_t g = min((uint32_t)(tid + i * NT), pre[kMaxBlockSet] - 1);  // past the end: last vector again, never stored
            uint32_t base = lo[0], first = 0;
#pragma unroll
            for (int j = 1; j < kMaxBlockSet; ++j)
                if (g >= pre[j]) { base = lo[j]; first = pre[j]; }
            cv[i] = *reinterpret_cast<const u32x4*>(a.w0.stream + base + (size_t)(g - first) * 4);
        }
        if constexpr (MT == 1) {
            if (a.x_mode == kStageRowCopy) {
                // vector v of the group: piece v % vpt of tile v / vpt, vpt pieces per tile
                const int vpt = a.tile_rows / VE;
#pragma unroll
                for (int i = 0; i < XPR; ++i) {
                    const int v = min(tid + i * NT, nt * vpt - 1);
                    const int tile = (int)(((unsigned long long)(unsigned)v * a.vpt_magic) >> 32);  // v / vpt
                    const int k = min((t + tile) * a.tile_rows + (v - tile * vpt) * VE, a.K - VE);   // pieces past K re-read the last one
                    const u32x4 q = *reinterpret_cast<const u32x4*>(Xb + (size_t)k * ES);
                    xr[i * 4 / RPS][i * 4 % RPS] = q[0]; xr[(i * 4 + 1) / RPS][(i * 4 + 1) % RPS] = q[1];
                    xr[(i * 4 + 2) / RPS][(i * 4 + 2) % RPS] = q[2]; xr[(i * 4 + 3) / RPS][(i * 4 + 3) % RPS] = q[3];
                }
                return;
            }
        }
        if constexpr (MT <= 4) {
            if (a.x_mode == kStageRowVectors) {
                // vectors [v_lo, v_hi) of a row cover the group's k range
                const int k_lo = t * a.tile_rows, k_hi = min(a.K, (t + nt) * a.tile_rows);
                const int v_lo = k_lo / VE, v_hi = (k_hi + VE - 1) / VE;
#pragma unroll
                for (int m = 0; m < MT; ++m) {
                    const int row = min(m0 + m, a.M - 1);  // rows past M re-read the last row; they are never stored to Y
#pragma unroll
                    for (int i = 0; i < XPR; ++i) {
                        const int v = min(v_lo + tid + i * NT, v_hi - 1);
                        const u32x4 q = *reinterpret_cast<const u32x4*>(Xb + ((size_t)row * a.ldx + (size_t)v * VE) * ES);
                        const int f = (m * XPR + i) * 4;
                        xr[f / RPS][f % RPS] = q[0]; xr[(f + 1) / RPS][(f + 1) % RPS] = q[1];
                        xr[(f + 2) / RPS][(f + 2) % RPS] = q[2]; xr[(f + 3) / RPS][(f + 3) % RPS] = q[3];
                    }
                }
                return;
            }
        }
#pragma unroll
        for (int s = 0; s < SPT; ++s) {
            const int e = tid + s * NT;  // slot of the group's LDS image
            const int tile = e >> 8, r = e & 255;
            // slots that hold no row re-read a valid element; they are stored as zeros
            const int k = min((t + min(tile, nt - 1)) * a.tile_rows + min(r, a.tile_rows - 1), a.K - 1);
            if (a.x_mode == kStageSlotVectors) {
                if constexpr (VPS > 0) {
                    const unsigned char* src = Xb + ((size_t)k * a.ldx + m0) * ES;
#pragma unroll
                    for (int v = 0; v < VPS; ++v) {
                        const u32x4 q = *reinterpret_cast<const u32x4*>(src + v * 16);
                        xr[s][4 * v + 0] = q[0]; xr[s][4 * v + 1] = q[1]; xr[s][4 * v + 2] = q[2]; xr[s][4 * v + 3] = q[3];
                    }
                }
            } else if constexpr (MT <= 4) {
                const unsigned char* src = Xb + (size_t)k * a.x_sk * ES;
#pragma unroll
                for (int m = 0; m < MT; ++m) {
                    const unsigned char* p = src + (size_t)min(m0 + m, a.M - 1) * a.x_sm * ES;  // rows past M re-read the last row
                    if constexpr (XF16) xr[s][m] = *reinterpret_cast<const unsigned short*>(p);
                    else xr[s][m] = *reinterpret_cast<const uint32_t*>(p);
                }
            }
        }
    };
    // registers -> LDS
    auto commit = [&](int t, int nt) {
        uint32_t lo[kMaxBlockSet], pre[kMaxBlockSet + 1];
        pre[0] = 0;
#pragma unroll
        for (int j = 0; j < kMaxBlockSet; ++j) {
            const bool live = j < bs;
            lo[j] = live ? cs[(size_t)j * a.T + t] : 0u;
            pre[j + 1] = pre[j] + (live ? (cs[(size_t)j * a.T + t + nt] - lo[j]) / 4 : 0u);
        }
#pragma unroll
        for (int i = 0; i < NV; ++i)
            if ((uint32_t)(tid + i * NT) < pre[kMaxBlockSet]) reinterpret_cast<u32x4*>(buf)[tid + i * NT] = cv[i];
        if (tid < kMaxBlockSet * (TG + 1)) {
            const int j = tid / (TG + 1), tl = tid % (TG + 1);
            if (j < bs && tl <= nt) cst[tid] = pre[j] * 4 + cs[(size_t)j * a.T + t + tl] - lo[j];
        }
        if constexpr (MT == 1) {
            if (a.x_mode == kStageRowCopy) {
                // slots past a tile's height (the sentinel slot among them) were zeroed once and are never written
                const int vpt = a.tile_rows / VE;
#pragma unroll
                for (int i = 0; i < XPR; ++i) {
                    const int v = tid + i * NT;
                    const int tile = (int)(((unsigned long long)(unsigned)v * a.vpt_magic) >> 32);
                    const int j = v - tile * vpt;
                    if (v < nt * vpt && (t + tile) * a.tile_rows + j * VE < a.K)
                        *reinterpret_cast<u32x4*>(reinterpret_cast<unsigned char*>(xs) + ((size_t)tile * kTileSlots + (size_t)j * VE) * ES) =
                            u32x4{xr[i * 4 / RPS][i * 4 % RPS], xr[(i * 4 + 1) / RPS][(i * 4 + 1) % RPS],
                                  xr[(i * 4 + 2) / RPS][(i * 4 + 2) % RPS], xr[(i * 4 + 3) / RPS][(i * 4 + 3) % RPS]};
                }
                return;
            }
        }
        if constexpr (MT <= 4) {
            if (a.x_mode == kStageRowVectors) {
                // slots the rows do not cover (past a tile's height, the sentinel slot) must read as zero
                for (int e = tid; e < nt * kTileSlots; e += NT)
                    if ((e & 255) >= min(a.tile_rows, a.K - (t + (e >> 8)) * a.tile_rows)) {
#pragma unroll
                        for (int m = 0; m < MT; ++m) xs[(size_t)e * MT + m] = XT(0.0f);
                    }
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
                        for (int el = 0; el < VE; ++el) {
                            if (k >= k_lo && k < k_hi) {
                                XT* dst = xs + (size_t)((tile - t) * kTileSlots + r) * MT;
#pragma unroll
                                for (int m = 0; m < MT; ++m) {
                                    const int f = (m * XPR + i) * 4 + (XF16 ? el / 2 : el);
                                    const uint32_t word = xr[f / RPS][f % RPS];
                                    if constexpr (XF16) dst[m] = __ushort_as_half((unsigned short)(el % 2 ? word >> 16 : word & 0xffffu));
                                    else dst[m] = __uint_as_float(word);
                                }
                            }
                            ++k;
                            if (++r == a.tile_rows) { r = 0; ++tile; }
                        }
                    }
                }
                return;
            }
        }
#pragma unroll
        for (int s = 0; s < SPT; ++s) {
            const int e = tid + s * NT;
            const int tile = e >> 8, r = e & 255;
            if (tile < nt) {
                const bool real = r < min(a.tile_rows, a.K - (t + tile) * a.tile_rows);
                uint32_t packed[MT * ES / 4 > 0 ? MT * ES / 4 : 1];
                if (a.x_mode == kStageSlotVectors && VPS > 0) {
#pragma unroll
                    for (int d = 0; d < MT * ES / 4; ++d) packed[d] = real ? xr[s][d] : 0u;
                } else if constexpr (XF16) {
                    if constexpr (MT == 1) packed[0] = real ? xr[s][0] : 0u;
#pragma unroll
                    for (int d = 0; d < MT / 2; ++d) packed[d] = real ? (xr[s][2 * d] | (xr[s][2 * d + 1] << 16)) : 0u;
                } else {
#pragma unroll
                    for (int d = 0; d < MT; ++d) packed[d] = real ? xr[s][d] : 0u;
                }
                unsigned char* dst = reinterpret_cast<unsigned char*>(xs) + (size_t)e * MT * ES;
                if constexpr (MT * ES >= 16) {
#pragma unroll
                    for (int v = 0; v < MT * ES / 16; ++v)
                        reinterpret_cast<u32x4*>(dst)[v] = u32x4{packed[4 * v], packed[4 * v + 1], packed[4 * v + 2], packed[4 * v + 3]};
                } else if constexpr (MT * ES == 8) {
                    *reinterpret_cast<uint2*>(dst) = make_uint2(packed[0], packed[1]);
                } else if constexpr (MT * ES == 4) {
                    *reinterpret_cast<uint32_t*>(dst) = packed[0];
                } else {
                    *reinterpret_cast<unsigned short*>(dst) = (unsigned short)packed[0];
                }
            }
        }
    };

    const int lpc_shift = a.lpc_shift, lw_shift = a.lw_shift;
    const int LPC = 1 << lpc_shift, LW = 1 << lw_shift, TP = LPC >> lw_shift;
    const int col = tid >> lpc_shift, lig = tid & (LPC - 1);
    const int blk = col >> 4, c16 = col & 15;
    const int tp = lig >> lw_shift, lw = lig & (LW - 1);
    const uint32_t* my_cst = cst + blk * (TG + 1);
    float acc[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[m] = 0.f;

    if constexpr (MT == 1) {
        if (a.x_mode == kStageRowCopy)
            for (int e = tid; e < a.xs_bytes / 16; e += NT) reinterpret_cast<u32x4*>(xs)[e] = u32x4{0u, 0u, 0u, 0u};
    }
    constexpr int TU = 2;  // tiles of one lane whose LDS reads are issued together
    prefetch(0, min(TG, a.T));
    for (int t = 0; t < a.T; t += TG) {
        const int nt = min(TG, a.T - t);
        __syncthreads();  // the previous group has been consumed
        commit(t, nt);
        __syncthreads();
        if (t + TG < a.T) prefetch(t + TG, min(TG, a.T - t - TG));
        if (blk < bs) {
            for (int tl0 = tp; tl0 < nt; tl0 += TP * TU) {
                uint32_t d[TU];
                const uint32_t* run[TU];
#pragma unroll
                for (int u = 0; u < TU; ++u) {
                    const int tl = tl0 + u * TP;
                    const uint32_t* chunk = buf + my_cst[min(tl, nt - 1)];
                    d[u] = tl < nt ? chunk[c16] : 0u;  // tiles past the group: empty run
                    run[u] = chunk + (d[u] >> 16);
                }
                uint32_t w[TU];
#pragma unroll
                for (int u = 0; u < TU; ++u)  // lanes past the run's end take an all-sentinel word: four gathers of zero
                    w[u] = lw < run_pos_dwords(d[u]) + run_neg_dwords(d[u]) ? run[u][lw] : 0xffffffffu;
#pragma unroll
                for (int u = 0; u < TU; ++u) {
                    const int pd = run_pos_dwords(d[u]), tot = pd + run_neg_dwords(d[u]);
                    if (u > 0 && __builtin_amdgcn_ballot_w64(tot > 0) == 0) continue;  // no lane of the wave has this tile
                    const XT* xt = xs + (size_t)min(tl0 + u * TP, nt - 1) * kTileSlots * MT;
                    gather_add<MT, XT>(acc, xt, w[u], lw < pd ? 1.0f : -1.0f);
                    for (int i = lw + LW; i < tot; i += LW)  // runs longer than the lane group
                        gather_add<MT, XT>(acc, xt, run[u][i], i < pd ? 1.0f : -1.0f);
                }
            }
        }
    }
    // fold the LPC partial sums of a column; per step the MT exchanges are independent of each other
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) {
        if (off < LPC) {
            float other[MT];
#pragma unroll
            for (int m = 0; m < MT; ++m) other[m] = __shfl_xor(acc[m], off, 64);
#pragma unroll
            for (int m = 0; m < MT; ++m) acc[m] += other[m];
        }
    }
    const int n = (nb0 + blk) * TL_BLOCK_COLUMNS + c16;
    if (lig == 0 && blk < bs && n < a.N) {
        const float s = load_scale(a.w0.scale, a.scale_f16, n);
#pragma unroll
        for (int m = 0; m < MT; ++m)
            if (m0 + m < a.M) store_out(a.Y, a.y_f16, (long long)(m0 + m) * a.ldy + n, acc[m] * s);
    }
}

// The activation images of a group of tiles, global -> LDS, for tl_spmm_quad and tl_spmm_octet.  Piece p = p0 + tid of
// the group (16 bytes; VPS pieces per slot, 256 slots per tile) belongs to tile p / PT, slot (p % PT) / VPS.  NT and
// PT = 256 * VPS are powers of two, so the part of that which depends on the thread is the same in every turn of the
// loop: it is worked out once per kernel (ImageLane), and a turn adds a wave-uniform base address -- two or three
// vector instructions per piece instead of the 64-bit multiplications of the full address.
struct ImageLane {
    int tile, row;      // the thread's tile within a turn (workgroups wider than a tile) and its slot's share of the row index
    uint32_t offset;    // bytes from the turn's base address to the thread's piece
};

template <int VPS, int NT>
__device__ __forceinline__ ImageLane image_lane(const KernelArgs& a, int tid, size_t row_bytes)
{
    constexpr int PT = kTileSlots * VPS;
    ImageLane l;
    l.tile = NT >= PT ? tid / PT : 0;
    const int rem = NT >= PT ? tid % PT : tid;
    l.row = rem / VPS;
    l.offset = (uint32_t)(l.tile * a.tile_rows + l.row) * (uint32_t)row_bytes + (uint32_t)(rem % VPS) * 16u;
    return l;
}

template <int VPS, int NT>
__device__ __forceinline__ void issue_images(const KernelArgs& a, const unsigned char* Xb, size_t row_bytes, unsigned char* xs, int t, int nt,
                                             int wave, int lane, const ImageLane& l)
{
    using global_ptr = const __attribute__((address_space(1))) void*;
    using lds_ptr = __attribute__((address_space(3))) void*;
    constexpr int PT = kTileSlots * VPS;
    const int pieces = nt * PT;  // a multiple of 64: whole waves
    for (int p0 = 0; p0 + wave * 64 < pieces; p0 += NT) {
        const int first = p0 + wave * 64;
        const int tile_u = p0 / PT, row_u = (p0 % PT) / VPS;  // wave-uniform: the turn's first tile and row
        const int r = row_u + l.row, k = (t + tile_u + l.tile) * a.tile_rows + r;
        if (r < a.tile_rows && k < a.K) {
            const unsigned char* base = Xb + ((size_t)(t + tile_u) * a.tile_rows + row_u) * row_bytes;
            __builtin_amdgcn_global_load_lds((global_ptr)(base + l.offset), (lds_ptr)(xs + (size_t)first * 16), 16, 0, 0);
        } else {
            *reinterpret_cast<u32x4*>(xs + (size_t)(first + lane) * 16) = u32x4{0u, 0u, 0u, 0u};
        }
    }
}

// A value of a row of halves or floats as it lies in memory, and its conversion (apart, so that the load can be
// issued long before the value is needed).
__device__ __forceinline__ uint32_t load_raw(const void* p, int is_f16, long long n)
{
    return is_f16 ? (uint32_t)static_cast<const uint16_t*>(p)[n] : static_cast<const uint32_t*>(p)[n];
}
__device__ __forceinline__ float raw_value(uint32_t raw, int is_f16)
{
    return is_f16 ? __half2float(__ushort_as_half((unsigned short)raw)) : __uint_as_float(raw);
}

// What the epilogue of a 16-row block multiplies and adds: the column's scale, the residual values of a lane's four
// rows of column n and the next norm's weight of that column.  Asked for early, so that they are there at the very
// end, and kept as loaded: a conversion where they are asked for would make the wave wait for each of them in turn
// (and for every tile load issued before).
struct ChainOperands {
    uint32_t res[4];
    uint32_t w;
    uint32_t scale;
};

__device__ __forceinline__ ChainOperands chain_operands(const KernelArgs& a, int n, int q)
{
    ChainOperands o = {{0u, 0u, 0u, 0u}, 0u, 0u};
    if (n < a.N) {
        if (a.w0.scale) o.scale = load_raw(a.w0.scale, a.scale_f16, n);
        if (a.chain_res) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (q * 4 + j < a.M) o.res[j] = load_raw(a.chain_res, a.y_f16, (long long)(q * 4 + j) * a.chain_ldres + n);
        }
        if (a.chain_image) o.w = load_raw(a.chain_w, a.y_f16, n);
    }
    return o;
}
// the column's scale among them (0 past the last column, 1 without a scale)
__device__ __forceinline__ float chain_scale(const KernelArgs& a, int n, const ChainOperands& early)
{
    return n < a.N ? (a.w0.scale ? raw_value(early.scale, a.scale_f16) : 1.0f) : 0.f;
}

// The chained part of the way out of a block of 16 columns x 16 rows.  Called by one whole wave: lane = column
// c16 = lane / 4 of block nb (n = its column), rows 4q .. 4q + 3 (q = lane % 4); `out` = the lane's four sums times
// the column's scale on the way in, what Y gets on the way out.
__device__ __forceinline__ void chain_epilogue16(const KernelArgs& a, int nb, int n, int c16, int q, float (&out)[4], const float4& row_factors,
                                                 const ChainOperands& early)
{
    if (a.chain_sq_in) {  // q == lane % 4: the lane's own rows
        out[0] *= row_factors.x; out[1] *= row_factors.y; out[2] *= row_factors.z; out[3] *= row_factors.w;
    }
    if (a.chain_res) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (n < a.N && q * 4 + j < a.M) out[j] = as_output(out[j], a.y_f16) + raw_value(early.res[j], a.y_f16);
    }
    if (a.chain_image) {
        const float w = raw_value(early.w, a.y_f16);
        float sq[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float v = (n < a.N && q * 4 + j < a.M) ? as_output(out[j], a.y_f16) : 0.f;  // what Y will hold
            sq[j] = v * v;
            if (n < a.N && q * 4 + j < a.chain_ild) store_out(a.chain_image, a.y_f16, (long long)n * a.chain_ild + q * 4 + j, v * w);
        }
#pragma unroll
        for (int off = 4; off < 64; off <<= 1) {  // over the 16 columns of the block
#pragma unroll
            for (int j = 0; j < 4; ++j) sq[j] += __shfl_xor(sq[j], off, 64);
        }
        if (c16 == 0) {
#pragma unroll
            for (int j = 0; j < 4; ++j) a.chain_sq_out[(size_t)nb * 16 + q * 4 + j] = sq[j];
        }
    }
}

// ---------------------------------------------------------------------------
// Small-M kernel for slots of 8 and 16 rows, staged by direct global -> LDS loads.
// ---------------------------------------------------------------------------
// One workgroup owns one block of 16 columns and MT activation rows over all of K, walked in groups
// of TG tiles.  A group's chunks and its activation rows (from the aligned K-major image, whose row k
// holds the MT values of slot k side by side) are copied into LDS by `global_load_lds_dwordx4`: a lane
// names 16 bytes in memory, they land at M0 + 16 * lane, and no register holds them on the way.  Two
// LDS buffers alternate: the loads of group g + 1 are issued before group g is consumed, and one
// barrier per group orders both the reuse of a buffer and the arrival of the next one.  Slots past a
// tile's height (the sentinel among them) are written as zeros by ordinary stores.
// With no staging registers a workgroup needs few registers, so several share a compute unit and
// hide each other's waits; the launcher sizes TG for that.
// Gather: a lane owns four rows of one column, the MT / 4 lanes of a column sit side by side and the 16
// columns next to each other, so one gather instruction reads 16 slots (one per column) as whole
// contiguous pieces.  The P lane groups of a column share its runs: TP tiles side by side, LW groups
// per run, up to four dwords (16 independent gathers) per turn.  The P partial sums are folded through LDS.
template <int MT, bool XF16, int NT = kBlockThreads>
__global__ __launch_bounds__(NT) void tl_spmm_quad(KernelArgs a)
{
    extern __shared__ __align__(16) unsigned char lds[];
    using XT = typename std::conditional<XF16, __half, float>::type;
    constexpr int ES = (int)sizeof(XT);
    constexpr int SLOT = MT * ES;      // bytes of a slot
    constexpr int VPS = SLOT / 16;     // 16-byte pieces per slot
    constexpr int Q = MT / 4;
    static_assert(MT == 8 || MT == 16, "row quads of 8- and 16-row slots");
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int TG = a.tiles_per_group;
    const int nb = blockIdx.x, m0 = blockIdx.y * MT;
    const int stage_bytes = a.xs_bytes + a.buf_bytes;
    uint32_t* cst = reinterpret_cast<uint32_t*>(lds + 2 * stage_bytes);  // [2][TG + 1] chunk starts inside a buffer's chunk copies
    const_u32_ptr cs = as_const(a.w0.chunkstart) + (size_t)nb * a.T;
    const unsigned char* Xb = static_cast<const unsigned char*>(a.X) + (size_t)m0 * ES;
    const size_t row_bytes = (size_t)a.ldx * ES;
    using global_ptr = const __attribute__((address_space(1))) void*;
    using lds_ptr = __attribute__((address_space(3))) void*;

    // global -> LDS buffer `which` for the tiles [t, t + nt)
    const ImageLane image = image_lane<VPS, NT>(a, tid, row_bytes);
    auto issue = [&](int t, int nt, int which) {
        unsigned char* xs = lds + which * stage_bytes;
        unsigned char* buf = xs + a.xs_bytes;
        issue_images<VPS, NT>(a, Xb, row_bytes, xs, t, nt, wave, lane, image);
        const uint32_t lo = cs[t];
        const int vectors = (int)((cs[t + nt] - lo) / 4);
        for (int first = wave * 64; first < vectors; first += NT)
            if (first + lane < vectors)
                __builtin_amdgcn_global_load_lds((global_ptr)(a.w0.stream + lo + (size_t)(first + lane) * 4), (lds_ptr)(buf + (size_t)first * 16), 16, 0, 0);
        if (tid <= nt) cst[which * (TG + 1) + tid] = cs[t + tid] - lo;
    };

    const int lw_shift = a.lw_shift;
    const int LPC = 1 << a.lpc_shift, LW = 1 << lw_shift, TP = LPC >> lw_shift;
    const int q = tid % Q, c16 = (tid / Q) & 15, lig = tid / (Q * TL_BLOCK_COLUMNS);
    const int tp = lig >> lw_shift, lw = lig & (LW - 1);
    float acc[4] = {0.f, 0.f, 0.f, 0.f};

    issue(0, min(TG, a.T), 0);
    float4 row_factors = make_float4(1.f, 1.f, 1.f, 1.f);  // chained product, first wave: the factors of rows 4 * (lane % 4) .. + 3
    if (MT == 16 && a.chain_sq_in && tid < 64) row_factors = chain_row_factors(a, tid);
    // what the chained epilogue of the first wave adds and multiplies, asked for now rather than at the very end
    ChainOperands early = {{0u, 0u, 0u, 0u}, 0u, 0u};
    if (MT == 16 && tid < 64) early = chain_operands(a, nb * TL_BLOCK_COLUMNS + ((tid / Q) & 15), tid % Q);
    int which = 0;
    for (int t = 0; t < a.T; t += TG, which ^= 1) {
        const int nt = min(TG, a.T - t);
        // this wave's loads have landed; after the barrier everybody's have, and the other buffer is free
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (t + TG < a.T) issue(t + TG, min(TG, a.T - t - TG), which ^ 1);
        const unsigned char* xs = lds + which * stage_bytes;
        const uint32_t* buf = reinterpret_cast<const uint32_t*>(xs + a.xs_bytes);
        const uint32_t* my_cst = cst + which * (TG + 1);
        for (int tl = tp; tl < nt; tl += TP) {
            const uint32_t* chunk = buf + my_cst[tl];
            const uint32_t d = chunk[c16];
            const uint32_t* run = chunk + (d >> 16);
            const int pd = run_pos_dwords(d), tot = pd + run_neg_dwords(d);
            const XT* xq = reinterpret_cast<const XT*>(xs) + (size_t)tl * kTileSlots * MT + q * 4;
            // two dwords a turn: the eight reads are in flight together, and those of the second dword land
            // while the first is accumulated
            typename QuadRead<XT>::type va[4], vb[4];
            int i = lw;
            for (; i + LW < tot; i += 2 * LW) {
                const uint32_t w0 = run[i], w1 = run[i + LW];
                quad_issue<MT, XT>(va, xq, w0);
                quad_issue<MT, XT>(vb, xq, w1);
                quad_wait<4>(va);
                quad_accumulate<XT>(acc, va, i < pd ? 1.0f : -1.0f);
                quad_wait<0>(vb);
                quad_accumulate<XT>(acc, vb, i + LW < pd ? 1.0f : -1.0f);
            }
            if (i < tot) {
                quad_issue<MT, XT>(va, xq, run[i]);
                quad_wait<0>(va);
                quad_accumulate<XT>(acc, va, i < pd ? 1.0f : -1.0f);
            }
        }
    }
    // fold the LPC partial sums of each (column, row quad) through LDS
    __syncthreads();
    float4* red = reinterpret_cast<float4*>(lds);
    red[tid] = make_float4(acc[0], acc[1], acc[2], acc[3]);
    __syncthreads();
    constexpr int per_group = TL_BLOCK_COLUMNS * Q;  // threads of one lane group
    if (tid < per_group) {
        float4 sum = red[tid];
#pragma unroll 4
        for (int l = 1; l < LPC; ++l) {
            const float4 o = red[l * per_group + tid];
            sum.x += o.x; sum.y += o.y; sum.z += o.z; sum.w += o.w;
        }
        const int n = nb * TL_BLOCK_COLUMNS + c16;
        const float sc = MT == 16 ? chain_scale(a, n, early) : n < a.N ? load_scale(a.w0.scale, a.scale_f16, n) : 0.f;
        float out[4] = {sum.x * sc, sum.y * sc, sum.z * sc, sum.w * sc};
        if constexpr (MT == 16) chain_epilogue16(a, nb, n, c16, q, out, row_factors, early);  // (one wave here: 16 columns x 4 row quads)
        if (n < a.N) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (m0 + q * 4 + j < a.M) store_out(a.Y, a.y_f16, (long long)(m0 + q * 4 + j) * a.ldy + n, out[j]);
        }
    }
}

// ---------------------------------------------------------------------------
// 16 fp16 rows, eight per lane, two column blocks per workgroup.
// ---------------------------------------------------------------------------
// tl_spmm_quad<16, true> with the work cut differently: a lane owns EIGHT rows of one column (one 16-byte LDS
// read and eight accumulates per index, so each index is decoded by two lanes instead of four), and the 64 lanes
// of a wave cover 32 columns -- two neighbouring blocks, which share the staged activation image.  Per non-zero
// that is five vector ops fewer in the loop, and half as many lanes go through a run's set-up and tail; per block
// the image is staged half as often.  The launcher uses it where it still leaves every compute unit workgroups
// enough (wide outputs).
__global__ __launch_bounds__(kBlockThreads) void tl_spmm_octet(KernelArgs a)
{
    extern __shared__ __align__(16) unsigned char lds[];
    using XT = __half;
    constexpr int NT = kBlockThreads;
    constexpr int MT = 16, ES = 2, VPS = MT * ES / 16, BS = 2, COLS = TL_BLOCK_COLUMNS * BS;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int TG = a.tiles_per_group;
    const int nb0 = blockIdx.x * BS, m0 = blockIdx.y * MT;
    const int bs = min(BS, a.NB - nb0);  // blocks this workgroup really has
    const int stage_bytes = a.xs_bytes + a.buf_bytes;
    const int block_buf_bytes = a.buf_bytes / BS;  // chunk copies of one block and group (a multiple of 16)
    uint32_t* cst = reinterpret_cast<uint32_t*>(lds + 2 * stage_bytes);  // [2][BS][TG + 1] chunk starts inside a block's chunk copies
    const_u32_ptr cs = as_const(a.w0.chunkstart) + (size_t)nb0 * a.T;
    const unsigned char* Xb = static_cast<const unsigned char*>(a.X) + (size_t)m0 * ES;
    const size_t row_bytes = (size_t)a.ldx * ES;
    using global_ptr = const __attribute__((address_space(1))) void*;
    using lds_ptr = __attribute__((address_space(3))) void*;

    auto issue = [&](int t, int nt, int which) {
        unsigned char* xs = lds + which * stage_bytes;
        unsigned char* buf = xs + a.xs_bytes;
        // (the full address per piece: the precomputed lane shares of tl_spmm_quad would take this kernel past 80
        // registers, a wave per SIMD less)
        const int pieces = nt * kTileSlots * VPS;  // a multiple of 64: whole waves
        for (int first = wave * 64; first < pieces; first += NT) {
            const int p = first + lane, slot = p / VPS, v = p % VPS;
            const int r = slot & (kTileSlots - 1), k = (t + (slot >> 8)) * a.tile_rows + r;
            if (r < a.tile_rows && k < a.K)
                __builtin_amdgcn_global_load_lds((global_ptr)(Xb + (size_t)k * row_bytes + v * 16), (lds_ptr)(xs + (size_t)first * 16), 16, 0, 0);
            else
                *reinterpret_cast<u32x4*>(xs + (size_t)p * 16) = u32x4{0u, 0u, 0u, 0u};
        }
        for (int j = 0; j < bs; ++j) {
            const_u32_ptr csj = cs + (size_t)j * a.T;
            const uint32_t lo = csj[t];
            const int vectors = (int)((csj[t + nt] - lo) / 4);
            unsigned char* bufj = buf + (size_t)j * block_buf_bytes;
            for (int first = wave * 64; first < vectors; first += NT)
                if (first + lane < vectors)
                    __builtin_amdgcn_global_load_lds((global_ptr)(a.w0.stream + lo + (size_t)(first + lane) * 4), (lds_ptr)(bufj + (size_t)first * 16), 16, 0, 0);
            if (tid <= nt) cst[(which * BS + j) * (TG + 1) + tid] = csj[t + tid] - lo;
        }
    };

    const int lw_shift = a.lw_shift;
    const int LPC = 1 << a.lpc_shift, LW = 1 << lw_shift, TP = LPC >> lw_shift;
    // a wave is one lane group: lanes 2c, 2c + 1 hold rows 0-7 and 8-15 of column c of the workgroup's 32
    const int q = tid & 1, col = (tid >> 1) & (COLS - 1), lig = tid / (2 * COLS);
    const int blk = col / TL_BLOCK_COLUMNS, c16 = col % TL_BLOCK_COLUMNS;
    const int tp = lig >> lw_shift, lw = lig & (LW - 1);
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
    auto issue4 = [](u32x4 (&v)[4], const XT* xq, uint32_t word) {
        using lds_cptr = const __attribute__((address_space(3))) void*;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const uint32_t r = (word >> (8 * b)) & 0xffu;
            const uint32_t addr = (uint32_t)reinterpret_cast<uintptr_t>((lds_cptr)(xq + r * MT));
            asm volatile("ds_read_b128 %0, %1" : "=v"(v[b]) : "v"(addr) : "memory");
        }
    };
    auto add4 = [&](const u32x4 (&v)[4], float sign) {
#pragma unroll
        for (int b = 0; b < 4; ++b)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                acc[2 * e] = fmaf(__half2float(__ushort_as_half((unsigned short)(v[b][e] & 0xffffu))), sign, acc[2 * e]);
                acc[2 * e + 1] = fmaf(__half2float(__ushort_as_half((unsigned short)(v[b][e] >> 16))), sign, acc[2 * e + 1]);
            }
    };

    issue(0, min(TG, a.T), 0);
    float4 row_factors = make_float4(1.f, 1.f, 1.f, 1.f);  // chained product, first wave: the factors of rows 4 * (lane % 4) .. + 3
    if (a.chain_sq_in && tid < 64) row_factors = chain_row_factors(a, tid);
    int which = 0;
    for (int t = 0; t < a.T; t += TG, which ^= 1) {
        const int nt = min(TG, a.T - t);
        // this wave's loads have landed; after the barrier everybody's have, and the other buffer is free
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (t + TG < a.T) issue(t + TG, min(TG, a.T - t - TG), which ^ 1);
        const unsigned char* xs = lds + which * stage_bytes;
        const uint32_t* buf = reinterpret_cast<const uint32_t*>(xs + a.xs_bytes + (size_t)blk * block_buf_bytes);
        const uint32_t* my_cst = cst + (which * BS + blk) * (TG + 1);
        if (blk < bs) {
            for (int tl = tp; tl < nt; tl += TP) {
                const uint32_t* chunk = buf + my_cst[tl];
                const uint32_t d = chunk[c16];
                const uint32_t* run = chunk + (d >> 16);
                const int pd = run_pos_dwords(d), tot = pd + run_neg_dwords(d);
                const XT* xq = reinterpret_cast<const XT*>(xs) + (size_t)tl * kTileSlots * MT + q * 8;
                u32x4 va[4], vb[4];
                int i = lw;
                for (; i + LW < tot; i += 2 * LW) {
                    const uint32_t w0 = run[i], w1 = run[i + LW];
                    issue4(va, xq, w0);
                    issue4(vb, xq, w1);
                    quad_wait<4>(va);
                    add4(va, i < pd ? 1.0f : -1.0f);
                    quad_wait<0>(vb);
                    add4(vb, i + LW < pd ? 1.0f : -1.0f);
                }
                if (i < tot) {
                    issue4(va, xq, run[i]);
                    quad_wait<0>(va);
                    add4(va, i < pd ? 1.0f : -1.0f);
                }
            }
        }
    }
    // fold the LPC partial sums of each (column, row octet) through LDS
    __syncthreads();
    float4* red = reinterpret_cast<float4*>(lds);  // [lane group][2][64 lanes]
    red[(size_t)lig * 128 + lane] = make_float4(acc[0], acc[1], acc[2], acc[3]);
    red[(size_t)lig * 128 + 64 + lane] = make_float4(acc[4], acc[5], acc[6], acc[7]);
    __syncthreads();
    if (tid < 64) {
        float4 s0 = red[tid], s1 = red[64 + tid];
#pragma unroll 4
        for (int l = 1; l < LPC; ++l) {
            const float4 o0 = red[(size_t)l * 128 + tid], o1 = red[(size_t)l * 128 + 64 + tid];
            s0.x += o0.x; s0.y += o0.y; s0.z += o0.z; s0.w += o0.w;
            s1.x += o1.x; s1.y += o1.y; s1.z += o1.z; s1.w += o1.w;
        }
        const int n = (nb0 + blk) * TL_BLOCK_COLUMNS + c16;
        const bool real = blk < bs && n < a.N;
        const float sc = real ? load_scale(a.w0.scale, a.scale_f16, n) : 0.f;
        float out[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
        if (a.chain_sq_in) {  // rows 8q .. 8q + 7: the row quads of lanes 2q and 2q + 1
            const float f[4] = {row_factors.x, row_factors.y, row_factors.z, row_factors.w};
#pragma unroll
            for (int j = 0; j < 8; ++j) out[j] *= __shfl(f[j & 3], 2 * q + (j >> 2), 64);
        }
        if (a.gated) {
            // gate and up column of a pair sit two lanes apart (same rows): the even column's lane writes the eight products
            float h[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float y = real ? as_output(out[j] * sc, a.y_f16) : 0.f;
                const float up = __shfl_xor(y, 2, 64);
                h[j] = m0 + q * 8 + j < a.M ? gate_pair(y, up, a.y_f16) : 0.f;  // zeros in the padding rows of a K-major image
            }
            if (!(c16 & 1) && real && n + 1 < a.N) {
                const int m = m0 + q * 8;
                if (a.y_kld && a.y_f16 && a.y_kld % 8 == 0 && m + 8 <= a.y_kld && reinterpret_cast<uintptr_t>(a.Y) % 16 == 0) {
                    // eight neighbouring rows of one column of the image: one 16-byte store
                    u32x4 packed;
                    __half* p = reinterpret_cast<__half*>(&packed);
#pragma unroll
                    for (int j = 0; j < 8; ++j) p[j] = __float2half(settled(h[j]));
                    *reinterpret_cast<u32x4*>(static_cast<__half*>(a.Y) + (long long)(n / 2) * a.y_kld + m) = packed;
                } else {
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        if (m + j < a.M) store_out(a.Y, a.y_f16, a.y_kld ? (long long)(n / 2) * a.y_kld + m + j : (long long)(m + j) * a.ldy + n / 2, h[j]);
                        else if (m + j < a.y_kld) store_out(a.Y, a.y_f16, (long long)(n / 2) * a.y_kld + m + j, 0.f);
                    }
                }
            }
            return;
        }
        if (real) {
#pragma unroll
            for (int j = 0; j < 8; ++j)
                if (m0 + q * 8 + j < a.M) store_out(a.Y, a.y_f16, (long long)(m0 + q * 8 + j) * a.ldy + n, out[j] * sc);
        }
    }
}

// ---------------------------------------------------------------------------
// 16 fp16 rows or 8 fp32 rows: the whole activation image resident in LDS, the index stream straight into registers.
// ---------------------------------------------------------------------------
// One workgroup of 16 waves per compute unit.  The image of ALL of K ([tile][256 slots][32 bytes]: 16 fp16 or 8 fp32
// rows, 8 KB a tile) is loaded once per workgroup and stays; from then on only weights move, and they never touch LDS: a lane
// loads the dwords of its own run from the stream into registers, one (block, tile) unit ahead of their use, its
// descriptor two units ahead, the chunk offset three.  A workgroup owns a range of whole column blocks; its
// (block, tile) units, in block-major order (= the order of the stream), are cut into 16 contiguous pieces, one per
// wave, so that after the barrier behind the image no wave waits for another until the column sums meet at the end.
// In a unit the 64 lanes are 2 signs x 16 columns x 2 halves of a slot: a lane walks ONE run (the +1 or the -1 rows
// of its column) from start to end for eight fp16 or four fp32 rows -- one 16-byte LDS read and eight (four)
// accumulates per index, the sign a constant of the lane.  More rows than a slot holds are further workgroups
// (blockIdx.y) with an image of their own.  Where a wave's units pass from one block to the next it leaves its sums for the block in
// an LDS slot; slot (wave + block) is unique because both only grow along the unit order.  After the one barrier
// at the end the slots of a block are added in wave order (the same order every time) and the sums go out.
constexpr int kResWaves = 16;

// ROWS_IN: the activations come as row-major rows of whole, aligned 16-byte pieces (else: an aligned K-major image, whose
// slots are copied straight into LDS) and the workgroup turns them into its image itself: a thread takes the same
// 16-byte piece of four rows, transposes the 4 x 4 (fp32) or 4 x 8 (fp16) values in registers and writes one slot
// quarter per value of k.  Threads of a wave would all write slots that are equal modulo 8 -- the same banks -- so
// each rotates its values by its piece number first and writes them in the rotated order.
template <bool XF16, int NP, bool ROWS_IN>  // NP: 16-byte pieces of a run that a lane holds in registers (longer runs: the rest dword by dword)
__global__ __launch_bounds__(kResWaves * 64) void tl_spmm_res(KernelArgs a)
{
    extern __shared__ __align__(16) unsigned char lds[];
    constexpr int NT = kResWaves * 64, W = kResWaves, MT = XF16 ? 16 : 8, ES = XF16 ? 2 : 4, VPS = MT * ES / 16;
    constexpr int NA = MT / 2;                              // rows (accumulators) of a lane
    constexpr int kResSlotFloats = TL_BLOCK_COLUMNS * MT;   // sums of one block: [column][row]
    static_assert(MT * ES == 32 && VPS == 2, "a slot is two 16-byte pieces");
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int G = (int)gridDim.x, g = (int)blockIdx.x;
    const int b0 = (int)((long long)g * a.NB / G), nblk = (int)((long long)(g + 1) * a.NB / G) - b0;
    const int T = a.T;
    const int U = nblk * T;                                    // units of this workgroup, unit u = (block u / T, tile u % T)
    const int u0 = wave * U / W, u1 = (wave + 1) * U / W;      // this wave's
    const int m0 = (int)blockIdx.y * MT;                       // first row of this workgroup's slot
    unsigned char* image = lds;                                // [T][256 slots][MT rows]
    float* slots = reinterpret_cast<float*>(lds + a.xs_bytes); // [W + nblk - 1][column][row]
    using global_ptr = const __attribute__((address_space(1))) void*;
    using lds_ptr = __attribute__((address_space(3))) void*;

    // chunk offsets of the wave's first units, ahead of everything else (entries past the wave's units are read and
    // not used; past the table's end lies the stream)
    const_u32_ptr cs = as_const(a.w0.chunkstart) + (size_t)b0 * T;
    const int last = max(u1 - 1, u0);  // units past the wave's last stand for it (loaded again, never used)
    const uint32_t cs_a = cs[u0], cs_b = cs[u0 + 1], cs_c = cs[u0 + 2];

    // The LDS serves a 16-byte read of a wave in four passes of 16 lanes: lanes 0-3, 12-15, 20-27 / 4-11, 16-19, 28-31 and
    // the same of lanes 32-63 (measured: two lanes of a pass on one bank cost a cycle more, lanes of different passes
    // do not).  Lanes are given columns so that a pass holds 8 NEIGHBOURING columns of one sign, two lanes (the row
    // octets) to a column: the packer orders the rows of such a group so that, position by position, they differ
    // modulo 8, i.e. fall on different banks.
    const int sgn = lane >> 5, h = lane & 1;
    const int c16 = 2 * (int)((0x73261540u >> (4 * ((lane >> 2) & 7))) & 7u) + ((lane >> 1) & 1);
    const float sign = sgn ? -1.0f : 1.0f;
    // A lane past the end of its run gathers zeros: from the slot behind the tile's rows that lies in the class of its
    // column (slots 248 .. 255 are all zero when a tile has 248 rows at most), so that it stays out of the way of the
    // pass's other columns -- the packer counts on that; taller tiles have the one zero slot.
    const uint32_t zero_word = (uint32_t)(a.tile_rows <= kMaxTileRows - 7 ? kMaxTileRows - 7 + (c16 & 7) : kSentinel) * 0x01010101u;
    const uint32_t* stream = a.w0.stream;
    // where this lane's run of the unit with descriptor d and chunk offset c starts, and its dwords
    auto run_of = [&](uint32_t d, uint32_t c, uint32_t& start, int& len) {
        const int pd = run_pos_dwords(d), nd = run_neg_dwords(d);
        start = c + (d >> 16) + (sgn ? (uint32_t)pd : 0u);
        len = sgn ? nd : pd;
    };
    auto load_pieces = [&](u32x4 (&p)[NP], uint32_t start) {
#pragma unroll
        for (int j = 0; j < NP; ++j)  // dword-aligned 16-byte loads; what lies past the run is never used
            p[j] = *reinterpret_cast<const u32x4_a4*>(stream + start + 4 * j);
    };
    uint32_t c_cur = cs_a, c_nxt = u0 + 1 <= last ? cs_b : cs_a, c_nx2 = u0 + 2 <= last ? cs_c : c_nxt, d_cur, d_nxt;
    u32x4 p_cur[NP], p_nxt[NP];
    // (straight-line code, every load unconditional: a wave without units reads what a neighbour reads; the waits are
    // then counted exactly, and nothing below waits for more than it needs)
    d_cur = stream[c_cur + c16];
    d_nxt = stream[c_nxt + c16];
    // every 64th byte of the first two chunks, so that the runs behind their descriptors come from the cache (a chunk
    // that is not this wave's has length 0 here: cs_b and cs_c are table entries only as far as the wave's units go)
    const uint32_t len_a = u0 < u1 ? cs_b - cs_a : 0u, len_b = u0 + 1 <= last ? cs_c - cs_b : 0u;
    const uint32_t touched = stream[c_cur + min((uint32_t)lane * 16u, max(len_a, 1u) - 1u)];
    const uint32_t touched2 = stream[c_nxt + min((uint32_t)lane * 16u, max(len_b, 1u) - 1u)];
    // the first unit's runs: asked for behind the image's loads, as soon as its descriptor is here
    auto first_pieces = [&]() {
        uint32_t start;
        int len;
        run_of(d_cur, c_cur, start, len);
        load_pieces(p_nxt, start);
    };
    if constexpr (!ROWS_IN) {   // the image: rows of the K-major activations, zeros behind a tile's rows and behind K
        // (the workgroup's 1024 pieces a turn are two whole tiles: a thread's slot and piece of the slot never change,
        // a turn moves its address two tiles on)
        static_assert(NT == 2 * kTileSlots * VPS, "a turn of the image loop covers two tiles");
        const size_t row_bytes = (size_t)a.ldx * ES;
        const int r = (tid >> 1) & (kTileSlots - 1), v = tid & 1, tsub = wave >> 3;
        const unsigned char* src = static_cast<const unsigned char*>(a.X) + (size_t)m0 * ES + ((size_t)tsub * a.tile_rows + r) * row_bytes + v * 16;
        const size_t step = (size_t)2 * a.tile_rows * row_bytes;
        for (int tile = tsub; tile < T; tile += 2, src += step) {
            if (r < a.tile_rows && tile * a.tile_rows + r < a.K)
                __builtin_amdgcn_global_load_lds((global_ptr)src, (lds_ptr)(image + ((size_t)tile * kTileSlots * VPS + (wave & 7) * 64) * 16), 16, 0, 0);
            else
                *reinterpret_cast<u32x4*>(image + ((size_t)tile * kTileSlots * VPS + (tid & (kTileSlots * VPS - 1))) * 16) = u32x4{0u, 0u, 0u, 0u};
        }
        first_pieces();
    } else {
        constexpr int KV = 16 / ES;  // values of k in a 16-byte piece of a row
        constexpr int RQ = MT / 4;   // row quads of the slot
        constexpr int QB = 32 / RQ;  // bytes of a row quad in a slot
        constexpr int KSTEP = NT / RQ;  // pieces along k from one task of a thread to its next
        static_assert(NT % RQ == 0, "a thread keeps its row quad from task to task");
        // task t: row quad t % RQ, piece t / RQ of the rows; a thread's tasks are t = tid, tid + NT, ...: same four rows, KSTEP pieces on
        const int tasks = (a.K / KV) * RQ, rq = tid % RQ;
        const int row0 = m0 + 4 * rq;
        const bool whole = m0 + MT <= a.M;  // (wave-uniform: the slot has all its rows)
        const size_t row_bytes = (size_t)a.ldx * ES;
        const unsigned char* rp[4];  // the thread's piece of its four rows (rows that do not exist: the last one, zeroed below)
#pragma unroll
        for (int i = 0; i < 4; ++i)  // (a thread without a task reads the last piece: dropped below)
            rp[i] = static_cast<const unsigned char*>(a.X) + (size_t)min(row0 + i, a.M - 1) * row_bytes + (size_t)min(tid / RQ, a.K / KV - 1) * 16;
        u32x4 in[2][4];  // two tasks of a thread in flight
        auto load_task = [&](u32x4 (&v)[4], int turn) {  // (a task past the last reads the thread's first again: dropped below)
            const size_t off = (size_t)(tid + turn * NT < tasks ? turn : 0) * KSTEP * 16;
#pragma unroll
            for (int i = 0; i < 4; ++i) v[i] = *reinterpret_cast<const u32x4*>(rp[i] + off);
        };
        auto store_task = [&](u32x4 (&v)[4], int turn) {
            if (tid + turn * NT >= tasks) return;
            const int kp = tid / RQ + turn * KSTEP, k = kp * KV;
            const int tile = (int)(((unsigned long long)(unsigned)k * a.tile_magic) >> 32);  // k / tile_rows; a piece never straddles tiles
            unsigned char* base = image + (size_t)tile * kTileSlots * 32 + (size_t)(k - tile * a.tile_rows) * 32 + rq * QB;
            if (!whole) {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (row0 + i >= a.M) v[i] = u32x4{0u, 0u, 0u, 0u};
            }
            // Written in k order every thread of a wave would hit the same banks (slots equal modulo 8), 16 to a bank: each
            // thread rotates its values by its piece number first and writes them in the rotated order.
            const int rot = kp & (KV - 1);
            if constexpr (XF16) {
                uint2 out[8];  // out[j]: the four rows' values of k + j
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const uint32_t a0 = v[0][j / 2], a1 = v[1][j / 2], a2 = v[2][j / 2], a3 = v[3][j / 2];
                    // (low halves / high halves of two dwords side by side: one byte permute each)
                    out[j] = (j & 1) ? make_uint2(__builtin_amdgcn_perm(a1, a0, 0x07060302u), __builtin_amdgcn_perm(a3, a2, 0x07060302u))
                                     : make_uint2(__builtin_amdgcn_perm(a1, a0, 0x05040100u), __builtin_amdgcn_perm(a3, a2, 0x05040100u));
                }
#pragma unroll
                for (int sh = 1; sh < 8; sh <<= 1) {
                    uint2 t[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) t[j] = (rot & sh) ? out[(j + sh) & 7] : out[j];
#pragma unroll
                    for (int j = 0; j < 8; ++j) out[j] = t[j];
                }
#pragma unroll
                for (int j = 0; j < 8; ++j) *reinterpret_cast<uint2*>(base + (size_t)((j + rot) & 7) * 32) = out[j];
            } else {
                u32x4 out[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) out[j] = u32x4{v[0][j], v[1][j], v[2][j], v[3][j]};
#pragma unroll
                for (int sh = 1; sh < 4; sh <<= 1) {
                    u32x4 t[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) t[j] = (rot & sh) ? out[(j + sh) & 3] : out[j];
#pragma unroll
                    for (int j = 0; j < 4; ++j) out[j] = t[j];
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) *reinterpret_cast<u32x4*>(base + (size_t)((j + rot) & 3) * 32) = out[j];
            }
        };
        load_task(in[0], 0);
        load_task(in[1], 1);
        // zeros behind a tile's rows and behind K, while the rows are on their way: the slots behind the full height of
        // every tile but the last, and those behind the rows that the last tile has
        {
            const int behind = (kTileSlots - a.tile_rows) * VPS, full = (T - 1) * behind;
            const int rows_last = a.K - (T - 1) * a.tile_rows, count = full + (kTileSlots - rows_last) * VPS;
            for (int i = tid; i < count; i += NT) {
                const int p = i < full ? (i / behind) * kTileSlots * VPS + a.tile_rows * VPS + i % behind
                                       : (T - 1) * kTileSlots * VPS + rows_last * VPS + (i - full);
                *reinterpret_cast<u32x4*>(image + (size_t)p * 16) = u32x4{0u, 0u, 0u, 0u};
            }
        }
        first_pieces();  // (the descriptors were asked for before the rows: they are here first)
        for (int turn = 0; tid + turn * NT < tasks; turn += 2) {
            store_task(in[0], turn);
            if (wave * 64 + (turn + 2) * NT < tasks) load_task(in[0], turn + 2);  // (wave-uniform)
            store_task(in[1], turn + 1);
            if (wave * 64 + (turn + 3) * NT < tasks) load_task(in[1], turn + 3);
        }
    }
    // the blocks this wave sends out at the end (b = wave, wave + 16, ...): what their chained epilogue needs, asked for now
    float4 row_factors = make_float4(1.f, 1.f, 1.f, 1.f);
    ChainOperands early = {{0u, 0u, 0u, 0u}, 0u, 0u};
    if (XF16 && wave < nblk) {
        if (a.chain_sq_in) row_factors = chain_row_factors(a, lane);
        early = chain_operands(a, (b0 + wave) * TL_BLOCK_COLUMNS + (lane >> 2), lane & 3);
    }
    // this wave's share of the image has landed when only the NP loads of its first runs, asked for behind it, are
    // outstanding (the row-major path wrote the image with ordinary stores, which the barrier itself waits for)
    if constexpr (!ROWS_IN) {
        if constexpr (NP == 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
        static_assert(NP == 4 || NP == 6, "the wait counts the loads of the first runs");
    }
    __syncthreads();

    float acc[NA];
#pragma unroll
    for (int e = 0; e < NA; ++e) acc[e] = 0.f;
    auto issue4 = [](u32x4 (&v)[4], const unsigned char* xq, uint32_t word) {
        using lds_cptr = const __attribute__((address_space(3))) void*;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const uint32_t r = (word >> (8 * b)) & 0xffu;
            const uint32_t addr = (uint32_t)reinterpret_cast<uintptr_t>((lds_cptr)(xq + r * (MT * ES)));
            asm volatile("ds_read_b128 %0, %1" : "=v"(v[b]) : "v"(addr) : "memory");
        }
    };
    auto add4 = [&](const u32x4 (&v)[4]) {
#pragma unroll
        for (int b = 0; b < 4; ++b)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if constexpr (XF16) {
                    acc[2 * e] = fmaf(__half2float(__ushort_as_half((unsigned short)(v[b][e] & 0xffffu))), sign, acc[2 * e]);
                    acc[2 * e + 1] = fmaf(__half2float(__ushort_as_half((unsigned short)(v[b][e] >> 16))), sign, acc[2 * e + 1]);
                } else {
                    acc[e] = fmaf(__uint_as_float(v[b][e]), sign, acc[e]);
                }
            }
    };

    for (int u = u0; u < u1; ++u) {
        // the pieces of this unit are here (asked for one unit ago); so is the next unit's descriptor
        uint32_t start;
        int len;
        run_of(d_cur, c_cur, start, len);
#pragma unroll
        for (int j = 0; j < NP; ++j) p_cur[j] = p_nxt[j];
        {
            uint32_t nstart;
            int nlen;
            run_of(d_nxt, c_nxt, nstart, nlen);
            load_pieces(p_nxt, nstart);
        }
        const uint32_t d_nx2 = stream[c_nx2 + c16];
        const uint32_t c_nx3 = cs[min(u + 3, last)];

        const int b = u / T, tl = u - b * T;
        const unsigned char* xq = image + (size_t)tl * kTileSlots * MT * ES + h * 16;
        u32x4 va[4], vb[4];
#pragma unroll
        for (int j = 0; j < NP; ++j) {
            // two dwords at a time, as far as the longest run of the wave goes (the branches are wave-uniform, so the
            // counted waits see the reads they count)
            if (__builtin_amdgcn_ballot_w64(len > 4 * j) == 0) break;
            uint32_t w[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) w[k] = 4 * j + k < len ? p_cur[j][k] : zero_word;  // past the run: four gathers of zero
            issue4(va, xq, w[0]);
            issue4(vb, xq, w[1]);
            quad_wait<4>(va);
            add4(va);
            if (__builtin_amdgcn_ballot_w64(len > 4 * j + 2) != 0) {
                issue4(va, xq, w[2]);
                quad_wait<4>(vb);
                add4(vb);
                issue4(vb, xq, w[3]);
                quad_wait<4>(va);
                add4(va);
            }
            quad_wait<0>(vb);
            add4(vb);
        }
        for (int i = 4 * NP; __builtin_amdgcn_ballot_w64(i < len) != 0; ++i) {  // runs longer than the registers hold
            const uint32_t word = i < len ? stream[start + i] : zero_word;
            issue4(va, xq, word);
            quad_wait<0>(va);
            add4(va);
        }

        if (u + 1 == u1 || (u + 1) / T != b) {
            // last unit of this wave in block b: fold the two signs of a column, leave the sums in slot (wave + b)
#pragma unroll
            for (int e = 0; e < NA; ++e) acc[e] += __shfl_xor(acc[e], 32, 64);
            if (sgn == 0) {
                float4* out = reinterpret_cast<float4*>(slots + (size_t)(wave + b) * kResSlotFloats + c16 * MT + h * NA);
                out[0] = make_float4(acc[0], acc[1], acc[2], acc[3]);
                if constexpr (NA == 8) out[1] = make_float4(acc[4], acc[5], acc[6], acc[7]);
            }
#pragma unroll
            for (int e = 0; e < NA; ++e) acc[e] = 0.f;
        }
        c_cur = c_nxt; c_nxt = c_nx2; c_nx2 = c_nx3;
        d_cur = d_nxt; d_nxt = d_nx2;
    }
    if ((touched ^ touched2) == 0x5a5aa5a5u && a.M < 0) slots[0] = 0.f;  // (never: keeps the cache-warming loads in the program)
    __syncthreads();
    // Block b goes out through wave b % 16: lane = column lane / 4, rows 4 * (lane % 4) .. + 3, the slots of the waves
    // that had units in the block added in wave order.
    for (int b = wave; b < nblk; b += W) {
        const int col = lane >> 2, q = lane & 3;
        // the waves with units in block b, in order: unit x belongs to wave ((x + 1) * W - 1) / U
        const int w_first = ((b * T + 1) * W - 1) / U, w_last = ((b + 1) * T * W - 1) / U;
        const int nb = b0 + b, n = nb * TL_BLOCK_COLUMNS + col;
        if constexpr (!XF16) {
            const float sc = n < a.N ? load_scale(a.w0.scale, a.scale_f16, n) : 0.f;
            // eight fp32 rows: two per lane; the plain product only
            float2 pair = make_float2(0.f, 0.f);
            for (int w = w_first; w <= w_last; ++w)
                if (w * U / W < (w + 1) * U / W) {  // (a wave without units left nothing)
                    const float2 o = *reinterpret_cast<const float2*>(slots + (size_t)(w + b) * kResSlotFloats + col * MT + q * 2);
                    pair.x += o.x; pair.y += o.y;
                }
            if (n < a.N) {
                if (m0 + q * 2 < a.M) store_out(a.Y, a.y_f16, (long long)(m0 + q * 2) * a.ldy + n, pair.x * sc);
                if (m0 + q * 2 + 1 < a.M) store_out(a.Y, a.y_f16, (long long)(m0 + q * 2 + 1) * a.ldy + n, pair.y * sc);
            }
            continue;
        }
        float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int w = w_first; w <= w_last; ++w)
            if (w * U / W < (w + 1) * U / W) {  // (a wave without units left nothing)
                const float4 o = *reinterpret_cast<const float4*>(slots + (size_t)(w + b) * kResSlotFloats + col * MT + q * 4);
                sum.x += o.x; sum.y += o.y; sum.z += o.z; sum.w += o.w;
            }
        if (b >= W) {  // (more than 16 blocks per workgroup: asked for late)
            if (a.chain_sq_in) row_factors = chain_row_factors(a, lane);
            early = chain_operands(a, n, q);
        }
        const float sc = chain_scale(a, n, early);
        if (a.gated) {
            // gate and up column of a pair sit four lanes apart (same rows): the even column's lane writes the four products
            // (the row factor multiplies the scaled sum, as in the plain product that tl_silu_mul_pairs would follow)
            const float f[4] = {row_factors.x, row_factors.y, row_factors.z, row_factors.w};
            const float s4[4] = {sum.x, sum.y, sum.z, sum.w};
            float hh[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float y = n < a.N ? as_output(a.chain_sq_in ? s4[j] * sc * f[j] : s4[j] * sc, a.y_f16) : 0.f;
                const float up = __shfl_xor(y, 4, 64);
                hh[j] = q * 4 + j < a.M ? gate_pair(y, up, a.y_f16) : 0.f;  // zeros in the padding rows of a K-major image
            }
            if (!(col & 1) && n + 1 < a.N) {
                const int m = q * 4;
                if (a.y_kld && a.y_f16 && a.y_kld % 4 == 0 && m + 4 <= a.y_kld && reinterpret_cast<uintptr_t>(a.Y) % 8 == 0) {
                    // four neighbouring rows of one column of the image: one 8-byte store
                    uint2 packed;
                    __half* ph = reinterpret_cast<__half*>(&packed);
#pragma unroll
                    for (int j = 0; j < 4; ++j) ph[j] = __float2half(settled(hh[j]));
                    *reinterpret_cast<uint2*>(static_cast<__half*>(a.Y) + (long long)(n / 2) * a.y_kld + m) = packed;
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        if (m + j < a.M) store_out(a.Y, a.y_f16, a.y_kld ? (long long)(n / 2) * a.y_kld + m + j : (long long)(m + j) * a.ldy + n / 2, hh[j]);
                        else if (m + j < a.y_kld) store_out(a.Y, a.y_f16, (long long)(n / 2) * a.y_kld + m + j, 0.f);
                    }
                }
            }
            continue;
        }
        float out[4] = {sum.x * sc, sum.y * sc, sum.z * sc, sum.w * sc};
        chain_epilogue16(a, nb, n, col, q, out, row_factors, early);
        if (n < a.N) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (q * 4 + j < a.M) store_out(a.Y, a.y_f16, (long long)(q * 4 + j) * a.ldy + n, out[j]);
        }
    }
}

// ---------------------------------------------------------------------------
// One activation row (decode), staged by direct global -> LDS loads.
// ---------------------------------------------------------------------------
// As tl_spmm_quad, for M = 1 and a contiguous, 16-byte aligned activation row whose tiles are whole
// 16-byte pieces: a tile's LDS image [256 slots] is a straight copy of its piece of the row, followed by
// zeros.  One workgroup owns one block of 16 columns; 32 lanes share a column as in tl_spmm_block
// (TP tiles side by side, LW lanes per run, one dword per lane and pass, two tiles' reads issued
// together), and fold their sums with cross-lane shuffles.  When all of K fits the LDS there is a
// single group: every load of the workgroup is in flight at once and nothing is staged twice.
//
// PRO names what produces the row: kProNone, the row lies in memory (copied by direct loads); with the other
// two the workgroup computes it while the chunks are on their way, every workgroup for itself (a row is a
// few thousand values), so that the producer needs no launch and no trip through memory of its own:
//   kProSiluGate  x[k] = silu(in[k]) * in[K + k] for a side-by-side gate | up row `in` of 2K values;
//   kProAddNorm   s = in + in2 (in2 may be null), x = s * rsqrt(mean(s^2) + eps) * norm_w; the first workgroup
//                 also writes s to sum_out (the residual stream of a decoder layer).
//   kProAttnCombine  x = the attention output that tl_decode_attention_split's pieces add up to: per head h,
//                 x[h * HD + d] = sum_s w_s * piece_s[d] with w_s = exp(top_s - top) / sum_s exp(top_s - top) * norm_s
//                 (`in` = the pieces, fp32 [heads][splits][HD + 4]: HD sums, maximum, sum of exponentials).
// Roundings are those of the separate kernels (tl_silu_mul, tl_add_rmsnorm, tl_attn_combine): s, the SiLU and x
// are rounded to the activation type.
constexpr int kProNone = 0, kProSiluGate = 1, kProAddNorm = 2, kProAttnCombine = 3;

// exp(m - top) for the top score m of one piece of a head's cache rows and the top of all of them; a piece without
// rows (m = -inf) weighs nothing
__device__ __forceinline__ float attn_piece_weight(float m, float top) { return m == -INFINITY ? 0.f : __expf(m - top); }

constexpr int kProNormDeferred = 4;  // launcher only: RMSNorm whose factor multiplies the sums (tl_spmv_tiles), else kProAddNorm
constexpr int kProNormSums = 5;      // launcher only: the row comes multiplied by the norm weight, its squares summed in pieces (tl_spmv_tiles alone)

template <bool F16>
__device__ __forceinline__ float round_to_x(float v)
{
    if constexpr (F16) return __half2float(__float2half(v));
    else return v;
}

template <bool XF16, int NT, int PRO = kProNone>
__global__ __launch_bounds__(NT) void tl_spmv_direct(KernelArgs a)
{
    extern __shared__ __align__(16) unsigned char lds[];
    using XT = typename std::conditional<XF16, __half, float>::type;
    constexpr int ES = (int)sizeof(XT);
    constexpr int VE = 16 / ES;                  // values per 16-byte piece
    constexpr int PITCH = kTileSlots + kSpmvImageSkew / ES;  // slots from one tile image to the next: each starts 4 banks further round
    constexpr int PPT = PITCH / VE;              // pieces per tile image
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int TG = a.tiles_per_group;
    const int nb = blockIdx.x;
    const int stage_bytes = a.xs_bytes + a.buf_bytes;
    const int buffers = TG < a.T ? 2 : 1;
    uint32_t* cst = reinterpret_cast<uint32_t*>(lds + buffers * stage_bytes);  // [buffers][TG + 1] chunk starts inside a buffer's chunk copies
    const_u32_ptr cs = as_const(a.w0.chunkstart) + (size_t)nb * a.T;
    const unsigned char* Xb = static_cast<const unsigned char*>(a.X);
    using global_ptr = const __attribute__((address_space(1))) void*;
    using lds_ptr = __attribute__((address_space(3))) void*;
    float inv_rms = 1.0f;  // kProAddNorm: rsqrt(mean(s^2) + eps), known before any tile is staged
    const float* piece_w = nullptr;  // kProAttnCombine: [heads][splits] weights of the pieces, in LDS

    // the 16-byte piece of the row that starts at value k, as the producer makes it
    auto produce = [&](int k) -> u32x4 {
        u32x4 out;
        XT* o = reinterpret_cast<XT*>(&out);
        if constexpr (PRO == kProSiluGate) {
            const u32x4 gv = *reinterpret_cast<const u32x4*>(Xb + (size_t)k * ES);
            const u32x4 uv = *reinterpret_cast<const u32x4*>(Xb + ((size_t)a.K + k) * ES);
            const XT* g = reinterpret_cast<const XT*>(&gv);
            const XT* u = reinterpret_cast<const XT*>(&uv);
#pragma unroll
            for (int e = 0; e < VE; ++e) {
                const float gf = (float)g[e];
                o[e] = XT(round_to_x<XF16>(gf / (1.0f + __expf(-gf))) * (float)u[e]);
            }
        } else if constexpr (PRO == kProAttnCombine) {
            const int hd = a.pro_hd, sp = a.pro_splits;
            const int h = k / hd, d = k - h * hd;  // a piece of VE values never straddles heads (HD is a multiple of VE)
            const float* src = static_cast<const float*>(a.X) + (size_t)h * sp * (hd + 4) + d;
            float f[VE];
#pragma unroll
            for (int e = 0; e < VE; ++e) f[e] = 0.f;
            for (int sidx = 0; sidx < sp; ++sidx) {
                const float w = piece_w[h * sp + sidx];
#pragma unroll
                for (int e4 = 0; e4 < VE; e4 += 4) {
                    const float4 v = *reinterpret_cast<const float4*>(src + (size_t)sidx * (hd + 4) + e4);
                    f[e4] = fmaf(v.x, w, f[e4]);
                    f[e4 + 1] = fmaf(v.y, w, f[e4 + 1]);
                    f[e4 + 2] = fmaf(v.z, w, f[e4 + 2]);
                    f[e4 + 3] = fmaf(v.w, w, f[e4 + 3]);
                }
            }
#pragma unroll
            for (int e = 0; e < VE; ++e) o[e] = XT(f[e]);
        } else {
            const u32x4 xv = *reinterpret_cast<const u32x4*>(Xb + (size_t)k * ES);
            const u32x4 wv = *reinterpret_cast<const u32x4*>(static_cast<const unsigned char*>(a.norm_w) + (size_t)k * ES);
            u32x4 yv = u32x4{0u, 0u, 0u, 0u};
            if (a.X2) yv = *reinterpret_cast<const u32x4*>(static_cast<const unsigned char*>(a.X2) + (size_t)k * ES);
            const XT* x = reinterpret_cast<const XT*>(&xv);
            const XT* y = reinterpret_cast<const XT*>(&yv);
            const XT* w = reinterpret_cast<const XT*>(&wv);
#pragma unroll
            for (int e = 0; e < VE; ++e) {
                const float sv = a.X2 ? round_to_x<XF16>((float)x[e] + (float)y[e]) : (float)x[e];
                o[e] = XT(sv * inv_rms * (float)w[e]);
            }
        }
        return out;
    };

    auto issue = [&](int t, int nt, int which) {
        unsigned char* xs = lds + which * stage_bytes;
        unsigned char* buf = xs + a.xs_bytes;
        const uint32_t lo = cs[t];
        const int vectors = (int)((cs[t + nt] - lo) / 4);
        for (int first = wave * 64; first < vectors; first += NT)
            if (first + lane < vectors)
                __builtin_amdgcn_global_load_lds((global_ptr)(a.w0.stream + lo + (size_t)(first + lane) * 4), (lds_ptr)(buf + (size_t)first * 16), 16, 0, 0);
        if (tid <= nt) cst[which * (TG + 1) + tid] = cs[t + tid] - lo;
    };
    // the tile images of the group: copies of the row's pieces (or what the producer makes of them), zeros behind a tile's rows
    auto stage_row = [&](int t, int nt, int which) {
        unsigned char* xs = lds + which * stage_bytes;
        const int pieces = nt * PPT;  // images lie back to back, PPT pieces each (the last one or two of an image only ever hold zeros)
        for (int first = wave * 64; first < pieces; first += NT) {
            const int p = first + lane, tile = p / PPT, k = (t + tile) * a.tile_rows + (p % PPT) * VE;
            if (p < pieces) {
                const bool real = (p % PPT) * VE < a.tile_rows && k < a.K;
                if constexpr (PRO == kProNone) {
                    if (real)
                        __builtin_amdgcn_global_load_lds((global_ptr)(Xb + (size_t)k * ES), (lds_ptr)(xs + (size_t)first * 16), 16, 0, 0);
                    else
                        *reinterpret_cast<u32x4*>(xs + (size_t)p * 16) = u32x4{0u, 0u, 0u, 0u};
                } else {
                    *reinterpret_cast<u32x4*>(xs + (size_t)p * 16) = real ? produce(k) : u32x4{0u, 0u, 0u, 0u};
                }
            }
        }
    };

    const int lpc_shift = a.lpc_shift, lw_shift = a.lw_shift;
    const int LPC = 1 << lpc_shift, LW = 1 << lw_shift, TP = LPC >> lw_shift;
    // The LW lanes of a run sit side by side, the 16 columns of a tile next to each other, the TP tiles that are worked on
    // together one after the other: with four lanes per run a wave reads one tile, 8 neighbouring columns per half wave
    // -- the lanes that the packer's order of the rows inside runs keeps off each other's LDS banks.
    const int c16 = (tid >> lw_shift) & (TL_BLOCK_COLUMNS - 1), lw = tid & (LW - 1), tp = tid >> (lw_shift + 4);
    float acc[1] = {0.f};
    constexpr int TU = 2;  // tiles of one lane whose LDS reads are issued together

    issue(0, min(TG, a.T), 0);
    if constexpr (PRO == kProAddNorm) {
        // mean square of s = in + in2 over the row, while the chunks are on their way; the first workgroup keeps s
        float* red = reinterpret_cast<float*>(cst + buffers * (TG + 1));  // [NT / 64]
        float ss = 0.f;
        for (int v = tid; v < a.K / VE; v += NT) {
            const u32x4 xv = *reinterpret_cast<const u32x4*>(Xb + (size_t)v * 16);
            u32x4 sv = xv;
            if (a.X2) {
                const u32x4 yv = *reinterpret_cast<const u32x4*>(static_cast<const unsigned char*>(a.X2) + (size_t)v * 16);
                const XT* x = reinterpret_cast<const XT*>(&xv);
                const XT* y = reinterpret_cast<const XT*>(&yv);
                XT* o = reinterpret_cast<XT*>(&sv);
#pragma unroll
                for (int e = 0; e < VE; ++e) o[e] = XT((float)x[e] + (float)y[e]);
            }
            const XT* sp = reinterpret_cast<const XT*>(&sv);
#pragma unroll
            for (int e = 0; e < VE; ++e) ss = fmaf((float)sp[e], (float)sp[e], ss);
            if (nb == 0 && a.sum_out) *reinterpret_cast<u32x4*>(static_cast<unsigned char*>(a.sum_out) + (size_t)v * 16) = sv;
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
        if (lane == 0) red[wave] = ss;
        __syncthreads();
        float total = 0.f;
#pragma unroll
        for (int v = 0; v < NT / 64; ++v) total += red[v];
        inv_rms = rsqrtf(total / (float)a.K + a.eps);
    }
    if constexpr (PRO == kProAttnCombine) {
        // the weight of every piece, while the chunks are on their way
        float* wts = reinterpret_cast<float*>(cst + buffers * (TG + 1));  // [heads][splits]
        const int hd = a.pro_hd, sp = a.pro_splits, heads = a.K / hd;
        for (int h = tid; h < heads; h += NT) {
            const float* stats = static_cast<const float*>(a.X) + (size_t)h * sp * (hd + 4) + hd;
            float top = -INFINITY;
            for (int sidx = 0; sidx < sp; ++sidx) top = fmaxf(top, stats[(size_t)sidx * (hd + 4)]);
            float norm = 0.f;
            for (int sidx = 0; sidx < sp; ++sidx) norm = fmaf(stats[(size_t)sidx * (hd + 4) + 1], attn_piece_weight(stats[(size_t)sidx * (hd + 4)], top), norm);
            const float inv = __builtin_amdgcn_rcpf(norm);  // (tl_spmv_tiles' kNormCombine takes the same steps)
            for (int sidx = 0; sidx < sp; ++sidx) wts[h * sp + sidx] = attn_piece_weight(stats[(size_t)sidx * (hd + 4)], top) * inv;
        }
        piece_w = wts;
        __syncthreads();
    }
    stage_row(0, min(TG, a.T), 0);
    int which = 0;
    for (int t = 0; t < a.T; t += TG, which ^= 1) {
        const int nt = min(TG, a.T - t);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (t + TG < a.T) {
            issue(t + TG, min(TG, a.T - t - TG), which ^ 1);
            stage_row(t + TG, min(TG, a.T - t - TG), which ^ 1);
        }
        const XT* xs = reinterpret_cast<const XT*>(lds + which * stage_bytes);
        const uint32_t* buf = reinterpret_cast<const uint32_t*>(lds + which * stage_bytes + a.xs_bytes);
        const uint32_t* my_cst = cst + which * (TG + 1);
        for (int tl0 = tp; tl0 < nt; tl0 += TP * TU) {
            uint32_t d[TU];
            const uint32_t* run[TU];
#pragma unroll
            for (int u = 0; u < TU; ++u) {
                const int tl = tl0 + u * TP;
                const uint32_t* chunk = buf + my_cst[min(tl, nt - 1)];
                d[u] = tl < nt ? chunk[c16] : 0u;  // tiles past the group: empty run
                run[u] = chunk + (d[u] >> 16);
            }
            uint32_t w[TU];
#pragma unroll
            for (int u = 0; u < TU; ++u)  // lanes past the run's end take an all-sentinel word: four gathers of zero
                w[u] = lw < run_pos_dwords(d[u]) + run_neg_dwords(d[u]) ? run[u][lw] : 0xffffffffu;
#pragma unroll
            for (int u = 0; u < TU; ++u) {
                const int pd = run_pos_dwords(d[u]), tot = pd + run_neg_dwords(d[u]);
                if (u > 0 && __builtin_amdgcn_ballot_w64(tot > 0) == 0) continue;  // no lane of the wave has this tile
                const XT* xt = xs + (size_t)min(tl0 + u * TP, nt - 1) * PITCH;
                gather_add<1, XT>(acc, xt, w[u], lw < pd ? 1.0f : -1.0f);
                for (int i = lw + LW; i < tot; i += LW)  // runs longer than the lane group
                    gather_add<1, XT>(acc, xt, run[u][i], i < pd ? 1.0f : -1.0f);
            }
        }
    }
    // fold: the LW lanes of a run by shuffles, the TP sums of a column through LDS (no wave may still be gathering from it)
#pragma unroll
    for (int off = 1; off < 64; off <<= 1)
        if (off < LW) acc[0] += __shfl_xor(acc[0], off, 64);
    __syncthreads();
    float* red = reinterpret_cast<float*>(lds);  // [TP][16]
    if (lw == 0) red[tp * TL_BLOCK_COLUMNS + c16] = acc[0];
    __syncthreads();
    if (tid < TL_BLOCK_COLUMNS) {
        float sum = 0.f;
        for (int i = 0; i < TP; ++i) sum += red[i * TL_BLOCK_COLUMNS + tid];
        const int n = nb * TL_BLOCK_COLUMNS + tid;
        if (a.gated) {
            const float y = n < a.N ? as_output(sum * load_scale(a.w0.scale, a.scale_f16, n), a.y_f16) : 0.f;
            const float up = __shfl_xor(y, 1, 64);  // the odd neighbour's
            if (!(tid & 1) && n + 1 < a.N) store_out(a.Y, a.y_f16, n / 2, gate_pair(y, up, a.y_f16));
            return;
        }
        if (n < a.N) store_result(a, n, sum * load_scale(a.w0.scale, a.scale_f16, n));
    }
}

// ---------------------------------------------------------------------------
// One activation row, a tile per wave.
// ---------------------------------------------------------------------------
// tl_spmv_direct with the work cut the other way: a wave owns whole TILES of the workgroup's block (tiles w,
// w + W, ... of W waves), all 16 columns of them, four lanes to a run.  What a wave gathers from -- its tiles' chunks
// and their pieces of the activation row -- it loads itself, so no wave waits for another until the column sums
// are folded at the very end: a wave starts on a tile when that tile's loads have landed (its own vmcnt, no
// barrier), while the loads of later tiles and of the other waves are still in flight.  The kernel's length is
// then about the time the block's bytes take to arrive plus one tile's gather, where tl_spmv_direct, which splits
// a tile's columns over the waves and so needs every wave's loads behind a barrier, adds the whole gather to it.
// With a producer whose operands must arrive and be worked on before the first gather, tl_spmv_direct is the
// faster of the two (the residual add needs a third image in LDS, the normalisation a barrier in the middle).
// The one producer that runs here is an RMSNorm whose factor is DEFERRED (NORM): the row in LDS is
// in[k] * norm_w[k], made by each wave for its own tiles from two direct loads issued ahead of the chunks (waited
// for by count, so the chunks stay in flight), the waves add up in[k]^2 on the side, and rsqrt(mean + eps), one
// number for the whole row, multiplies the column sums at the very end -- no wave waits for another before it
// gathers.  (The row is thus rounded to the activation type as in * norm_w, not as in * factor * norm_w.)
// NORM == 2 is the same product with the two steps in front of the gather taken away: the row arrives already
// multiplied by the norm weight, with the sums of squares of its values in pieces beside it -- what the product
// that made the row leaves in its epilogue (chain_w below) -- so this kernel is the plain one plus a factor at the
// end, with one set of images and as many workgroups to a compute unit as the plain one.

// Waits until at most `later` of this wave's vector-memory instructions are outstanding (they complete in
// order): everything issued before the last `later` has then arrived.  Counts above 13 wait for a few more.
__device__ __forceinline__ void tiles_wait_vm(int later)
{
    switch (later) {
        case 0: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
        case 1: asm volatile("s_waitcnt vmcnt(1)" ::: "memory"); break;
        case 2: asm volatile("s_waitcnt vmcnt(2)" ::: "memory"); break;
        case 3: asm volatile("s_waitcnt vmcnt(3)" ::: "memory"); break;
        case 4: asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); break;
        case 5: asm volatile("s_waitcnt vmcnt(5)" ::: "memory"); break;
        case 6: asm volatile("s_waitcnt vmcnt(6)" ::: "memory"); break;
        case 7: asm volatile("s_waitcnt vmcnt(7)" ::: "memory"); break;
        case 8: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;
        case 9: asm volatile("s_waitcnt vmcnt(9)" ::: "memory"); break;
        case 10: asm volatile("s_waitcnt vmcnt(10)" ::: "memory"); break;
        case 11: asm volatile("s_waitcnt vmcnt(11)" ::: "memory"); break;
        case 12: asm volatile("s_waitcnt vmcnt(12)" ::: "memory"); break;
        default: asm volatile("s_waitcnt vmcnt(13)" ::: "memory"); break;
    }
}

constexpr int kTilesMaxOwn = 8;  // tiles a wave of tl_spmv_tiles may own

constexpr int kNormNone = 0, kNormInside = 1, kNormSums = 2, kNormCombine = 3;

// NORM == kNormCombine: the row is the attention output that the pieces of a split decode attention add up to (the
// layout tl_spmv_direct's kProAttnCombine reads, and its arithmetic, operation for operation).  A wave fetches the
// pieces of its own tiles -- per split 16 bytes (4 rows) per lane, and the (top, norm) pairs of the heads the tile
// touches -- into LDS ahead of its chunks, folds them while the chunks are on their way and writes the tile's image;
// it waits for no other wave.  A wave owns at most kCombineOwn tiles here.
constexpr int kCombineOwn = 2;
constexpr int kCombineStats = 40;  // (top, norm) entries (heads a tile touches x splits) a tile may need, 16 bytes each

// EPI: what the epilogue does, as far as the launcher knows it when it picks the kernel.  kEpiAny looks at the
// arguments; kEpiNone has no scale, residual row or next norm's weight to read and is built without that code (it
// would stand in front of the plain product's first loads); the others are the decoder's three epilogues with every
// operand a row of halves: a scale alone, a scale and the SiLU gate, a scale + residual row + next norm's weight.
constexpr int kEpiNone = 0, kEpiAny = 1, kEpiScale = 2, kEpiGated = 3, kEpiChain = 4;

template <bool XF16, int NT, int NORM = kNormNone, int EPI = kEpiAny>
__global__ __launch_bounds__(NT) void tl_spmv_tiles(KernelArgs a)
{
    constexpr bool OPERANDS = EPI != kEpiNone;
    constexpr bool FIXED = EPI >= kEpiScale;  // the set of operands and their types are known here
    const bool has_scale = FIXED ? true : a.w0.scale != nullptr;
    const bool has_residual = EPI == kEpiChain ? true : EPI == kEpiAny ? a.residual != nullptr : false;
    const bool has_next = EPI == kEpiChain ? true : EPI == kEpiAny ? a.chain_w != nullptr : false;
    const bool gated = EPI == kEpiGated ? true : EPI <= kEpiAny ? a.gated != 0 : false;
    const int scale_f16 = FIXED ? 1 : a.scale_f16, y_f16 = FIXED ? 1 : a.y_f16;
    extern __shared__ __align__(16) unsigned char lds[];
    using XT = typename std::conditional<XF16, __half, float>::type;
    constexpr int ES = (int)sizeof(XT);
    constexpr int VE = 16 / ES;                  // values per 16-byte piece
    constexpr int PITCH = kTileSlots + kSpmvImageSkew / ES;  // slots from one tile image to the next
    constexpr int W = NT / 64;                   // waves
    constexpr int kMaxOwn = NORM == kNormCombine ? kCombineOwn : kTilesMaxOwn;  // tiles a wave may own (the launcher holds T to W * kMaxOwn)
    constexpr bool NORMED = NORM == kNormInside || NORM == kNormSums;  // the sums are multiplied by the row's 1/rms at the end
    constexpr bool ROW_MADE = NORM == kNormInside || NORM == kNormCombine;  // the images are made here, not copied from the row
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nb = blockIdx.x;
    const_u32_ptr cs = as_const(a.w0.chunkstart) + (size_t)nb * a.T;
    const unsigned char* Xb = static_cast<const unsigned char*>(a.X);
    unsigned char* xs = lds;                     // [T] tile images
    unsigned char* buf = lds + a.xs_bytes;       // the block's chunks, as they lie in the stream
    float* red = reinterpret_cast<float*>(lds + a.xs_bytes + a.buf_bytes);  // [W][16] column sums of the waves, then [W] sums of squares
    unsigned char* weights = reinterpret_cast<unsigned char*>(red + ((W * (TL_BLOCK_COLUMNS + 1) + 3) & ~3));  // NORM: [T] images of norm_w
    using global_ptr = const __attribute__((address_space(1))) void*;
    using lds_ptr = __attribute__((address_space(3))) void*;
    const uint32_t base = cs[0];
    // (the table entries of this wave's first tile are asked for together with the block's first: what stands
    // between here and the tile loop then runs while they are on their way.  Asking for those of all its tiles here
    // made the decoder's step 3 % slower, in one batch behind the first tile's loads 2 %.)
    const int first_tile = OPERANDS ? min(wave, a.T - 1) : 0;
    const uint32_t first_lo = OPERANDS ? cs[first_tile] : 0u, first_hi = OPERANDS ? cs[first_tile + 1] : 0u;

    // What the epilogue's 16 lanes need from memory besides the sums -- the column's scale, the residual value, the
    // next norm's weight -- is asked for here, ahead of everything else: a load at the end would add its trip to
    // memory to the launch.  (Kept as loaded: a conversion here would wait for the value.  Issued behind the wave's
    // tile loads instead, the decoder's step was 1.6 % slower.)
    uint32_t raw_scale = 0u, raw_residual = 0u, raw_next_w = 0u;
    if (OPERANDS && tid < TL_BLOCK_COLUMNS && nb * TL_BLOCK_COLUMNS + tid < a.N) {
        const int n = nb * TL_BLOCK_COLUMNS + tid;
        if (has_scale) raw_scale = load_raw(a.w0.scale, scale_f16, n);
        if (has_residual) raw_residual = load_raw(a.residual, y_f16, n);
        if (has_next) raw_next_w = load_raw(a.chain_w, y_f16, n);
    }

    float squares = 0.f;  // this lane's share of sum(in^2): of the row itself (kNormInside), of the sums that came with it (kNormSums)
    if constexpr (NORM == kNormSums) {
        // One number per 16 values of the row, shared out over the threads: loads issued ahead of every load that
        // is waited for by count, their values first used after the last tile (no wave waits for them here).
        const int blocks = a.chain_sq_blocks;
        const float s0 = tid < blocks ? a.chain_sq_in[tid] : 0.f;
        const float s1 = tid + NT < blocks ? a.chain_sq_in[tid + NT] : 0.f;
        squares = s0 + s1;
        for (int i = tid + 2 * NT; i < blocks; i += NT) squares += a.chain_sq_in[i];  // (K above 16 * 2 * NT)
    }
    float* pcs = reinterpret_cast<float*>(weights);  // kNormCombine: [T][splits][256] values of the pieces, a tile's rows side by side
    unsigned char* stats = weights + (size_t)a.T * a.pro_splits * (kTileSlots * 4) + (size_t)wave * (kCombineOwn * kCombineStats * 16);  // this wave's [kCombineOwn][kCombineStats] entries
    if constexpr (NORM == kNormCombine) {
        // the pieces of this wave's tiles, ahead of every chunk (k / head width by multiplication; offsets in 32 bits:
        // the launcher holds the pieces to 2^31 bytes)
        const int S = a.pro_splits, hd = a.pro_hd, pitch = hd + 4;
        const float* pieces = static_cast<const float*>(a.X);
        const int stat_at = lane * pitch + hd;  // lane l asks for the l-th (top, norm) entry from the tile's first head on
#pragma unroll
        for (int j = 0; j < kMaxOwn; ++j) {
            const int t = wave + j * W;
            if (t < a.T) {
                const int k0 = t * a.tile_rows, rows_here = min(a.tile_rows, a.K - k0);
                const int k = k0 + lane * 4, h = (int)__umulhi((unsigned)k, a.tile_magic);
                const float* src = pieces + (unsigned)(h * (S - 1) * pitch + h * 4 + k);  // (h * S) * pitch + (k - h * hd)
                float* dst = pcs + (unsigned)(t * S) * kTileSlots;
                for (int sidx = 0; sidx < S; ++sidx)
                    if (lane * 4 < rows_here)
                        __builtin_amdgcn_global_load_lds((global_ptr)(src + (unsigned)(sidx * pitch)), (lds_ptr)(dst + sidx * kTileSlots), 16, 0, 0);
                const int h0 = (int)__umulhi((unsigned)k0, a.tile_magic), nh = (int)__umulhi((unsigned)(k0 + rows_here - 1), a.tile_magic) - h0 + 1;
                if (lane < nh * S)
                    __builtin_amdgcn_global_load_lds((global_ptr)(pieces + (unsigned)(h0 * S * pitch + stat_at)), (lds_ptr)(stats + j * (kCombineStats * 16)), 16, 0, 0);
            }
        }
    }
    if constexpr (NORM == kNormInside) {
        // the row and the norm weight of this wave's tiles, ahead of every chunk
#pragma unroll
        for (int j = 0; j < kMaxOwn; ++j) {
            const int t = wave + j * W;
            if (t < a.T && lane * VE < min(a.tile_rows, a.K - t * a.tile_rows)) {
                const size_t k = (size_t)t * a.tile_rows + (size_t)lane * VE, image = (size_t)t * PITCH * ES;
                __builtin_amdgcn_global_load_lds((global_ptr)(Xb + k * ES), (lds_ptr)(xs + image), 16, 0, 0);
                __builtin_amdgcn_global_load_lds((global_ptr)(static_cast<const unsigned char*>(a.norm_w) + k * ES), (lds_ptr)(weights + image), 16, 0, 0);
            }
        }
    }

    // every load of this wave, tile after tile; loads[j] = vector-memory instructions of its j-th tile
    int loads[kMaxOwn];
#pragma unroll
    for (int j = 0; j < kMaxOwn; ++j) {
        loads[j] = 0;
        const int t = wave + j * W;
        if (t < a.T) {
            const uint32_t lo = OPERANDS && j == 0 ? first_lo : cs[t];
            const int vectors = (int)(((OPERANDS && j == 0 ? first_hi : cs[t + 1]) - lo) / 4);
            unsigned char* dst = buf + (size_t)(lo - base) * 4;
            for (int first = 0; first < vectors; first += 64) {
                if (first + lane < vectors)
                    __builtin_amdgcn_global_load_lds((global_ptr)(a.w0.stream + lo + (size_t)(first + lane) * 4), (lds_ptr)(dst + (size_t)first * 16), 16, 0, 0);
                ++loads[j];
            }
            // the tile's piece of the row: pieces of rows that exist are copied, the rest of the 256 slots (the zero
            // slot among them) is zeroed
            const int rows_here = min(a.tile_rows, a.K - t * a.tile_rows);
            unsigned char* image = xs + (size_t)t * PITCH * ES;
            if constexpr (!ROW_MADE) {
                if (lane * VE < rows_here)
                    __builtin_amdgcn_global_load_lds((global_ptr)(Xb + ((size_t)t * a.tile_rows + (size_t)lane * VE) * ES), (lds_ptr)image, 16, 0, 0);
                ++loads[j];
            }
            if (lane * VE >= rows_here && lane * VE < kTileSlots) *reinterpret_cast<u32x4*>(image + (size_t)lane * 16) = u32x4{0u, 0u, 0u, 0u};
        }
    }

    if constexpr (NORM == kNormInside) {
        int chunk_loads = 0;
#pragma unroll
        for (int j = 0; j < kMaxOwn; ++j) chunk_loads += loads[j];
        tiles_wait_vm(chunk_loads);  // row and weight pieces are here when only the chunk loads are outstanding
#pragma unroll 1
        for (int t = wave; t < a.T; t += W) {
            if (lane * VE < min(a.tile_rows, a.K - t * a.tile_rows)) {
                const size_t at = (size_t)t * PITCH * ES + (size_t)lane * 16;
                u32x4 v = *reinterpret_cast<const u32x4*>(xs + at);
                const u32x4 wv = *reinterpret_cast<const u32x4*>(weights + at);
                XT* x = reinterpret_cast<XT*>(&v);
                const XT* w = reinterpret_cast<const XT*>(&wv);
#pragma unroll
                for (int e = 0; e < VE; ++e) {
                    const float f = (float)x[e];
                    squares = fmaf(f, f, squares);
                    x[e] = XT(f * (float)w[e]);
                }
                *reinterpret_cast<u32x4*>(xs + at) = v;
            }
        }
    }

    if constexpr (NORM == kNormCombine) {
        int chunk_loads = 0;
#pragma unroll
        for (int j = 0; j < kMaxOwn; ++j) chunk_loads += loads[j];
        tiles_wait_vm(chunk_loads);  // the pieces are here when only the chunk loads are outstanding
        // SC: the number of pieces per head where the code is built for it (their weights then stay in registers), 0: any
        auto fold = [&](auto SC) {
            constexpr int SK = decltype(SC)::value;
            const int S = SK ? SK : a.pro_splits;
#pragma unroll
            for (int j = 0; j < kMaxOwn; ++j) {
                const int t = wave + j * W;
                if (t < a.T) {
                    const int k0 = t * a.tile_rows;
                    if (lane * VE < min(a.tile_rows, a.K - k0)) {
                        // the piece of VE values never straddles heads (the head width is a multiple of VE)
                        const int hh = (int)__umulhi((unsigned)(k0 + lane * VE), a.tile_magic) - (int)__umulhi((unsigned)k0, a.tile_magic);
                        const float4* st = reinterpret_cast<const float4*>(stats + j * (kCombineStats * 16)) + hh * S;
                        const float* p = pcs + (unsigned)(t * S) * kTileSlots + lane * VE;
                        float f[VE];
#pragma unroll
                        for (int e = 0; e < VE; ++e) f[e] = 0.f;
                        auto add_piece = [&](int sidx, float w) {
#pragma unroll
                            for (int e4 = 0; e4 < VE; e4 += 4) {
                                const float4 v = *reinterpret_cast<const float4*>(p + sidx * kTileSlots + e4);
                                f[e4] = fmaf(v.x, w, f[e4]);
                                f[e4 + 1] = fmaf(v.y, w, f[e4 + 1]);
                                f[e4 + 2] = fmaf(v.z, w, f[e4 + 2]);
                                f[e4 + 3] = fmaf(v.w, w, f[e4 + 3]);
                            }
                        };
                        float top = -INFINITY, norm = 0.f;
                        if constexpr (SK != 0) {
                            float ex[SK ? SK : 1];
#pragma unroll
                            for (int sidx = 0; sidx < SK; ++sidx) top = fmaxf(top, st[sidx].x);
#pragma unroll
                            for (int sidx = 0; sidx < SK; ++sidx) {
                                const float4 e = st[sidx];
                                ex[sidx] = attn_piece_weight(e.x, top);
                                norm = fmaf(e.y, ex[sidx], norm);
                            }
                            const float inv = __builtin_amdgcn_rcpf(norm);
#pragma unroll
                            for (int sidx = 0; sidx < SK; ++sidx) add_piece(sidx, ex[sidx] * inv);
                        } else {
                            for (int sidx = 0; sidx < S; ++sidx) top = fmaxf(top, st[sidx].x);
                            for (int sidx = 0; sidx < S; ++sidx) {
                                const float4 e = st[sidx];
                                norm = fmaf(e.y, attn_piece_weight(e.x, top), norm);
                            }
                            const float inv = __builtin_amdgcn_rcpf(norm);
                            for (int sidx = 0; sidx < S; ++sidx) add_piece(sidx, attn_piece_weight(st[sidx].x, top) * inv);
                        }
                        u32x4 out;
                        XT* o = reinterpret_cast<XT*>(&out);
#pragma unroll
                        for (int e = 0; e < VE; ++e) o[e] = XT(f[e]);
                        *reinterpret_cast<u32x4*>(xs + (size_t)t * PITCH * ES + (size_t)lane * 16) = out;
                    }
                }
            }
        };
        if (a.pro_splits == 2) fold(std::integral_constant<int, 2>());
        else if (a.pro_splits == 4) fold(std::integral_constant<int, 4>());
        else fold(std::integral_constant<int, 0>());
    }

    const int c16 = lane >> 2, lw = lane & 3;
    float acc[1] = {0.f};
#pragma unroll
    for (int j = 0; j < kMaxOwn; ++j) {
        const int t = wave + j * W;
        if (t < a.T) {
            int later = 0;  // loads issued after this tile's
#pragma unroll
            for (int q = j + 1; q < kMaxOwn; ++q) later += loads[q];
            tiles_wait_vm(later);
            const uint32_t* chunk = reinterpret_cast<const uint32_t*>(buf) + (cs[t] - base);
            const uint32_t d = chunk[c16];
            const uint32_t* run = chunk + (d >> 16);
            const int pd = run_pos_dwords(d), tot = pd + run_neg_dwords(d);
            const XT* xt = reinterpret_cast<const XT*>(xs) + (size_t)t * PITCH;
            for (int i = lw; i < tot; i += 4) gather_add<1, XT>(acc, xt, run[i], i < pd ? 1.0f : -1.0f);
        }
    }
    acc[0] += __shfl_xor(acc[0], 1, 64);
    acc[0] += __shfl_xor(acc[0], 2, 64);
    if (lw == 0) red[wave * TL_BLOCK_COLUMNS + c16] = acc[0];
    if constexpr (NORMED) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) squares += __shfl_xor(squares, off, 64);
        if (lane == 0) red[W * TL_BLOCK_COLUMNS + wave] = squares;
    }
    __syncthreads();
    if (tid < TL_BLOCK_COLUMNS) {
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < W; ++w) sum += red[w * TL_BLOCK_COLUMNS + tid];
        if constexpr (NORMED) {
            float total = 0.f;
#pragma unroll
            for (int w = 0; w < W; ++w) total += red[W * TL_BLOCK_COLUMNS + w];
            sum *= rsqrtf(total / (float)a.K + a.eps);
        }
        const int n = nb * TL_BLOCK_COLUMNS + tid;
        const float col_scale = OPERANDS && has_scale ? raw_value(raw_scale, scale_f16) : 1.0f;
        const float col_residual = raw_value(raw_residual, y_f16), col_next_w = raw_value(raw_next_w, y_f16);
        if (gated) {
            const float y = n < a.N ? as_output(sum * col_scale, y_f16) : 0.f;
            const float up = __shfl_xor(y, 1, 64);  // the odd neighbour's
            if (!(tid & 1) && n + 1 < a.N) store_out(a.Y, y_f16, n / 2, gate_pair(y, up, y_f16));
            return;
        }
        float v = sum * col_scale;
        if (has_residual) v = as_output(v, y_f16) + col_residual;  // (as store_result adds it)
        if (has_next) {
            // The row goes on into an RMSNorm and a product: leave it multiplied by that norm's weight (rounded as the
            // norm inside the next kernel would round it) and the block's share of the sum of its squares beside the
            // row itself, so that the next product starts as a plain one (kNormSums).
            float y = 0.f;
            if (n < a.N) {
                y = as_output(v, y_f16);
                store_out(a.Y, y_f16, n, v);
                store_out(a.chain_image, y_f16, n, y * col_next_w);
            }
            float q = y * y;
#pragma unroll
            for (int off = 1; off < TL_BLOCK_COLUMNS; off <<= 1) q += __shfl_xor(q, off, 64);
            if (tid == 0) a.chain_sq_out[nb] = q;
            return;
        }
        if (n < a.N) store_out(a.Y, y_f16, n, v);
    }
}

// out[k][m] = x(m, k) for m < M, zero for M <= m < ldo (ldo <= 48), from activations of any layout
// (element strides sm, sk): the aligned K-major image the small-M kernel copies as vectors.
// A workgroup moves 64 values of k.
template <typename T>
__global__ __launch_bounds__(256) void tl_to_kmajor(const T* __restrict__ X, long long sm, long long sk, T* __restrict__ out, int ldo, int M, int K)
{
    __shared__ T tile[48][65];
    const int k0 = blockIdx.x * 64;
    T v[12];
#pragma unroll
    for (int i = 0; i < 12; ++i) {
        const int idx = threadIdx.x + i * 256, m = idx >> 6, k = k0 + (idx & 63);
        v[i] = (m < M && k < K) ? X[(size_t)m * sm + (size_t)k * sk] : T(0.0f);
    }
#pragma unroll
    for (int i = 0; i < 12; ++i) {
        const int idx = threadIdx.x + i * 256, m = idx >> 6;
        if (m < ldo) tile[m][idx & 63] = v[i];
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < 64 * ldo; idx += 256) {
        const int kk = idx / ldo, m = idx - kk * ldo;
        if (k0 + kk < K) out[(size_t)(k0 + kk) * ldo + m] = tile[m][kk];
    }
}

// LDS one workgroup of the small-M kernel may use: two workgroups fit a compute unit's 160 KB; a launch
// with no more workgroups than compute units lets each have (nearly) all of it.
constexpr int kSmallLdsShared = 78 * 1024;
constexpr int kSmallLdsAlone = 158 * 1024;

template <int MT, bool XF16>
int launch_block_kernel(KernelArgs a, const tl_layout_header* h, hipStream_t st)
{
    constexpr int es = XF16 ? 2 : 4;
    using Shape = BlockShape<MT, es, kBlockThreads>;
    const int tile_bytes = kTileSlots * MT * es;
    const int64_t chunk_bytes = (int64_t)h->max_chunk_dwords * 4;
    if (chunk_bytes * a.block_set > Shape::kStreamCap) return fail(TL_ERR_UNSUPPORTED, "a tile's chunks do not fit the staging registers");
    const unsigned gx = (unsigned)ceil_div(a.NB, a.block_set), gy = (unsigned)ceil_div(a.M, MT);
    const int budget = knob(TL_SMALL_LDS, (int64_t)gx * gy <= compute_units() ? kSmallLdsAlone : kSmallLdsShared);
    // tiles per group: bounded by the registers of the staging (Shape), by the LDS budget shared between
    // the activation image and the chunk copies, and by the stream bytes one group may hold
    const int per_tile = tile_bytes + (int)chunk_bytes * a.block_set;
    int tg = std::min(Shape::kTiles, (budget - 1024) / per_tile);
    tg = std::min(tg, (int)(Shape::kStreamCap / (chunk_bytes * a.block_set)));
    tg = std::max(1, std::min(std::min(tg, a.T), 255));
    tg = std::max(1, std::min(tg, knob(TL_TILE_GROUP, tg)));
    tg = (int)ceil_div(a.T, ceil_div(a.T, tg));  // same number of groups, evened out
    a.tiles_per_group = tg;
    a.xs_bytes = tg * tile_bytes;
    a.buf_bytes = (int)round_up(std::min<int64_t>(chunk_bytes * a.block_set * tg, Shape::kStreamCap), 16);
    const size_t lds = (size_t)a.xs_bytes + a.buf_bytes + (size_t)kMaxBlockSet * (tg + 1) * 4;
    if (lds > 160 * 1024) return fail(TL_ERR_UNSUPPORTED, "one tile of %d rows needs %zu bytes of LDS", MT, lds);
    auto kernel = tl_spmm_block<MT, XF16>;
    static bool raised = false;  // per instantiation; a repeated or racing call is harmless
    if (!raised) {
        if (int rc = raise_lds_limit(kernel, 160 * 1024)) return rc;
        raised = true;
    }
    hipLaunchKernelGGL(kernel, dim3(gx, gy), dim3(kBlockThreads), lds, st, a);
    return TL_OK;
}

inline int log2_exact(int v)
{
    int s = 0;
    while ((1 << s) < v) ++s;
    return s;
}

// The direct-load kernel for 8- and 16-row slots.  Its LDS holds two buffers of TG tiles (activation image +
// chunk copies); TG is sized so that `share` workgroups fit a compute unit, as many as the launch can
// give each compute unit, up to four.
template <int MT, bool XF16, int NT = kBlockThreads>
int launch_quad_kernel(KernelArgs a, const tl_layout_header* h, hipStream_t st)
{
    constexpr int es = XF16 ? 2 : 4;
    constexpr int groups = NT / (TL_BLOCK_COLUMNS * (MT / 4));  // lane groups per column
    const int tile_bytes = kTileSlots * MT * es;
    const int chunk_bytes = (int)h->max_chunk_dwords * 4;
    const unsigned gx = (unsigned)a.NB, gy = (unsigned)ceil_div(a.M, MT);
    const int share = std::max(1, std::min(knob(TL_QUAD_SHARE, 4), (int)ceil_div((int64_t)gx * gy, compute_units())));
    const int budget = 160 * 1024 / share - 1024;
    int tg = std::max(1, std::min(a.T, (budget - 256) / (2 * (tile_bytes + chunk_bytes))));
    tg = std::max(1, std::min(tg, knob(TL_TILE_GROUP, tg)));
    tg = (int)ceil_div(a.T, ceil_div(a.T, tg));  // same number of groups, evened out
    a.tiles_per_group = tg;
    a.xs_bytes = tg * tile_bytes;
    a.buf_bytes = (int)round_up((int64_t)tg * chunk_bytes, 16);
    const size_t lds = std::max<size_t>(2 * ((size_t)a.xs_bytes + a.buf_bytes) + 2 * (size_t)(tg + 1) * 4, (size_t)NT * 16);
    if (lds > 160 * 1024) return fail(TL_ERR_UNSUPPORTED, "two tiles of %d rows need %zu bytes of LDS", MT, lds);
    // lane groups per run: a run's dwords go round the LW groups, four per group and turn; no more
    // tiles side by side than a group of tiles has
    const double mean_run = h->mean_run_dwords_x16 / 16.0;
    int lw = 2;
    while (lw < groups && lw * (NT > kBlockThreads ? 16 : 8) < mean_run) lw *= 2;  // the wide workgroup has tiles enough side by side
    while (groups / lw > tg) lw *= 2;
    lw = std::min(knob(TL_LW, lw), groups);
    if (lw < 1 || (lw & (lw - 1))) return fail(TL_ERR_ARG, "TL_LW=%d (a power of two expected)", lw);
    a.lpc_shift = log2_exact(groups);
    a.lw_shift = log2_exact(lw);
    auto kernel = tl_spmm_quad<MT, XF16, NT>;
    static bool raised = false;  // per instantiation; a repeated or racing call is harmless
    if (!raised) {
        if (int rc = raise_lds_limit(kernel, 160 * 1024)) return rc;
        raised = true;
    }
    hipLaunchKernelGGL(kernel, dim3(gx, gy), dim3(NT), lds, st, a);
    return TL_OK;
}

// tl_spmm_octet: two blocks per workgroup, LDS sized for up to three workgroups per compute unit.
int launch_octet_kernel(KernelArgs a, const tl_layout_header* h, hipStream_t st)
{
    constexpr int groups = kBlockThreads / 64;  // lane groups: one per wave
    const int tile_bytes = kTileSlots * 16 * 2;
    const int chunk_bytes = (int)h->max_chunk_dwords * 4;
    const unsigned gx = (unsigned)ceil_div(a.NB, 2), gy = (unsigned)ceil_div(a.M, 16);
    const int share = std::max(1, std::min(knob(TL_QUAD_SHARE, 3), (int)ceil_div((int64_t)gx * gy, compute_units())));
    const int budget = 160 * 1024 / share - 1024;
    const int per_tile = tile_bytes + 2 * chunk_bytes;
    int tg = std::max(1, std::min(a.T, (budget - 256) / (2 * per_tile)));
    tg = std::max(1, std::min(tg, knob(TL_TILE_GROUP, tg)));
    tg = (int)ceil_div(a.T, ceil_div(a.T, tg));  // same number of groups, evened out
    a.tiles_per_group = tg;
    a.xs_bytes = tg * tile_bytes;
    a.buf_bytes = 2 * (int)round_up((int64_t)tg * chunk_bytes, 16);
    const size_t lds = std::max<size_t>(2 * ((size_t)a.xs_bytes + a.buf_bytes) + 2 * 2 * (size_t)(tg + 1) * 4, (size_t)kBlockThreads * 32);
    if (lds > 160 * 1024) return fail(TL_ERR_UNSUPPORTED, "two tiles of 16 rows and two blocks need %zu bytes of LDS", lds);
    const double mean_run = h->mean_run_dwords_x16 / 16.0;
    int lw = 2;
    while (lw < groups && lw * 8 < mean_run) lw *= 2;
    while (groups / lw > tg) lw *= 2;
    lw = std::min(knob(TL_LW, lw), groups);
    if (lw < 1 || (lw & (lw - 1))) return fail(TL_ERR_ARG, "TL_LW=%d (a power of two expected)", lw);
    a.lpc_shift = log2_exact(groups);
    a.lw_shift = log2_exact(lw);
    static bool raised = false;  // a repeated or racing call is harmless
    if (!raised) {
        if (int rc = raise_lds_limit(tl_spmm_octet, 160 * 1024)) return rc;
        raised = true;
    }
    hipLaunchKernelGGL(tl_spmm_octet, dim3(gx, gy), dim3(kBlockThreads), lds, st, a);
    return TL_OK;
}

// tl_spmm_res: one workgroup per compute unit, each with a range of whole blocks of one slot of rows (16 fp16 or 8
// fp32 rows; the slots of a taller input share the compute units out among themselves).  It fits when the image of
// all of K and the slots of the block sums fit the LDS, and the runs are short enough for a lane's registers.
struct ResShape {
    int parts;       // slots of rows
    int groups;      // workgroups per slot
    int pieces;      // 16-byte pieces of a run in a lane's registers (4 or 6), 0: does not fit
    size_t lds;
};

inline ResShape res_shape(const KernelArgs& a, const tl_layout_header* h)
{
    ResShape r;
    const int rows = a.x_f16 ? 16 : 8;
    r.parts = (int)ceil_div(a.M, rows);
    r.groups = std::max(1, std::min(compute_units() / r.parts, a.NB));
    const int nblk_max = (int)ceil_div(a.NB, r.groups);
    r.lds = (size_t)a.T * kTileSlots * 32 + (size_t)(kResWaves + nblk_max - 1) * TL_BLOCK_COLUMNS * rows * 4;
    // a lane keeps 16 or 24 dwords (64 or 96 rows) of a run in registers and fetches the rest one by one: the mean
    // run of one sign (half of the header's figure, which counts both) should stay well below that
    r.pieces = h->mean_run_dwords_x16 <= 16 * 26 ? 4 : (h->mean_run_dwords_x16 <= 16 * 40 ? 6 : 0);
    if (r.lds > 160 * 1024 || r.parts > 3 || r.parts > compute_units()) r.pieces = 0;
    return r;
}

template <bool XF16, int NP, bool ROWS_IN>
int launch_res_np(KernelArgs a, const ResShape& shape, hipStream_t st)
{
    a.xs_bytes = a.T * kTileSlots * 32;
    a.tile_magic = (unsigned)(((1ull << 32) + a.tile_rows - 1) / a.tile_rows);
    auto kernel = tl_spmm_res<XF16, NP, ROWS_IN>;
    static bool raised = false;  // per instantiation; a repeated or racing call is harmless
    if (!raised) {
        if (int rc = raise_lds_limit(kernel, 160 * 1024)) return rc;
        raised = true;
    }
    hipLaunchKernelGGL(kernel, dim3((unsigned)shape.groups, (unsigned)shape.parts), dim3(kResWaves * 64), shape.lds, st, a);
    return TL_OK;
}

// Row-major activations that tl_spmm_res turns into its image itself: rows of whole 16-byte pieces, aligned, and tiles
// of whole pieces (no piece of a row straddles two tiles).
inline bool res_takes_rows(const KernelArgs& a)
{
    const int es = a.x_f16 ? 2 : 4, kv = 16 / es;
    return !a.x_kmajor && (a.ldx * es) % 16 == 0 && reinterpret_cast<uintptr_t>(a.X) % 16 == 0 && a.K % kv == 0 && a.tile_rows % kv == 0 &&
           a.K < (1 << 24);
}

template <bool XF16, bool ROWS_IN>
int launch_res_in(const KernelArgs& a, const ResShape& shape, hipStream_t st)
{
    return shape.pieces == 4 ? launch_res_np<XF16, 4, ROWS_IN>(a, shape, st) : launch_res_np<XF16, 6, ROWS_IN>(a, shape, st);
}

int launch_res_kernel(const KernelArgs& a, const tl_layout_header* h, hipStream_t st)
{
    const ResShape shape = res_shape(a, h);
    if (!a.x_kmajor) return a.x_f16 ? launch_res_in<true, true>(a, shape, st) : launch_res_in<false, true>(a, shape, st);
    return a.x_f16 ? launch_res_in<true, false>(a, shape, st) : launch_res_in<false, false>(a, shape, st);
}

// The direct-load kernel for one activation row.  All of K in one group when `share` workgroups of that
// size fit a compute unit, else two alternating buffers of TG tiles.
template <bool XF16, int NT, int PRO = kProNone>
int launch_spmv_direct_nt(KernelArgs a, const tl_layout_header* h, hipStream_t st)
{
    constexpr int es = XF16 ? 2 : 4;
    const int tile_bytes = kTileSlots * es + kSpmvImageSkew;
    const int chunk_bytes = (int)h->max_chunk_dwords * 4;
    const int share = std::max(1, std::min(knob(TL_SPMV_SHARE, 4), (int)ceil_div(a.NB, compute_units())));
    const int budget = 160 * 1024 / share - 1024;
    int tg = a.T;
    if ((int64_t)a.T * (tile_bytes + chunk_bytes) + 256 > budget) tg = std::max(1, (budget - 256) / (2 * (tile_bytes + chunk_bytes)));
    tg = std::max(1, std::min(tg, knob(TL_TILE_GROUP, tg)));
    tg = (int)ceil_div(a.T, ceil_div(a.T, tg));  // same number of groups, evened out
    a.tiles_per_group = tg;
    a.xs_bytes = tg * tile_bytes;
    a.buf_bytes = (int)round_up((int64_t)tg * chunk_bytes, 16);
    const int buffers = tg < a.T ? 2 : 1;
    // + what a producer keeps: the waves' partial mean squares, or the weights of the attention pieces
    const size_t pro_bytes = PRO == kProAttnCombine ? (size_t)(a.K / std::max(1, a.pro_hd)) * a.pro_splits * 4 : (size_t)(NT / 64) * 4;
    const size_t lds = (size_t)buffers * ((size_t)a.xs_bytes + a.buf_bytes) + (size_t)buffers * (tg + 1) * 4 + pro_bytes;
    if (lds > 160 * 1024) return fail(TL_ERR_UNSUPPORTED, "one tile needs %zu bytes of LDS", lds);
    const int lpc = NT / TL_BLOCK_COLUMNS;
    const double mean_run = h->mean_run_dwords_x16 / 16.0;
    int lw = 4;
    while (lw < lpc && lw * 3 < mean_run) lw *= 2;
    lw = std::min(knob(TL_LW, lw), lpc);
    if (lw < 1 || (lw & (lw - 1))) return fail(TL_ERR_ARG, "TL_LW=%d (a power of two expected)", lw);
    a.lpc_shift = log2_exact(lpc);
    a.lw_shift = log2_exact(lw);
    auto kernel = tl_spmv_direct<XF16, NT, PRO>;
    static bool raised = false;  // per instantiation; a repeated or racing call is harmless
    if (!raised) {
        if (int rc = raise_lds_limit(kernel, 160 * 1024)) return rc;
        raised = true;
    }
    hipLaunchKernelGGL(kernel, dim3((unsigned)a.NB), dim3(NT), lds, st, a);
    return TL_OK;
}

// tl_spmv_tiles: every tile of the block resident (a wave loads its own and waits for nobody else's).
// Returns TL_ERR_UNSUPPORTED when that does not fit; the caller then takes tl_spmv_direct.
template <bool XF16, int NT, int NORM = kNormNone, int EPI = kEpiAny>
int launch_spmv_tiles_nt(KernelArgs a, const tl_layout_header* h, hipStream_t st)
{
    constexpr int es = XF16 ? 2 : 4;
    const int tile_bytes = kTileSlots * es + kSpmvImageSkew;
    const int chunk_bytes = (int)h->max_chunk_dwords * 4;
    if (a.T > (NT / 64) * (NORM == kNormCombine ? kCombineOwn : kTilesMaxOwn)) return TL_ERR_UNSUPPORTED;
    a.xs_bytes = a.T * tile_bytes;
    a.buf_bytes = (int)round_up((int64_t)a.T * chunk_bytes, 16);
    size_t lds = (size_t)a.xs_bytes * (NORM == kNormInside ? 2 : 1) + a.buf_bytes + (size_t)(((NT / 64) * (TL_BLOCK_COLUMNS + 1) + 3) & ~3) * 4;
    if (NORM == kNormCombine) {
        // heads a tile may touch x splits: one 16-byte entry each in the wave's table; k / head width by multiplication
        const int heads_per_tile = (a.tile_rows + a.pro_hd - 2) / a.pro_hd + 1;
        if (heads_per_tile * a.pro_splits > kCombineStats || a.tile_rows % 4 || a.pro_hd % 4 || (int64_t)a.K * a.pro_hd >= (1ll << 32) ||
            (int64_t)(a.K / a.pro_hd) * a.pro_splits * (a.pro_hd + 4) * 4 >= (1ll << 31))
            return TL_ERR_UNSUPPORTED;
        lds += (size_t)a.T * a.pro_splits * (kTileSlots * 4) + (size_t)(NT / 64) * kCombineOwn * kCombineStats * 16;
        a.tile_magic = (unsigned)(((1ull << 32) + a.pro_hd - 1) / a.pro_hd);  // k / head width
    }
    int share = std::max(1, std::min(knob(TL_SPMV_SHARE, 4), (int)ceil_div(a.NB, compute_units())));
    if (NORM == kNormInside) share = std::min(share, 3);  // the second set of images: three workgroups of K = 4096 fit a compute unit, not four
    // (a product that only this kernel serves runs with fewer workgroups to a compute unit rather than not at all)
    if (NORM == kNormSums || a.chain_w) share = 1;
    if (lds > (size_t)(160 * 1024 / share - 1024)) return TL_ERR_UNSUPPORTED;
    auto kernel = tl_spmv_tiles<XF16, NT, NORM, EPI>;
    static bool raised = false;  // per instantiation; a repeated or racing call is harmless
    if (!raised) {
        if (int rc = raise_lds_limit(kernel, 160 * 1024)) return rc;
        raised = true;
    }
    hipLaunchKernelGGL(kernel, dim3((unsigned)a.NB), dim3(NT), lds, st, a);
    return TL_OK;
}

// The epilogue the arguments ask for, among those a kernel is built for.
template <bool XF16>
int tiles_epilogue(const KernelArgs& a)
{
    if (!a.w0.scale && !a.residual && !a.chain_w) return kEpiNone;
    if (XF16 && a.w0.scale && a.scale_f16 && a.y_f16) {
        if (a.gated && !a.residual && !a.chain_w) return kEpiGated;
        if (!a.gated && a.residual && a.chain_w) return kEpiChain;
        if (!a.gated && !a.residual && !a.chain_w) return kEpiScale;
    }
    return kEpiAny;
}

template <bool XF16, int NORM, int EPI>
int launch_spmv_tiles_wide(bool wide, const KernelArgs& a, const tl_layout_header* h, hipStream_t st)
{
    if (wide) return launch_spmv_tiles_nt<XF16, 1024, NORM, EPI>(a, h, st);
    // A ninth wave where it lowers the most tiles a wave owns (K = 4096 is 17 tiles: three for the first of eight waves,
    // two for each of nine) and the workgroups that share a compute unit still fit its 32 waves.  (4096 -> 12288: 9.5
    // against 9.7-9.9 us; with four workgroups to a compute unit, of which only three of nine waves fit, the decoder's
    // step was 3 % slower; the kernel that norms its row itself took 12.3 us with nine waves against 10 with eight.)
    if (NORM != kNormInside && ceil_div(a.NB, compute_units()) <= 3 && ceil_div(a.T, 9) < ceil_div(a.T, 8)) return launch_spmv_tiles_nt<XF16, kBlockThreads + 64, NORM, EPI>(a, h, st);
    return launch_spmv_tiles_nt<XF16, kBlockThreads, NORM, EPI>(a, h, st);
}

// tl_spmv_tiles with the epilogue picked: the plain product and the product on a row with its sums of squares have
// kernels for the decoder's epilogues (fp16 only), everything else takes the one that looks at its arguments.
template <bool XF16, int NORM>
int launch_spmv_tiles(bool wide, const KernelArgs& a, const tl_layout_header* h, hipStream_t st)
{
    const int epi = tiles_epilogue<XF16>(a);
    if constexpr (NORM == kNormCombine && XF16) {
        if (epi == kEpiChain) return launch_spmv_tiles_wide<XF16, NORM, kEpiChain>(wide, a, h, st);
    }
    if constexpr (NORM == kNormNone) {
        if (epi == kEpiNone) return launch_spmv_tiles_wide<XF16, NORM, kEpiNone>(wide, a, h, st);
        if constexpr (XF16) {
            if (epi == kEpiChain) return launch_spmv_tiles_wide<XF16, NORM, kEpiChain>(wide, a, h, st);
            if (epi == kEpiScale) return launch_spmv_tiles_wide<XF16, NORM, kEpiScale>(wide, a, h, st);
        }
    }
    return launch_spmv_tiles_wide<XF16, NORM, kEpiAny>(wide, a, h, st);
}

// With no more blocks than compute units a workgroup has its compute unit to itself: 1024 threads
// (64 lanes per column) then keep more gathers in flight than 512 do.
template <bool XF16, int PRO = kProNone>
int launch_spmv_direct(const KernelArgs& a, const tl_layout_header* h, hipStream_t st)
{
    const bool wide = knob(TL_SPMV_WIDE, a.NB <= compute_units() ? 1 : 0) != 0;
    if constexpr (PRO == kProNormSums) {
        const int rc = launch_spmv_tiles<XF16, kNormSums>(wide, a, h, st);
        if (rc == TL_ERR_UNSUPPORTED) return fail(TL_ERR_UNSUPPORTED, "the weight's blocks do not fit the kernel that takes a row with its sums of squares");
        return rc;
    } else if constexpr (PRO == kProNormDeferred) {
        if (knob(TL_SPMV_TILES, 1) != 0) {
            const int rc = launch_spmv_tiles<XF16, kNormInside>(wide, a, h, st);
            if (rc != TL_ERR_UNSUPPORTED) return rc;
        }
        return wide ? launch_spmv_direct_nt<XF16, 1024, kProAddNorm>(a, h, st) : launch_spmv_direct_nt<XF16, kBlockThreads, kProAddNorm>(a, h, st);
    } else {
        if constexpr (PRO == kProAttnCombine) {
            // the tile-per-wave kernel folds the pieces of a wave's own tiles; the other one folds all of them first
            if (knob(TL_SPMV_TILES, 1) != 0 || a.chain_w) {
                const int rc = launch_spmv_tiles<XF16, kNormCombine>(wide, a, h, st);
                if (rc != TL_ERR_UNSUPPORTED) return rc;
            }
            if (a.chain_w) return fail(TL_ERR_UNSUPPORTED, "the weight's blocks do not fit the kernel that leaves the row for the next norm");
        }
        if constexpr (PRO == kProNone) {
            // the tile-per-wave kernel where the block fits it; with the other producers it is the slower of the two
            if (knob(TL_SPMV_TILES, 1) != 0 || a.chain_w) {
                const int rc = launch_spmv_tiles<XF16, kNormNone>(wide, a, h, st);
                if (rc != TL_ERR_UNSUPPORTED) return rc;
            }
            if (a.chain_w) return fail(TL_ERR_UNSUPPORTED, "the weight's blocks do not fit the kernel that leaves the row for the next norm");
        }
        return wide ? launch_spmv_direct_nt<XF16, 1024, PRO>(a, h, st) : launch_spmv_direct_nt<XF16, kBlockThreads, PRO>(a, h, st);
    }
}

template <int MT>
int launch_small_mt(const KernelArgs& a, const tl_layout_header* h, hipStream_t st)
{
    return a.x_f16 ? launch_block_kernel<MT, true>(a, h, st) : launch_block_kernel<MT, false>(a, h, st);
}

int small_launch(KernelArgs a, const tl_layout_header* h, int x_dtype, void* workspace, int64_t workspace_bytes, hipStream_t st)
{
    int mt = 1;
    while (mt < a.M && mt < 16) mt *= 2;
    // 16-row slots with no more workgroups than compute units: 8-row slots give twice the workgroups,
    // each with half the LDS image, so that two share a compute unit and hide each other's waits.
    const bool alone = (int64_t)a.NB * ceil_div(a.M, 16) <= compute_units();  // a workgroup of 16-row slots would have its compute unit to itself
    // ... then it takes 1024 threads (16 lane groups: the index of a non-zero is decoded once for all 16 rows, and
    // the runs are shared out among fewer lanes each); TL_QUAD_WIDE=0 runs two 8-row halves of 512 threads instead
    const bool wide = mt == 16 && alone && knob(TL_QUAD_WIDE, 1) != 0;
    if (mt == 16 && alone && !wide) mt = 8;
    mt = knob(TL_SMALL_MT, mt);
    if (mt != 1 && mt != 2 && mt != 4 && mt != 8 && mt != 16) return fail(TL_ERR_ARG, "TL_SMALL_MT=%d (1, 2, 4, 8 or 16 expected)", mt);
    const int es = x_dtype == TL_F16 ? 2 : 4;
    a.x_sm = a.x_kmajor ? 1 : a.ldx;
    a.x_sk = a.x_kmajor ? a.ldx : 1;
    bool aligned = (a.ldx * es) % 16 == 0 && reinterpret_cast<uintptr_t>(a.X) % 16 == 0;
    const bool chain_out = a.chain_res || a.chain_image;
    // which kernel, and whether it has the epilogue that was asked for: decided before anything is launched
    bool octet = false, resident = false;
    if (mt >= 8) {
        // fp16, 16 rows: eight rows per lane and two blocks per workgroup where the workgroups still fill the chip
        octet = mt == 16 && a.x_f16 && knob(TL_OCTET, ceil_div(a.NB, 2) * ceil_div(a.M, 16) >= 2 * (int64_t)compute_units() ? 1 : 0) != 0;
        // ... or, up to 16 rows and where it fits, the whole image resident in LDS and one workgroup per compute unit
        // (it pays where a compute unit has more than one block to work through; TL_RES16=1 takes it wherever it fits, 0 never)
        if (mt == 16 && a.M <= 16 && (a.x_f16 ? (a.y_f16 || !(a.gated || chain_out || a.chain_sq_in)) : !(a.gated || chain_out || a.chain_sq_in))) {
            const ResShape shape = res_shape(a, h);
            resident = shape.pieces != 0 && knob(TL_RES16, (int64_t)a.NB * shape.parts > compute_units() ? 1 : 0) != 0;
        }
        if ((chain_out || a.chain_sq_in) && (mt != 16 || !a.x_f16 || !a.y_f16 || a.M > 16))
            return fail(TL_ERR_UNSUPPORTED, "chained products are for 9 to 16 fp16 rows");
        if (a.gated && !octet && !resident)
            return fail(TL_ERR_UNSUPPORTED, "no gated epilogue in the kernel for M=%d, N=%d (tl_spmm, then tl_silu_mul_pairs)", a.M, a.N);
        if (chain_out && octet && !resident) return fail(TL_ERR_UNSUPPORTED, "no residual / image epilogue in the kernel for N=%d", a.N);
    }
    // Slots of 8 and 16 rows are copied into LDS as 16-byte pieces of an aligned K-major image; activations
    // that are not one already are brought into that form in the workspace first.
    if (mt >= 8 && !(a.x_kmajor && aligned && a.ldx >= round_up(a.M, mt)) && !(resident && res_takes_rows(a))) {
        const int64_t need = small_kmajor_bytes(h, a.M, x_dtype);
        if (!workspace || workspace_bytes < need)
            return fail(TL_ERR_SIZE, "workspace has %lld bytes, %lld needed", (long long)workspace_bytes, (long long)need);
        if (reinterpret_cast<uintptr_t>(workspace) % 16) return fail(TL_ERR_ALIGN, "workspace must be 16-byte aligned");
        const int ldo = (int)round_up(a.M, 16);
        const unsigned blocks = (unsigned)ceil_div(a.K, 64);
        if (x_dtype == TL_F16)
            hipLaunchKernelGGL(tl_to_kmajor<__half>, dim3(blocks), dim3(256), 0, st, static_cast<const __half*>(a.X), a.x_sm, a.x_sk,
                               static_cast<__half*>(workspace), ldo, a.M, a.K);
        else
            hipLaunchKernelGGL(tl_to_kmajor<float>, dim3(blocks), dim3(256), 0, st, static_cast<const float*>(a.X), a.x_sm, a.x_sk,
                               static_cast<float*>(workspace), ldo, a.M, a.K);
        a.X = workspace;
        a.ldx = ldo;
        a.x_kmajor = 1;
        a.x_sm = 1;
        a.x_sk = ldo;
        aligned = true;
    }
    if (mt >= 8) {
        if (mt == 8) return a.x_f16 ? launch_quad_kernel<8, true>(a, h, st) : launch_quad_kernel<8, false>(a, h, st);
        if (resident) return launch_res_kernel(a, h, st);
        if (octet) return launch_octet_kernel(a, h, st);
        if (wide) return a.x_f16 ? launch_quad_kernel<16, true, 1024>(a, h, st) : launch_quad_kernel<16, false, 1024>(a, h, st);
        return a.x_f16 ? launch_quad_kernel<16, true>(a, h, st) : launch_quad_kernel<16, false>(a, h, st);
    }
    if (chain_out || a.chain_sq_in) return fail(TL_ERR_UNSUPPORTED, "chained products are for 9 to 16 fp16 rows");
    // one contiguous aligned row whose tiles are whole 16-byte pieces: straight copies into LDS
    if (mt == 1 && a.x_sk == 1 && reinterpret_cast<uintptr_t>(a.X) % 16 == 0 && h->tile_rows % (16 / es) == 0 && a.K % (16 / es) == 0 &&
        knob(TL_SPMV_DIRECT, 1))
        return a.x_f16 ? launch_spmv_direct<true>(a, h, st) : launch_spmv_direct<false>(a, h, st);
    if (a.gated) return fail(TL_ERR_UNSUPPORTED, "no gated epilogue in the kernel for M=%d and this activation layout (tl_spmm, then tl_silu_mul_pairs)", a.M);
    // Column blocks per workgroup.  A compute unit works through ceil(workgroups / 256) workgroups of
    // `set` blocks each: the narrowest set that keeps that product smallest.
    int set = 1;
    {
        int64_t best = -1;
        const int cus = compute_units();
        for (int cand = 1; cand <= kMaxBlockSet; cand *= 2) {
            if ((int64_t)h->max_chunk_dwords * 4 * cand > BlockShape<1, 2, kBlockThreads>::kStreamCap) break;
            const int64_t cost = ceil_div(ceil_div(a.NB, cand), cus) * cand;
            if (best < 0 || cost < best) { best = cost; set = cand; }
        }
    }
    set = knob(TL_BLOCK_SET, set);
    if (set != 1 && set != 2 && set != 4) return fail(TL_ERR_ARG, "TL_BLOCK_SET=%d (1, 2 or 4 expected)", set);
    a.block_set = set;
    const int lpc = kBlockThreads / (TL_BLOCK_COLUMNS * set);
    // lanes per run: one dword per lane should cover a typical run in a whole number of passes with
    // few idle lanes; runs hold mean_run dwords (+1 and -1 parts together)
    const double mean_run = h->mean_run_dwords_x16 / 16.0;
    int lw = 4;
    while (lw < lpc && lw * 3 < mean_run) lw *= 2;
    lw = std::min(knob(TL_LW, lw), lpc);
    if (lw != 1 && lw != 2 && lw != 4 && lw != 8 && lw != 16 && lw != 32) return fail(TL_ERR_ARG, "TL_LW=%d (a power of two up to 32 expected)", lw);
    a.lpc_shift = log2_exact(lpc);
    a.lw_shift = log2_exact(lw);
    a.x_mode = kStageElements;
    if (a.x_kmajor && mt * es >= 16 && aligned && a.ldx >= round_up(a.M, mt)) a.x_mode = kStageSlotVectors;
    // whole vectors of a row are read: K must be whole vectors too, so that none runs past a row's end
    if (!a.x_kmajor && mt <= 4 && aligned && ((int64_t)a.K * es) % 16 == 0) a.x_mode = kStageRowVectors;
    a.tile_magic = (unsigned)(((1ull << 32) + h->tile_rows - 1) / h->tile_rows);
    // one row whose tiles are whole aligned vectors: straight vector copies
    const int ve = 16 / es;
    if (mt == 1 && a.x_sk == 1 && reinterpret_cast<uintptr_t>(a.X) % 16 == 0 && h->tile_rows % ve == 0 && a.K % ve == 0) {
        a.x_mode = kStageRowCopy;
        a.vpt_magic = (unsigned)(((1ull << 32) + h->tile_rows / ve - 1) / (h->tile_rows / ve));
    }
    switch (mt) {
        case 1: return launch_small_mt<1>(a, h, st);
        case 2: return launch_small_mt<2>(a, h, st);
        default: return launch_small_mt<4>(a, h, st);
    }
}


}  // namespace

namespace {
int spmv_fused_call(const tl_layout_header* header, const void* blob_dev, int producer,
                    const void* in, const void* in2, const void* norm_weight, float eps, void* sum_out, int x_dtype,
                    void* Y, int y_dtype, const void* scale, int scale_dtype, void* stream, bool gated, const void* residual = nullptr,
                    const void* next_norm_weight = nullptr, void* image_out = nullptr, float* squares_out = nullptr)
{
    if (int rc = check_header(header)) return rc;
    if (gated && header->columns % 2) return fail(TL_ERR_SHAPE, "N=%u: gate and up columns come in pairs", header->columns);
    if (int rc = check_dtype(x_dtype, "x")) return rc;
    if (int rc = check_dtype(y_dtype, "y")) return rc;
    if (scale)
        if (int rc = check_dtype(scale_dtype, "scale")) return rc;
    if (producer != TL_PRODUCER_NONE && producer != TL_PRODUCER_SILU_GATE && producer != TL_PRODUCER_ADD_RMSNORM && producer != TL_PRODUCER_RMSNORM &&
        producer != TL_PRODUCER_RMSNORM_SUMS)
        return fail(TL_ERR_ARG, "producer code %d unknown", producer);
    if (residual && gated) return fail(TL_ERR_ARG, "a gated product has no residual row of its width");
    if (reinterpret_cast<uintptr_t>(residual) % (y_dtype == TL_F16 ? 2 : 4)) return fail(TL_ERR_ALIGN, "residual is not aligned to its type");
    if (!blob_dev || !in || !Y) return fail(TL_ERR_ARG, "device pointer is null");
    if (reinterpret_cast<uintptr_t>(blob_dev) % 256) return fail(TL_ERR_ALIGN, "weight blob must be 256-byte aligned");
    if ((producer == TL_PRODUCER_ADD_RMSNORM || producer == TL_PRODUCER_RMSNORM) && !norm_weight) return fail(TL_ERR_ARG, "norm_weight is null");
    if (producer == TL_PRODUCER_RMSNORM_SUMS) {
        if (!in2 || norm_weight || sum_out) return fail(TL_ERR_ARG, "TL_PRODUCER_RMSNORM_SUMS takes the sums of squares in in2, and neither norm_weight nor sum_out");
    } else if (producer != TL_PRODUCER_ADD_RMSNORM && (in2 || sum_out)) {
        return fail(TL_ERR_ARG, "in2 and sum_out belong to TL_PRODUCER_ADD_RMSNORM");
    }
    if (next_norm_weight) {
        if (!image_out || !squares_out) return fail(TL_ERR_ARG, "image_out or squares_out is null");
        if (image_out == Y || image_out == in || image_out == residual) return fail(TL_ERR_ARG, "image_out must be a row of its own");
        for (const void* p : {next_norm_weight, static_cast<const void*>(image_out), static_cast<const void*>(squares_out)})
            if (reinterpret_cast<uintptr_t>(p) % 16) return fail(TL_ERR_ALIGN, "next_norm_weight, image_out and squares_out must be 16-byte aligned");
    }
    if (sum_out && (sum_out == in || sum_out == in2)) return fail(TL_ERR_ARG, "sum_out must not be one of the inputs: other workgroups still read them");
    const int es = x_dtype == TL_F16 ? 2 : 4, ve = 16 / es;
    // what the direct-load kernel needs of a row: whole aligned 16-byte pieces per tile
    if (header->tile_rows % ve || header->inners % ve)
        return fail(TL_ERR_UNSUPPORTED, "K=%u, tile height %u: the fused single-row kernel needs whole 16-byte pieces per tile", header->inners, header->tile_rows);
    for (const void* p : {in, in2, norm_weight, static_cast<const void*>(sum_out)})
        if (reinterpret_cast<uintptr_t>(p) % 16) return fail(TL_ERR_ALIGN, "in, in2, norm_weight and sum_out must be 16-byte aligned");
    KernelArgs a;
    std::memset(&a, 0, sizeof(a));
    a.w0 = weight_ptrs(header, blob_dev, scale);
    a.X = in; a.X2 = in2; a.norm_w = norm_weight; a.sum_out = sum_out; a.eps = eps;
    a.Y = Y;
    a.ldx = header->inners; a.ldy = header->columns;
    a.M = 1; a.N = (int)header->columns; a.K = (int)header->inners; a.T = (int)header->n_tiles; a.tile_rows = (int)header->tile_rows;
    a.NB = (int)header->n_blocks;
    a.x_f16 = x_dtype == TL_F16; a.y_f16 = y_dtype == TL_F16; a.scale_f16 = scale_dtype == TL_F16;
    a.one = 1.0f;
    a.gated = gated;
    a.residual = residual;
    a.chain_w = next_norm_weight; a.chain_image = image_out; a.chain_sq_out = squares_out;
    hipStream_t st = static_cast<hipStream_t>(stream);
    int rc;
    if (producer == TL_PRODUCER_NONE)
        rc = a.x_f16 ? launch_spmv_direct<true>(a, header, st) : launch_spmv_direct<false>(a, header, st);
    else if (producer == TL_PRODUCER_RMSNORM_SUMS) {
        a.X2 = nullptr;
        a.chain_sq_in = static_cast<const float*>(in2);
        a.chain_sq_blocks = (int)ceil_div(header->inners, TL_BLOCK_COLUMNS);
        rc = a.x_f16 ? launch_spmv_direct<true, kProNormSums>(a, header, st) : launch_spmv_direct<false, kProNormSums>(a, header, st);
    } else if (producer == TL_PRODUCER_RMSNORM)
        rc = a.x_f16 ? launch_spmv_direct<true, kProNormDeferred>(a, header, st) : launch_spmv_direct<false, kProNormDeferred>(a, header, st);
    else if (producer == TL_PRODUCER_SILU_GATE)
        rc = a.x_f16 ? launch_spmv_direct<true, kProSiluGate>(a, header, st) : launch_spmv_direct<false, kProSiluGate>(a, header, st);
    else
        rc = a.x_f16 ? launch_spmv_direct<true, kProAddNorm>(a, header, st) : launch_spmv_direct<false, kProAddNorm>(a, header, st);
    if (rc) return rc;
    return finish_launch();
}
}  // namespace

extern "C" int tl_spmv_fused(const tl_layout_header* header, const void* blob_dev, int producer,
                             const void* in, const void* in2, const void* norm_weight, float eps, void* sum_out, int x_dtype,
                             void* Y, int y_dtype, const void* scale, int scale_dtype, void* stream)
{
    return spmv_fused_call(header, blob_dev, producer, in, in2, norm_weight, eps, sum_out, x_dtype, Y, y_dtype, scale, scale_dtype, stream, false);
}

extern "C" int tl_spmv_add(const tl_layout_header* header, const void* blob_dev, const void* x, int x_dtype, const void* residual,
                           void* Y, int y_dtype, const void* scale, int scale_dtype, void* stream)
{
    if (!residual) return fail(TL_ERR_ARG, "residual is null");
    return spmv_fused_call(header, blob_dev, TL_PRODUCER_NONE, x, nullptr, nullptr, 0.f, nullptr, x_dtype, Y, y_dtype, scale, scale_dtype, stream, false,
                           residual);
}

extern "C" int tl_spmv_add_norm(const tl_layout_header* header, const void* blob_dev, const void* x, int x_dtype, const void* residual,
                                void* Y, int y_dtype, const void* scale, int scale_dtype, const void* next_norm_weight,
                                void* image_out, float* squares_out, void* stream)
{
    if (!residual) return fail(TL_ERR_ARG, "residual is null");
    if (!next_norm_weight) return fail(TL_ERR_ARG, "next_norm_weight is null");
    return spmv_fused_call(header, blob_dev, TL_PRODUCER_NONE, x, nullptr, nullptr, 0.f, nullptr, x_dtype, Y, y_dtype, scale, scale_dtype, stream, false,
                           residual, next_norm_weight, image_out, squares_out);
}

extern "C" int tl_spmv_fused_gated(const tl_layout_header* header, const void* blob_dev, int producer,
                                   const void* in, const void* in2, const void* norm_weight, float eps, void* sum_out, int x_dtype,
                                   void* Y, int y_dtype, const void* scale, int scale_dtype, void* stream)
{
    return spmv_fused_call(header, blob_dev, producer, in, in2, norm_weight, eps, sum_out, x_dtype, Y, y_dtype, scale, scale_dtype, stream, true);
}

namespace {
int attn_combine_call(const tl_layout_header* header, const void* blob_dev, const void* pieces, int splits, int head_dim,
                      int x_dtype, void* Y, int y_dtype, const void* scale, int scale_dtype, void* stream, const void* residual,
                      const void* next_norm_weight = nullptr, void* image_out = nullptr, float* squares_out = nullptr)
{
    if (int rc = check_header(header)) return rc;
    if (next_norm_weight) {
        if (!image_out || !squares_out) return fail(TL_ERR_ARG, "image_out or squares_out is null");
        if (image_out == Y || image_out == residual) return fail(TL_ERR_ARG, "image_out must be a row of its own");
        for (const void* p : {next_norm_weight, static_cast<const void*>(image_out), static_cast<const void*>(squares_out)})
            if (reinterpret_cast<uintptr_t>(p) % 16) return fail(TL_ERR_ALIGN, "next_norm_weight, image_out and squares_out must be 16-byte aligned");
    }
    if (reinterpret_cast<uintptr_t>(residual) % (y_dtype == TL_F16 ? 2 : 4)) return fail(TL_ERR_ALIGN, "residual is not aligned to its type");
    if (int rc = check_dtype(x_dtype, "x")) return rc;
    if (int rc = check_dtype(y_dtype, "y")) return rc;
    if (scale)
        if (int rc = check_dtype(scale_dtype, "scale")) return rc;
    if (!blob_dev || !pieces || !Y) return fail(TL_ERR_ARG, "device pointer is null");
    if (reinterpret_cast<uintptr_t>(blob_dev) % 256) return fail(TL_ERR_ALIGN, "weight blob must be 256-byte aligned");
    if (reinterpret_cast<uintptr_t>(pieces) % 16) return fail(TL_ERR_ALIGN, "pieces must be 16-byte aligned");
    if (splits < 1 || splits > 8) return fail(TL_ERR_ARG, "splits=%d (1 to 8 expected)", splits);
    const int es = x_dtype == TL_F16 ? 2 : 4, ve = 16 / es;
    if (head_dim <= 0 || head_dim % ve || header->inners % (uint32_t)head_dim)
        return fail(TL_ERR_SHAPE, "head_dim=%d must be a multiple of %d and divide K=%u", head_dim, ve, header->inners);
    if (header->tile_rows % ve || header->inners % ve)
        return fail(TL_ERR_UNSUPPORTED, "K=%u, tile height %u: the fused single-row kernel needs whole 16-byte pieces per tile", header->inners, header->tile_rows);
    if ((int64_t)(header->inners / head_dim) * splits * 4 > 16 * 1024) return fail(TL_ERR_UNSUPPORTED, "too many heads x splits for the kernel's LDS table");
    KernelArgs a;
    std::memset(&a, 0, sizeof(a));
    a.w0 = weight_ptrs(header, blob_dev, scale);
    a.X = pieces; a.pro_splits = splits; a.pro_hd = head_dim;
    a.Y = Y;
    a.ldx = header->inners; a.ldy = header->columns;
    a.M = 1; a.N = (int)header->columns; a.K = (int)header->inners; a.T = (int)header->n_tiles; a.tile_rows = (int)header->tile_rows;
    a.NB = (int)header->n_blocks;
    a.x_f16 = x_dtype == TL_F16; a.y_f16 = y_dtype == TL_F16; a.scale_f16 = scale_dtype == TL_F16;
    a.one = 1.0f;
    a.residual = residual;
    a.chain_w = next_norm_weight; a.chain_image = image_out; a.chain_sq_out = squares_out;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int rc = a.x_f16 ? launch_spmv_direct<true, kProAttnCombine>(a, header, st) : launch_spmv_direct<false, kProAttnCombine>(a, header, st);
    if (rc) return rc;
    return finish_launch();
}
}  // namespace

extern "C" int tl_spmv_attn_combine(const tl_layout_header* header, const void* blob_dev, const void* pieces, int splits, int head_dim,
                                    int x_dtype, void* Y, int y_dtype, const void* scale, int scale_dtype, void* stream)
{
    return attn_combine_call(header, blob_dev, pieces, splits, head_dim, x_dtype, Y, y_dtype, scale, scale_dtype, stream, nullptr);
}

extern "C" int tl_spmv_attn_combine_add(const tl_layout_header* header, const void* blob_dev, const void* pieces, int splits, int head_dim,
                                        int x_dtype, const void* residual, void* Y, int y_dtype, const void* scale, int scale_dtype, void* stream)
{
    if (!residual) return fail(TL_ERR_ARG, "residual is null");
    return attn_combine_call(header, blob_dev, pieces, splits, head_dim, x_dtype, Y, y_dtype, scale, scale_dtype, stream, residual);
}

extern "C" int tl_spmv_attn_combine_add_norm(const tl_layout_header* header, const void* blob_dev, const void* pieces, int splits, int head_dim,
                                             int x_dtype, const void* residual, void* Y, int y_dtype, const void* scale, int scale_dtype,
                                             const void* next_norm_weight, void* image_out, float* squares_out, void* stream)
{
    if (!residual) return fail(TL_ERR_ARG, "residual is null");
    if (!next_norm_weight) return fail(TL_ERR_ARG, "next_norm_weight is null");
    return attn_combine_call(header, blob_dev, pieces, splits, head_dim, x_dtype, Y, y_dtype, scale, scale_dtype, stream, residual, next_norm_weight,
                             image_out, squares_out);
}

int tl::launch_small(KernelArgs a, const tl_layout_header* h, int x_dtype, void* workspace, int64_t workspace_bytes, hipStream_t st)
{
    return small_launch(a, h, x_dtype, workspace, workspace_bytes, st);
}
