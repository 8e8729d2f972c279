// What the translation units of libternary_spmm's device code share: the argument block of the kernels, the
// device helpers every kernel family uses, and the host helpers of the launchers (knobs, device facts, checks).
//   tl_small_m.hip  the kernels for 1 to 48 activation rows and their launchers
//   tl_rows.hip     the row-parallel kernel (more than 48 rows), its re-layout and fix-up kernels and launchers
//   tl_kernels.hip  the entry points, the checks in front of them, the knobs, the measurement helpers
#pragma once
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <type_traits>

#include "tl_common.h"

namespace tl {

// Loads through this pointer type may use the scalar (constant) path when the address is wave-uniform.
typedef const __attribute__((address_space(4))) uint32_t* const_u32_ptr;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));  // one 16-byte chunk in registers
typedef uint32_t u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));  // the same, loaded from a dword-aligned address
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
    int block_set;        // small-M kernel: column blocks per workgroup (1, 2 or 4)
    int lpc_shift, lw_shift;  // small-M kernel: log2 of lanes per column and of lanes per run
    int xs_bytes, buf_bytes;  // small-M kernel: LDS for the staged activations / for the chunk copies
    int x_mode;           // small-M kernel: how activations are staged (kStageElements / kStageSlotVectors / kStageRowVectors)
    unsigned vpt_magic;   // small-M kernel, row-copy staging: ceil(2^32 / (tile_rows / values per vector))
    unsigned tile_magic;  // ceil(2^32 / tile_rows): k / tile_rows == (k * tile_magic) >> 32 for every k < 2^24
    long long x_sm, x_sk; // small-M kernel: element strides of the activations along M and along K
    long long split_steps;  // row kernel: 0, or the number of (output tile, K tile) steps shared out among the workgroups
    int whole_units;        // row kernel: output tiles every workgroup works through on its own first
    int split_first_unit;   // row kernel: first output tile of those whose steps are shared out
    float* partial;         // row kernel: partial sums of output tiles whose K tiles were shared out
    float one;  // 1.0f, passed in so that the fp16 -> fp32 accumulate stays a single mixed-precision fma
    // single-row kernel with a fused producer of its input (tl_spmv_fused)
    const void* X2;       // second summand of the residual add, or null
    const void* norm_w;   // RMSNorm weight [K]
    void* sum_out;        // where the first workgroup writes X + X2, or null
    float eps;
    int pro_splits;       // attention-combine producer: pieces per head, and the head width
    int pro_hd;
    // gated epilogue: columns 2j, 2j + 1 of the weight are gate and up column j; Y[j] = silu(y[2j]) * y[2j + 1] (N / 2 outputs)
    int gated;
    const void* residual;  // single-row kernels: null, or a row of N values of Y's type: Y[n] = residual[n] + the product (rounded to that type first)
    long long y_kld;      // gated epilogue of the 16-row kernel: 0, or the leading dimension of a K-major output [N / 2][y_kld]
    // 16-row kernels, a decoder layer without kernels for the residual add and the RMSNorm (tl_spmm_chain):
    const void* chain_res;    // [M][chain_ldres], Y's type: Y = chain_res + product
    long long chain_ldres;
    const void* chain_w;      // [N] weight of the NEXT norm: chain_image[n][m] = Y[m][n] * chain_w[n], chain_sq_out[block][m] = sum over the block's columns of Y[m][n]^2
    void* chain_image;        // K-major [N][chain_ild], Y's type, rows M .. chain_ild - 1 zeroed
    long long chain_ild;
    float* chain_sq_out;      // [NB][16]
    const float* chain_sq_in; // [chain_sq_blocks][16] sums of squares of the rows X was made from: the product is multiplied by rsqrt(sum / K + eps), row by row
    int chain_sq_blocks;
};

// rsqrt(mean square + eps) of the rows behind a chained product.  Called by the first 64 threads of a workgroup (one
// wave), all of them; lane L gets the factors of rows 4 * (L % 4) .. + 3.  The partial sums [blocks][16] are read as
// 16-byte pieces, several in flight per lane (one after the other they would cost a trip to memory each).
__device__ __forceinline__ float4 chain_row_factors(const KernelArgs& a, int lane)
{
    const float4* pieces = reinterpret_cast<const float4*>(a.chain_sq_in);  // piece i: block i / 4, rows 4 * (i % 4) .. + 3
    const int count = a.chain_sq_blocks * 4;
    constexpr int U = 16;  // pieces of a lane in flight together: 256 blocks (K = 4096) in one trip
    float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int first = lane; first < count; first += 64 * U) {
        float4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = first + 64 * u < count ? pieces[first + 64 * u] : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int u = 0; u < U; ++u) { sum.x += v[u].x; sum.y += v[u].y; sum.z += v[u].z; sum.w += v[u].w; }
    }
#pragma unroll
    for (int off = 4; off < 64; off <<= 1) {  // the lanes with the same rows
        sum.x += __shfl_xor(sum.x, off, 64); sum.y += __shfl_xor(sum.y, off, 64);
        sum.z += __shfl_xor(sum.z, off, 64); sum.w += __shfl_xor(sum.w, off, 64);
    }
    const float k = 1.0f / (float)a.K;
    return make_float4(rsqrtf(sum.x * k + a.eps), rsqrtf(sum.y * k + a.eps), rsqrtf(sum.z * k + a.eps), rsqrtf(sum.w * k + a.eps));
}

__device__ __forceinline__ float load_scale(const void* scale, int is_f16, int n)
{
    if (!scale) return 1.0f;
    return is_f16 ? __half2float(static_cast<const __half*>(scale)[n]) : static_cast<const float*>(scale)[n];
}

// An fp32 value on its way to an fp16 result is kept apart from the conversion: left to the compiler, a product
// that feeds the conversion becomes one instruction that rounds the exact product straight to fp16
// (v_fma_mixlo_f16) in one kernel and a multiply plus a conversion in another, and the two differ on near-ties.
// Every kernel of this file converts the rounded fp32 value.
__device__ __forceinline__ float settled(float v)
{
    asm volatile("" : "+v"(v));
    return v;
}

__device__ __forceinline__ void store_out(void* Y, int is_f16, long long off, float v)
{
    if (is_f16) static_cast<__half*>(Y)[off] = __float2half(settled(v));
    else static_cast<float*>(Y)[off] = v;
}

__device__ __forceinline__ float silu(float g) { return g / (1.0f + __expf(-g)); }

// v as a stored output of the call's type would read back
__device__ __forceinline__ float as_output(float v, int is_f16) { return is_f16 ? __half2float(__float2half(settled(v))) : v; }

// silu(g) * u for a product's outputs g, u (already rounded to the output type), with the roundings of the separate
// operator: the SiLU is rounded to the type before the product.
__device__ __forceinline__ float gate_pair(float g, float u, int is_f16) { return as_output(g / (1.0f + __expf(-g)), is_f16) * u; }

// One output of a single-row product on its way out: plain, or added to the residual row as a separate add of the
// stored product would add it.
__device__ __forceinline__ void store_result(const KernelArgs& a, int n, float v)
{
    if (a.residual) v = as_output(v, a.y_f16) + load_scale(a.residual, a.y_f16, n);
    store_out(a.Y, a.y_f16, n, v);
}

__device__ __forceinline__ int run_pos_dwords(uint32_t d) { return (int)(((d & 0xffu) + 3u) >> 2); }
__device__ __forceinline__ int run_neg_dwords(uint32_t d) { return (int)((((d >> 8) & 0xffu) + 3u) >> 2); }

// ---------------------------------------------------------------------------
// Host side, shared by the launchers.
// ---------------------------------------------------------------------------
constexpr int kSmallMaxM = 48;       // above this the row-parallel kernel takes over
constexpr int kRowsWaves = 16;
constexpr int kRowsCols = 4;       // columns per wave of the fused gate/up kernel (two accumulator sets)
constexpr int kRowsColsPlain = 8;  // columns per wave of the plain kernel: an activation tile then serves 128 columns
constexpr int kMaxComputeUnits = 256;
constexpr int kMaxChunkBytes = (TL_BLOCK_COLUMNS + TL_BLOCK_COLUMNS * 128) * 4;  // a chunk of all-non-zero columns

inline int rows_mtile(int x_dtype) { return x_dtype == TL_F16 ? 256 : 128; }

// Tuning knobs (environment variables of the same names).  They are read once, at the first launch of the
// process; tl_reload_options() reads them again.  A knob that is not set leaves the launcher's own choice.
enum Knob { TL_SMALL_LDS, TL_TILE_GROUP, TL_QUAD_SHARE, TL_LW, TL_SPMV_SHARE, TL_SPMV_WIDE, TL_SMALL_MT, TL_SPMV_DIRECT,
            TL_BLOCK_SET, TL_ROWS_SPLIT, TL_OCTET, TL_QUAD_WIDE, TL_SPMV_TILES, TL_RES16, kKnobCount };
int knob(Knob which, int fallback);   // tl_kernels.hip
int compute_units();                  // of the current device, read once per device
int check_header(const tl_layout_header* h);
int check_dtype(int d, const char* what);
int finish_launch();
int check_io(const void* blob_dev, const void* X, void* Y, int x_dtype, int x_layout, int64_t ldx, int64_t M, int y_dtype,
             int64_t ldy, const void* scale, int scale_dtype, const tl_layout_header* h);
WeightPtrs weight_ptrs(const tl_layout_header* h, const void* blob_dev, const void* scale);

template <typename KernelT>
int raise_lds_limit(KernelT kernel, size_t bytes)
{
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e != hipSuccess) return fail(TL_ERR_LAUNCH, "hipFuncSetAttribute(%zu bytes of LDS): %s", bytes, hipGetErrorString(e));
    return TL_OK;
}

// tl_small_m.hip
inline int64_t small_kmajor_bytes(const tl_layout_header* h, int64_t M, int x_dtype)
{
    return M > 4 ? (int64_t)h->inners * round_up(M, 16) * (x_dtype == TL_F16 ? 2 : 4) : 0;
}
int launch_small(KernelArgs a, const tl_layout_header* h, int x_dtype, void* workspace, int64_t workspace_bytes, hipStream_t st);

// tl_rows.hip
// Bytes of partial sums the row kernel may leave when K tiles are shared out (both weight sets of the
// fused gate/up kernel): two slots per workgroup of a one-workgroup-per-compute-unit launch.
constexpr int64_t kRowsPartialBytes = (int64_t)kMaxComputeUnits * 2 * 2 * kRowsWaves * kRowsCols * 4 * 64 * sizeof(float);
inline int64_t rows_relayout_bytes(int64_t K, int64_t M, int x_dtype)
{
    return round_up(K * round_up(M, rows_mtile(x_dtype)) * (x_dtype == TL_F16 ? 2 : 4), 256);
}
int launch_rows(KernelArgs a, int x_dtype, void* workspace, int64_t workspace_bytes, bool gated, hipStream_t st);

}  // namespace tl
