// Entry points of libternary_spmm's device code (include/ternary_spmm.h): the checks in front of every launch, the
// choice between the kernels for few rows (tl_small_m.hip) and the row-parallel kernel (tl_rows.hip), the tuning
// knobs, the scratch of the entry point that allocates nothing, and the measurement helpers.
#include "tl_device.h"

using namespace tl;

namespace tl {
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

const char* const kKnobNames[kKnobCount] = {"TL_SMALL_LDS", "TL_TILE_GROUP", "TL_QUAD_SHARE", "TL_LW", "TL_SPMV_SHARE", "TL_SPMV_WIDE",
                                            "TL_SMALL_MT", "TL_SPMV_DIRECT", "TL_BLOCK_SET", "TL_ROWS_SPLIT", "TL_OCTET", "TL_QUAD_WIDE", "TL_SPMV_TILES", "TL_RES16"};
struct Knobs {
    bool set[kKnobCount];
    int value[kKnobCount];
};
std::atomic<const Knobs*> g_knobs{nullptr};

const Knobs* read_knobs()
{
    Knobs* k = new Knobs;
    for (int i = 0; i < kKnobCount; ++i) {
        const char* v = std::getenv(kKnobNames[i]);
        k->set[i] = v && *v;
        k->value[i] = k->set[i] ? std::atoi(v) : 0;
    }
    return k;
}

int knob(Knob which, int fallback)
{
    const Knobs* k = g_knobs.load(std::memory_order_acquire);
    if (!k) {
        const Knobs* fresh = read_knobs();
        if (g_knobs.compare_exchange_strong(k, fresh, std::memory_order_acq_rel)) k = fresh;
        else delete fresh;  // another thread was first; k now holds its table
    }
    return k->set[which] ? k->value[which] : fallback;
}

// Compute units of the current device, asked once per device.  Launch shapes are sized by it; the row
// kernel's one-workgroup-per-unit launch is capped at kMaxComputeUnits, which sizes its partial-sum area.
int compute_units()
{
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return kMaxComputeUnits;
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = kMaxComputeUnits;
        cached[dev].store(n, std::memory_order_relaxed);
    }
    return n;
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

}  // namespace tl

extern "C" int tl_reload_options(void)
{
    const Knobs* old = g_knobs.exchange(read_knobs(), std::memory_order_acq_rel);
    (void)old;  // a launch on another thread may still be reading it: the few bytes are left alone
    return TL_OK;
}

extern "C" int tl_spmm_workspace(const tl_layout_header* header, int64_t M, int x_dtype, int x_layout, int64_t* workspace_bytes)
{
    if (int rc = check_header(header)) return rc;
    if (int rc = check_dtype(x_dtype, "x")) return rc;
    if (!workspace_bytes) return fail(TL_ERR_ARG, "workspace_bytes is null");
    if (M <= 0) return fail(TL_ERR_SHAPE, "M=%lld must be positive", (long long)M);
    if (M <= kSmallMaxM) {  // room for the aligned K-major image of the activations (more than 4 rows)
        (void)x_layout;  // K-major activations need it too when they are not aligned vectors
        *workspace_bytes = small_kmajor_bytes(header, M, x_dtype);
        return TL_OK;
    }
    // the K-major image of the activations, then room for the partial sums of shared-out output tiles
    *workspace_bytes = rows_relayout_bytes(header->inners, M, x_dtype) + kRowsPartialBytes;
    return TL_OK;
}

namespace {
// tl_spmm, or (y_layout >= 0) tl_spmm_gated with that output layout
int spmm_call(const tl_layout_header* header, const void* blob_dev, const void* X, int x_dtype, int x_layout, int64_t ldx, int64_t M,
              void* Y, int y_dtype, int64_t ldy, int y_layout, const void* scale, int scale_dtype, void* workspace, int64_t workspace_bytes,
              void* stream, const tl_chain* chain = nullptr)
{
    if (int rc = check_header(header)) return rc;
    const bool gated = y_layout >= 0;
    // the checks of tl_spmm, with the width of the gated output where ldy is compared
    if (int rc = check_io(blob_dev, X, Y, x_dtype, x_layout, ldx, M, y_dtype, gated ? (int64_t)header->columns : ldy, scale, scale_dtype, header)) return rc;
    if (gated) {
        if (y_layout != TL_X_ROW_MAJOR && y_layout != TL_X_K_MAJOR) return fail(TL_ERR_ARG, "y_layout=%d unknown", y_layout);
        if (header->columns % 2) return fail(TL_ERR_SHAPE, "N=%u: gate and up columns come in pairs", header->columns);
        const int64_t min_ldy = y_layout == TL_X_K_MAJOR ? M : (int64_t)header->columns / 2;
        if (ldy < min_ldy) return fail(TL_ERR_SHAPE, "ldy=%lld smaller than %lld", (long long)ldy, (long long)min_ldy);
        if (y_layout == TL_X_K_MAJOR && (M <= 8 || M > 16)) return fail(TL_ERR_UNSUPPORTED, "a K-major gated output is written for 9 to 16 rows");
    }
    KernelArgs a;
    std::memset(&a, 0, sizeof(a));
    a.gated = gated;
    if (gated && y_layout == TL_X_K_MAJOR) a.y_kld = ldy;
    if (chain) {
        const bool out = chain->next_norm_weight || chain->image_out || chain->squares_out;
        if (out && !(chain->next_norm_weight && chain->image_out && chain->squares_out))
            return fail(TL_ERR_ARG, "next_norm_weight, image_out and squares_out come together");
        if ((out || chain->residual) && gated) return fail(TL_ERR_ARG, "a gated product has no residual or image epilogue");
        if (M < 9 || M > 16) return fail(TL_ERR_UNSUPPORTED, "chained products are for 9 to 16 fp16 rows");
        if (chain->residual && chain->residual_ld < (int64_t)header->columns) return fail(TL_ERR_SHAPE, "residual_ld=%lld smaller than N", (long long)chain->residual_ld);
        if (out && (chain->image_ld < M || chain->image_ld > 16))  // the epilogue writes (and zeroes) 16 rows of the image at most
            return fail(TL_ERR_SHAPE, "image_ld=%lld outside M=%lld .. 16", (long long)chain->image_ld, (long long)M);
        if (chain->squares_in && chain->squares_blocks <= 0) return fail(TL_ERR_ARG, "squares_blocks must be positive");
        const uintptr_t es = y_dtype == TL_F16 ? 2 : 4;
        for (const void* p : {chain->residual, chain->next_norm_weight, static_cast<const void*>(chain->image_out)})
            if (reinterpret_cast<uintptr_t>(p) % es) return fail(TL_ERR_ALIGN, "residual, next_norm_weight and image_out must be aligned to y_dtype");
        for (const void* p : {static_cast<const void*>(chain->squares_out), static_cast<const void*>(chain->squares_in)})
            if (reinterpret_cast<uintptr_t>(p) % 16) return fail(TL_ERR_ALIGN, "squares_out and squares_in must be 16-byte aligned");
        a.chain_res = chain->residual; a.chain_ldres = chain->residual_ld;
        a.chain_w = chain->next_norm_weight; a.chain_image = chain->image_out; a.chain_ild = chain->image_ld; a.chain_sq_out = chain->squares_out;
        a.chain_sq_in = chain->squares_in; a.chain_sq_blocks = chain->squares_blocks; a.eps = chain->eps;
    }
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
}  // namespace

extern "C" int tl_spmm(const tl_layout_header* header, const void* blob_dev,
                       const void* X, int x_dtype, int x_layout, int64_t ldx, int64_t M,
                       void* Y, int y_dtype, int64_t ldy,
                       const void* scale, int scale_dtype,
                       void* workspace, int64_t workspace_bytes, void* stream)
{
    return spmm_call(header, blob_dev, X, x_dtype, x_layout, ldx, M, Y, y_dtype, ldy, -1, scale, scale_dtype, workspace, workspace_bytes, stream);
}

extern "C" int tl_spmm_chain(const tl_layout_header* header, const void* blob_dev,
                             const void* X, int x_dtype, int x_layout, int64_t ldx, int64_t M,
                             void* Y, int y_dtype, int64_t ldy, int y_layout,
                             const void* scale, int scale_dtype, const tl_chain* chain,
                             void* workspace, int64_t workspace_bytes, void* stream)
{
    if (!chain) return fail(TL_ERR_ARG, "chain is null");
    return spmm_call(header, blob_dev, X, x_dtype, x_layout, ldx, M, Y, y_dtype, ldy, y_layout, scale, scale_dtype, workspace, workspace_bytes, stream, chain);
}

extern "C" int tl_spmm_gated(const tl_layout_header* header, const void* blob_dev,
                             const void* X, int x_dtype, int x_layout, int64_t ldx, int64_t M,
                             void* Y, int y_dtype, int64_t ldy, int y_layout,
                             const void* scale, int scale_dtype,
                             void* workspace, int64_t workspace_bytes, void* stream)
{
    return spmm_call(header, blob_dev, X, x_dtype, x_layout, ldx, M, Y, y_dtype, ldy, y_layout, scale, scale_dtype, workspace, workspace_bytes, stream);
}

// Scratch of tl_spmm_noalloc: device memory that belongs to the library's code object, one copy per GPU,
// there from the moment the library is loaded on a device until the process ends.
constexpr int64_t kStaticScratchBytes = 32ll << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {
// Device address of `scratch` on the current device.  In host code the array's name is only a handle
// for the runtime; the address comes from hipGetSymbolAddress, asked once per device with that device
// current, and differs from GPU to GPU.
int static_scratch(void** out)
{
    static std::atomic<void*> address[64];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(TL_ERR_LAUNCH, "hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= 64) return fail(TL_ERR_UNSUPPORTED, "device ordinal %d: the static scratch serves ordinals 0 to 63", dev);
    void* p = address[dev].load(std::memory_order_acquire);
    if (!p) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) return fail(TL_ERR_LAUNCH, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
        address[dev].store(p, std::memory_order_release);
    }
    *out = p;
    return TL_OK;
}
}  // namespace

extern "C" int tl_spmm_noalloc(const tl_layout_header* header, const void* blob_dev,
                               const void* X, int x_dtype, int x_layout, int64_t ldx, int64_t M,
                               void* Y, int y_dtype, int64_t ldy,
                               const void* scale, int scale_dtype, void* stream)
{
    if (int rc = check_header(header)) return rc;
    if (int rc = check_dtype(x_dtype, "x")) return rc;
    if (M <= 0) return fail(TL_ERR_SHAPE, "M=%lld must be positive", (long long)M);
    // what the kernels stage in the scratch: the K-major image of the activations (none for 4 rows and fewer).
    // Room for partial sums is not offered, so the row kernel gives every output tile a workgroup of its own.
    const int64_t need = M <= kSmallMaxM ? small_kmajor_bytes(header, M, x_dtype) : rows_relayout_bytes(header->inners, M, x_dtype);
    if (need > kStaticScratchBytes)
        return fail(TL_ERR_SIZE, "M=%lld rows of K=%u need %lld bytes of scratch; tl_spmm_noalloc has %lld (use tl_spmm with a workspace)",
                    (long long)M, header->inners, (long long)need, (long long)kStaticScratchBytes);
    void* ws = nullptr;
    if (int rc = static_scratch(&ws)) return rc;
    return tl_spmm(header, blob_dev, X, x_dtype, x_layout, ldx, M, Y, y_dtype, ldy, scale, scale_dtype, ws, need, stream);
}

// Reads `pieces` 16-byte pieces and folds them: what streaming that much memory costs a launch that writes next to
// nothing.  256 threads a workgroup, eight pieces of a thread in flight per turn.
__global__ __launch_bounds__(256) void tl_read_probe(const u32x4* __restrict__ src, long long pieces, uint32_t* __restrict__ out)
{
    constexpr int U = 8;
    const long long stride = (long long)gridDim.x * 256;
    uint32_t fold = 0;
    for (long long first = (long long)blockIdx.x * 256 + threadIdx.x; first < pieces; first += stride * U) {
        u32x4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = first + u * stride < pieces ? src[first + u * stride] : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
        for (int u = 0; u < U; ++u) fold ^= v[u][0] ^ v[u][1] ^ v[u][2] ^ v[u][3];
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) fold ^= __shfl_xor(fold, off, 64);
    __shared__ uint32_t part[4];
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = fold;
    __syncthreads();
    if (threadIdx.x == 0) out[blockIdx.x] = part[0] ^ part[1] ^ part[2] ^ part[3];
}

extern "C" int tl_read_probe_workgroups(void) { return 8 * compute_units(); }

extern "C" int tl_stream_read_probe(const void* src, int64_t bytes, void* out, void* stream)
{
    if (!src || !out) return fail(TL_ERR_ARG, "device pointer is null");
    if (bytes <= 0 || bytes % 16) return fail(TL_ERR_SIZE, "bytes=%lld must be a positive multiple of 16", (long long)bytes);
    if (reinterpret_cast<uintptr_t>(src) % 16 || reinterpret_cast<uintptr_t>(out) % 4) return fail(TL_ERR_ALIGN, "src must be 16-byte, out 4-byte aligned");
    const long long pieces = bytes / 16;
    const int groups = (int)std::min<long long>(tl_read_probe_workgroups(), ceil_div(pieces, 256));
    hipLaunchKernelGGL(tl_read_probe, dim3((unsigned)groups), dim3(256), 0, static_cast<hipStream_t>(stream), static_cast<const u32x4*>(src), pieces,
                       static_cast<uint32_t*>(out));
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

