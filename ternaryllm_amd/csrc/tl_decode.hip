// Two small kernels around the ternary products of a single-token decode step:
// rotary embedding fused with the KV-cache update, and softmax attention of one query per head over
// the cache.  They stand where the reference calls into the transformers package
// (ternaryLLM_GPU/TernaryLLM/TernaryAttn.py:93-113: apply_rotary_pos_emb, Cache.update, the eager
// matmul / softmax / matmul) -- a handful of tiny launches per layer there, two here.  Position and
// valid length are read from device memory, so a captured HIP graph of the step can be replayed for
// every token.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <climits>

#include "tl_common.h"

using namespace tl;

namespace {

template <typename T> __device__ __forceinline__ float to_f(T v);
template <> __device__ __forceinline__ float to_f<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f<__half>(__half v) { return __half2float(v); }
template <typename T> __device__ __forceinline__ T from_f(float v);
template <> __device__ __forceinline__ float from_f<float>(float v) { return v; }
template <> __device__ __forceinline__ __half from_f<__half>(float v) { return __float2half(v); }

// One value of the rotate-half rotary embedding: x at dimension d, xp its partner half a head away, sgn = -1
// below the middle and +1 above.  One explicit fma whose fp32 result is kept apart from the conversion that
// follows it, so that every kernel rounds the same way: left to the compiler, some uses become an fma that
// rounds straight to fp16 (v_fma_mixlo_f16) and others an fp32 fma plus a conversion, which differ on near-ties.
__device__ __forceinline__ float rope_value(float x, float xp, float c, float s, float sgn)
{
    float r = fmaf(sgn * xp, s, x * c);
    asm volatile("" : "+v"(r));
    return r;
}

// qkv: [batch][3][heads][head_dim] (q, k, v of one token per batch row, as the fused projection
// writes them).  Rotate-half form: out[d] = x[d] * cos[d] - x[d + h/2] * sin[d] for d < h/2,
// out[d] = x[d] * cos[d] + x[d - h/2] * sin[d] above.  q goes to q_out [batch][heads][head_dim];
// rotated k and plain v go to row `pos` of the caches [batch][heads][max_seq][head_dim].
template <typename T>
__global__ __launch_bounds__(256) void tl_rope_cache(const T* __restrict__ qkv, const T* __restrict__ cos_t,
                                                     const T* __restrict__ sin_t, const long long* __restrict__ pos_p,
                                                     T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache,
                                                     int batch, int heads, int head_dim, long long max_seq)
{
    const long long pos = *pos_p;
    const int half = head_dim / 2;
    const long long i = blockIdx.x * 256ll + threadIdx.x;  // over batch * heads * head_dim
    if (i >= (long long)batch * heads * head_dim || pos < 0 || pos >= max_seq) return;
    const int d = (int)(i % head_dim);
    const long long bh = i / head_dim;
    const int h = (int)(bh % heads);
    const long long b = bh / heads;
    const T* base = qkv + (size_t)b * 3 * heads * head_dim + (size_t)h * head_dim;
    const size_t plane = (size_t)heads * head_dim;
    const float c = to_f(cos_t[(size_t)pos * head_dim + d]), s = to_f(sin_t[(size_t)pos * head_dim + d]);
    const int partner = d < half ? d + half : d - half;
    const float sgn = d < half ? -1.0f : 1.0f;
    const float q = rope_value(to_f(base[d]), to_f(base[partner]), c, s, sgn);
    const float k = rope_value(to_f(base[plane + d]), to_f(base[plane + partner]), c, s, sgn);
    q_out[i] = from_f<T>(q);
    const size_t row = ((size_t)bh * max_seq + pos) * head_dim + d;
    k_cache[row] = from_f<T>(k);
    v_cache[row] = base[2 * plane + d];
}

// One workgroup per (batch row, head): scores of the query against cache rows [0, pos], softmax in
// fp32, weighted sum of the value rows.  out is [batch][heads * head_dim], the layout the output
// projection multiplies (or its K-major image).  A cache row is read as 16-byte pieces by CPR
// neighbouring lanes, and the workgroup's 1024 threads work on RG = 1024 / CPR rows side by side.
// One pass over the cache: a row group takes NB of its rows at a time, key and value pieces of all of
// them requested together, and keeps a running maximum, sum of exponentials and weighted sum (rescaled
// when the maximum moves), so nothing waits for memory a second time; the RG running results are
// combined through LDS at the end.
constexpr int kAttnThreads = 1024;
constexpr int kAttnBatch = 5;  // rows of a row group whose loads are in flight together
// With more workgroups than compute units (batches of nine rows and more at 32 heads) two workgroups to a compute unit
// run through the cache faster than one after the other: tl_decode_attn_packed is the same kernel held to 64
// registers a lane, which it fits with two rows of a row group in flight (fp16, heads of up to 128 values).  Batch
// 16 over 577 cache rows: 30.1 against 30.7-31.4 us per layer, over 101 rows 11.2 against 14.6; with three rows in
// flight it spills and takes 37.4.
constexpr int kAttnBatchPacked = 2;


// The value another lane of the same row of 16 holds, by a data-parallel-primitive code
template <int CTRL>
__device__ __forceinline__ float lane_permuted(float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}

//
// With `fresh` (q|k|v of the token as the projection wrote them, [batch][3][heads][HD], plus the rotary tables)
// the kernel is also what tl_rope_cache does: q is rotated on the way in; the rotated key and the value of the
// token stand in for cache row `pos`, which does not exist yet, and the workgroup whose rows include `pos` writes
// them there for the steps to come.  Values are rounded to T where the separate kernels would store them, so
// the result is theirs bit for bit.
template <typename T>
struct FreshToken {
    const T* qkv;    // null: q and the cache are complete already
    const T* cos_t;
    const T* sin_t;
    T* k_cache;      // the caches again, to write row `pos` through
    T* v_cache;
};

template <typename T, int HD, int NB>
__device__ __forceinline__ void decode_attn_body(const T* __restrict__ q, const T* __restrict__ k_cache,
                                                 const T* __restrict__ v_cache, const long long* __restrict__ pos_p,
                                                 T* __restrict__ out, long long out_kld, int heads, long long max_seq,
                                                 float scale, int splits, float* __restrict__ pieces,
                                                 unsigned* __restrict__ arrivals, const FreshToken<T>& fresh)
{
    constexpr int VE = 16 / (int)sizeof(T);   // values per 16-byte piece
    constexpr int CPR = HD / VE;              // lanes per cache row
    constexpr int RG = kAttnThreads / CPR;    // row groups
    static_assert(CPR <= 64 && (CPR & (CPR - 1)) == 0, "a row's lanes must sit in one wave");
    __shared__ float partial[RG][HD + 1];
    constexpr int SG = kAttnThreads / HD;     // threads that share the fold of one output value
    static_assert(RG % SG == 0, "the row groups are dealt out evenly to the threads of an output value");
    __shared__ float group_max[RG], group_sum[RG];
    __shared__ float fold_o[SG][HD], fold_norm[SG], fold_top;
    __shared__ int last_to_arrive;
    const int tid = threadIdx.x;
    const long long bh = blockIdx.x;
    const long long pos = *pos_p;
    const bool has_fresh = fresh.qkv != nullptr && pos >= 0 && pos < max_seq;  // row `pos` comes from fresh.qkv
    long long n = pos + 1;  // valid rows
    if (n > max_seq) n = max_seq;
    if (n < 1) n = 1;
    // With splits > 1 the rows of a (batch row, head) are shared out in contiguous pieces among gridDim.y
    // workgroups; each leaves its unnormalised sums, maximum and sum of exponentials for tl_attn_combine.
    long long lo = 0;
    if (splits > 1) {
        const long long piece = (n + splits - 1) / splits;
        lo = (long long)blockIdx.y * piece;
        n = lo + piece < n ? lo + piece : n;  // may leave this workgroup no rows (lo >= n)
    }
    const T* kc = k_cache + (size_t)bh * max_seq * HD;
    const T* vc = v_cache + (size_t)bh * max_seq * HD;
    const int c = tid % CPR, rg = tid / CPR;

    auto unpack = [](const uint4& v, float (&f)[VE]) {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
        if constexpr (sizeof(T) == 2) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                f[2 * e] = __half2float(__ushort_as_half((unsigned short)(w[e] & 0xffffu)));
                f[2 * e + 1] = __half2float(__ushort_as_half((unsigned short)(w[e] >> 16)));
            }
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) f[e] = __uint_as_float(w[e]);
        }
    };

    // A row group's rows come NB at a time; the first batch is asked for before q is ready.  (Asking for the next
    // batch before the current one is worked on, two register sets alternating, was no faster at 3 rows per batch
    // and slower at 4, where it needs more than the 128 registers a thread of 1024 may have.)
    // Every slot of a batch is loaded, without a branch: a slot past the group's last row takes the batch's first row
    // again (its score is masked below, so it adds exactly nothing), and the cache row the token will take is loaded
    // like any other and replaced by the token's own key and value before use.  Row numbers and offsets are 32-bit
    // (the launcher holds a head's cache under 2 GiB).
    const int n_rows = (int)n, fresh_row = has_fresh ? (int)pos : -1;
    auto row_of = [&](int j0, int u) {
        const int j = j0 + u * RG;
        return j < n_rows ? j : j0;
    };
    auto load_batch = [&](int j0, uint4 (&kk)[NB], uint4 (&vv)[NB]) {
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            const uint32_t off = (uint32_t)row_of(j0, u) * HD + c * VE;
            kk[u] = *reinterpret_cast<const uint4*>(kc + off);
            vv[u] = *reinterpret_cast<const uint4*>(vc + off);
        }
    };
    uint4 ka[NB], va[NB];
    constexpr int step = RG * NB;
    int j0 = (int)lo + rg;
    if (j0 < n_rows) load_batch(j0, ka, va);

    float qv[VE];
    uint4 k_new = make_uint4(0u, 0u, 0u, 0u), v_new = make_uint4(0u, 0u, 0u, 0u);  // this lane's piece of the token's key and value
    if (fresh.qkv) {
        static_assert((HD / 2) % VE == 0, "a 16-byte piece lies in one half of the head");
        const T* base = fresh.qkv + ((size_t)(bh / heads) * 3 * heads + (size_t)(bh % heads)) * HD;
        const size_t plane = (size_t)heads * HD;
        const int d0 = c * VE, p0 = d0 < HD / 2 ? d0 + HD / 2 : d0 - HD / 2;
        const float sgn = d0 < HD / 2 ? -1.0f : 1.0f;
        const long long table_row = pos < 0 ? 0 : pos < max_seq ? pos : max_seq - 1;
        // all seven pieces are asked for before the first is used: one trip to memory, not three
        const uint4 cos_piece = *reinterpret_cast<const uint4*>(fresh.cos_t + (size_t)table_row * HD + d0);
        const uint4 sin_piece = *reinterpret_cast<const uint4*>(fresh.sin_t + (size_t)table_row * HD + d0);
        const uint4 q_piece = *reinterpret_cast<const uint4*>(base + d0), q_partner = *reinterpret_cast<const uint4*>(base + p0);
        const uint4 k_piece = *reinterpret_cast<const uint4*>(base + plane + d0), k_partner = *reinterpret_cast<const uint4*>(base + plane + p0);
        v_new = *reinterpret_cast<const uint4*>(base + 2 * plane + d0);
        float cs[VE], sn[VE], x[VE], xp[VE];
        unpack(cos_piece, cs);
        unpack(sin_piece, sn);
        unpack(q_piece, x);
        unpack(q_partner, xp);
#pragma unroll
        for (int e = 0; e < VE; ++e) qv[e] = to_f(from_f<T>(rope_value(x[e], xp[e], cs[e], sn[e], sgn))) * scale;
        unpack(k_piece, x);
        unpack(k_partner, xp);
        T* kt = reinterpret_cast<T*>(&k_new);
#pragma unroll
        for (int e = 0; e < VE; ++e) kt[e] = from_f<T>(rope_value(x[e], xp[e], cs[e], sn[e], sgn));
    } else {
        float f[VE];
        unpack(*reinterpret_cast<const uint4*>(q + (size_t)bh * HD + c * VE), f);
#pragma unroll
        for (int e = 0; e < VE; ++e) qv[e] = f[e] * scale;
    }
    float m = -INFINITY, l = 0.f;  // the same in all lanes of a row group
    float acc[VE];
#pragma unroll
    for (int e = 0; e < VE; ++e) acc[e] = 0.f;
    auto work = [&](int j0, uint4 (&kk)[NB], uint4 (&vv)[NB]) {
        if (has_fresh) {
#pragma unroll
            for (int u = 0; u < NB; ++u)
                if (row_of(j0, u) == fresh_row) {  // the token itself: not in the cache yet
                    kk[u] = k_new;
                    vv[u] = v_new;
                }
        }
        float sc[NB];
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            float f[VE];
            unpack(kk[u], f);
            sc[u] = 0.f;
#pragma unroll
            for (int e = 0; e < VE; ++e) sc[u] = fmaf(f[e], qv[e], sc[u]);
        }
        // The CPR lanes of a row add up their shares, the NB rows side by side: their exchanges do not wait for each
        // other.  Inside 16 lanes the partner's value comes through the vector unit's own lane permutations
        // (mirror of 16, mirror of 8, pairs two apart, neighbours: every lane ends with the same total, as the sums of
        // both partners of a step are the same two numbers added); only wider steps go through the LDS crossbar.
#pragma unroll
        for (int off = CPR / 2; off >= 16; off >>= 1) {
            float other[NB];
#pragma unroll
            for (int u = 0; u < NB; ++u) other[u] = __shfl_xor(sc[u], off, 64);
#pragma unroll
            for (int u = 0; u < NB; ++u) sc[u] += other[u];
        }
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            if constexpr (CPR >= 16) sc[u] += lane_permuted<0x140>(sc[u]);  // lane i of 16 <- lane 15 - i
            if constexpr (CPR >= 8) sc[u] += lane_permuted<0x141>(sc[u]);   // lane i of 8 <- lane 7 - i
            if constexpr (CPR >= 4) sc[u] += lane_permuted<0x4E>(sc[u]);    // lanes [2, 3, 0, 1] of every four
            if constexpr (CPR >= 2) sc[u] += lane_permuted<0xB1>(sc[u]);    // lanes [1, 0, 3, 2] of every four
        }
        float top = m;
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            if (j0 + u * RG >= n_rows) sc[u] = -INFINITY;
            top = fmaxf(top, sc[u]);
        }
        const float keep = __expf(m - top);  // m == -inf on the first turn: exp(-inf) = 0, and l, acc are 0
        l *= keep;
#pragma unroll
        for (int e = 0; e < VE; ++e) acc[e] *= keep;
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            const float p = __expf(sc[u] - top);  // 0 for the rows past the end
            float f[VE];
            unpack(vv[u], f);
            l += p;
#pragma unroll
            for (int e = 0; e < VE; ++e) acc[e] = fmaf(p, f[e], acc[e]);
        }
        m = top;
    };
    if (j0 < n_rows) {
        work(j0, ka, va);
        for (j0 += step; j0 < n_rows; j0 += step) {
            load_batch(j0, ka, va);
            work(j0, ka, va);
        }
    }
    if (has_fresh && rg == 0 && pos >= lo && pos < n) {  // one workgroup per (batch row, head) has row `pos` among its rows
        *reinterpret_cast<uint4*>(fresh.k_cache + ((size_t)bh * max_seq + pos) * HD + c * VE) = k_new;
        *reinterpret_cast<uint4*>(fresh.v_cache + ((size_t)bh * max_seq + pos) * HD + c * VE) = v_new;
    }
#pragma unroll
    for (int e = 0; e < VE; ++e) partial[rg][c * VE + e] = acc[e];
    if (c == 0) {
        group_max[rg] = m;   // -inf for a row group without rows
        group_sum[rg] = l;
    }
    __syncthreads();
    {
        // The row groups' results are folded by all threads: SG threads per output value take RG / SG row groups each.
        float top = -INFINITY;
        for (int g = tid & 63; g < RG; g += 64) top = fmaxf(top, group_max[g]);
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) top = fmaxf(top, __shfl_xor(top, off, 64));
        const int d = tid % HD, sg = tid / HD;
        float norm = 0.f, o = 0.f;
#pragma unroll
        for (int i = 0; i < RG / SG; ++i) {
            const int g = sg * (RG / SG) + i;
            const float wgt = group_max[g] == -INFINITY ? 0.f : __expf(group_max[g] - top);
            norm = fmaf(group_sum[g], wgt, norm);
            o = fmaf(partial[g][d], wgt, o);
        }
        fold_o[sg][d] = o;
        if (d == 0) {
            fold_norm[sg] = norm;
            if (sg == 0) fold_top = top;
        }
    }
    __syncthreads();
    if (tid < HD) {
        const float top = fold_top;
        float norm = 0.f, o = 0.f;
#pragma unroll
        for (int sg = 0; sg < SG; ++sg) {
            norm += fold_norm[sg];
            o += fold_o[sg][tid];
        }
        if (pieces) {
            float* mine = pieces + ((size_t)bh * splits + blockIdx.y) * (HD + 4);
            // (o is 0 when the workgroup had no rows: top = -inf, norm = 0)
            if (arrivals) {
                // for another workgroup of this launch to read: stores that go through to memory past this chip
                // part's own cache, complete before this thread reaches the barrier below
                __hip_atomic_store(mine + tid, o, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (tid == 0) {
                    __hip_atomic_store(mine + HD, top, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    __hip_atomic_store(mine + HD + 1, norm, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            } else {
                mine[tid] = o;
                if (tid == 0) {
                    mine[HD] = top;
                    mine[HD + 1] = norm;
                }
            }
        } else {
            const long long b = bh / heads;
            const size_t col = (size_t)(bh % heads) * HD + tid;  // of the [batch][heads * head_dim] output
            out[out_kld ? col * out_kld + b : (size_t)b * heads * HD + col] = from_f<T>(o / norm);
        }
    }
    if (!pieces || !arrivals) return;
    // The workgroups of a (batch row, head) count themselves in once their pieces are out; the one that finds all the
    // others counted folds the pieces (as tl_attn_combine does) and leaves the counter at zero for the next call.
    // No workgroup waits for another.  Pieces and counter are written and read by accesses of device scope (they
    // pass the caches that the parts of the chip do not share), so no cache is written back or emptied for them.
    __syncthreads();
    if (tid == 0) {
        const unsigned before = __hip_atomic_fetch_add(arrivals + bh, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        last_to_arrive = before + 1u == (unsigned)splits;
        if (last_to_arrive) __hip_atomic_store(arrivals + bh, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!last_to_arrive) return;
    if (tid < HD) {
        const float* all = pieces + (size_t)bh * splits * (HD + 4);
        float top = -INFINITY;
        for (int s = 0; s < splits; ++s) top = fmaxf(top, __hip_atomic_load(all + (size_t)s * (HD + 4) + HD, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
        float norm = 0.f, o = 0.f;
        for (int s = 0; s < splits; ++s) {
            const float* piece = all + (size_t)s * (HD + 4);
            const float pm = __hip_atomic_load(piece + HD, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const float wgt = pm == -INFINITY ? 0.f : __expf(pm - top);
            norm = fmaf(__hip_atomic_load(piece + HD + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT), wgt, norm);
            o = fmaf(__hip_atomic_load(piece + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT), wgt, o);
        }
        const long long b = bh / heads;
        const size_t col = (size_t)(bh % heads) * HD + tid;
        out[out_kld ? col * out_kld + b : (size_t)b * heads * HD + col] = from_f<T>(o / norm);
    }
}

template <typename T, int HD>
__global__ __launch_bounds__(kAttnThreads) void tl_decode_attn(const T* __restrict__ q, const T* __restrict__ k_cache,
                                                               const T* __restrict__ v_cache, const long long* __restrict__ pos_p,
                                                               T* __restrict__ out, long long out_kld, int heads, long long max_seq,
                                                               float scale, int splits, float* __restrict__ pieces,
                                                               unsigned* __restrict__ arrivals, FreshToken<T> fresh)
{
    decode_attn_body<T, HD, kAttnBatch>(q, k_cache, v_cache, pos_p, out, out_kld, heads, max_seq, scale, splits, pieces, arrivals, fresh);
}

// two workgroups to a compute unit: eight waves per SIMD, 64 registers a lane
template <typename T, int HD>
__global__ __launch_bounds__(kAttnThreads) __attribute__((amdgpu_waves_per_eu(8, 8))) void tl_decode_attn_packed(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache, const long long* __restrict__ pos_p,
    T* __restrict__ out, long long out_kld, int heads, long long max_seq, float scale, int splits, float* __restrict__ pieces,
    unsigned* __restrict__ arrivals, FreshToken<T> fresh)
{
    decode_attn_body<T, HD, kAttnBatchPacked>(q, k_cache, v_cache, pos_p, out, out_kld, heads, max_seq, scale, splits, pieces, arrivals, fresh);
}

// Folds the pieces that a split tl_decode_attn left: one workgroup of HD threads per (batch row, head).
template <typename T, int HD>
__global__ __launch_bounds__(HD) void tl_attn_combine(const float* __restrict__ partial, int splits, T* __restrict__ out,
                                                      long long out_kld, int heads)
{
    const long long bh = blockIdx.x;
    const int tid = threadIdx.x;
    const float* mine = partial + (size_t)bh * splits * (HD + 4);
    float top = -INFINITY;
    for (int s = 0; s < splits; ++s) top = fmaxf(top, mine[(size_t)s * (HD + 4) + HD]);
    float norm = 0.f, o = 0.f;
    for (int s = 0; s < splits; ++s) {
        const float* piece = mine + (size_t)s * (HD + 4);
        const float wgt = piece[HD] == -INFINITY ? 0.f : __expf(piece[HD] - top);
        norm = fmaf(piece[HD + 1], wgt, norm);
        o = fmaf(piece[tid], wgt, o);
    }
    const long long b = bh / heads;
    const size_t col = (size_t)(bh % heads) * HD + tid;
    out[out_kld ? col * out_kld + b : (size_t)b * heads * HD + col] = from_f<T>(o / norm);
}

// x_out = x + y (rounded to T), h_out = x_out / rms(x_out) * weight: the residual add and the RMSNorm that
// follows it in a decoder layer, one workgroup per row.  y may be null (plain RMSNorm of x).
template <typename T>
__global__ __launch_bounds__(256) void tl_add_rmsnorm_k(const T* __restrict__ x, const T* __restrict__ y, const T* __restrict__ weight,
                                                        T* __restrict__ x_out, T* __restrict__ h_out, long long h_kld, int width, float eps)
{
    __shared__ float red[4];
    const size_t row = (size_t)blockIdx.x * width;
    float ss = 0.f;
    for (int i = threadIdx.x; i < width; i += 256) {
        float v = to_f(x[row + i]);
        if (y) v = to_f(from_f<T>(v + to_f(y[row + i])));
        if (x_out) x_out[row + i] = from_f<T>(v);
        ss = fmaf(v, v, ss);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float inv = rsqrtf((red[0] + red[1] + red[2] + red[3]) / (float)width + eps);
    for (int i = threadIdx.x; i < width; i += 256) {
        float v = to_f(x[row + i]);
        if (y) v = to_f(from_f<T>(v + to_f(y[row + i])));
        h_out[h_kld ? (size_t)i * h_kld + blockIdx.x : row + i] = from_f<T>(v * inv * to_f(weight[i]));
    }
}

// The same for rows that are whole 16-byte vectors and at most 4 vectors per thread of a 512-thread
// workgroup: every value is read once, all loads of a thread are in flight together.  With few rows the
// launch has gridDim.y workgroups per row: each reads the whole row (the sum of squares needs it) and writes
// its share of the columns -- the K-major image is written value by value, a row apart, and that is the slow part.
template <typename T>
__global__ __launch_bounds__(512) void tl_add_rmsnorm_vec(const T* __restrict__ x, const T* __restrict__ y, const T* __restrict__ weight,
                                                          T* __restrict__ x_out, T* __restrict__ h_out, long long h_kld, int width, float eps)
{
    constexpr int VE = 16 / (int)sizeof(T);
    constexpr int NV = 4;
    __shared__ float red[8];
    const size_t row = (size_t)blockIdx.x * width;
    const int nvec = width / VE;
    uint4 xv[NV], yv[NV], wv[NV];
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        const int v = min((int)threadIdx.x + k * 512, nvec - 1);
        xv[k] = *reinterpret_cast<const uint4*>(x + row + (size_t)v * VE);
        if (y) yv[k] = *reinterpret_cast<const uint4*>(y + row + (size_t)v * VE);
        wv[k] = *reinterpret_cast<const uint4*>(weight + (size_t)v * VE);
    }
    float val[NV][VE];
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        const T* xe = reinterpret_cast<const T*>(&xv[k]);
        const T* ye = reinterpret_cast<const T*>(&yv[k]);
        const bool live = (int)threadIdx.x + k * 512 < nvec;
#pragma unroll
        for (int e = 0; e < VE; ++e) {
            float v = to_f(xe[e]);
            if (y) v = to_f(from_f<T>(v + to_f(ye[e])));
            val[k][e] = v;
            if (live) ss = fmaf(v, v, ss);
        }
        const bool mine = (((int)threadIdx.x + k * 512) * (int)gridDim.y) / nvec == (int)blockIdx.y;  // this workgroup's share of the columns
        if (live && mine && x_out) {
            uint4 o;
            T* oe = reinterpret_cast<T*>(&o);
#pragma unroll
            for (int e = 0; e < VE; ++e) oe[e] = from_f<T>(val[k][e]);
            *reinterpret_cast<uint4*>(x_out + row + ((size_t)threadIdx.x + k * 512) * VE) = o;
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < 8; ++w) total += red[w];
    const float inv = rsqrtf(total / (float)width + eps);
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        if ((int)threadIdx.x + k * 512 < nvec && (((int)threadIdx.x + k * 512) * (int)gridDim.y) / nvec == (int)blockIdx.y) {
            const T* we = reinterpret_cast<const T*>(&wv[k]);
            uint4 o;
            T* oe = reinterpret_cast<T*>(&o);
#pragma unroll
            for (int e = 0; e < VE; ++e) oe[e] = from_f<T>(val[k][e] * inv * to_f(we[e]));
            const size_t col = ((size_t)threadIdx.x + k * 512) * VE;
            if (h_kld) {
#pragma unroll
                for (int e = 0; e < VE; ++e) h_out[(col + e) * h_kld + blockIdx.x] = oe[e];
            } else {
                *reinterpret_cast<uint4*>(h_out + row + col) = o;
            }
        }
    }
}

// out[r][i] = silu(gu[r][i]) * gu[r][width + i]: the gate of the MLP on the side-by-side gate | up product.
// With out_kld the result goes to a K-major image [width][out_kld]; threads then walk the image in its
// own order (rows of one column side by side, stores contiguous), and the columns past `rows` are zeroed.
template <typename T>
__global__ __launch_bounds__(256) void tl_silu_mul_k(const T* __restrict__ gu, T* __restrict__ out, long long out_kld, long long rows, int width,
                                                     int pairs)
{
    const long long i = blockIdx.x * 256ll + threadIdx.x;
    long long r;
    int c;
    if (out_kld) {
        if (i >= out_kld * width) return;
        c = (int)(i / out_kld);
        r = i - c * out_kld;
        if (r >= rows) {
            out[i] = from_f<T>(0.0f);
            return;
        }
    } else {
        if (i >= rows * width) return;
        r = i / width;
        c = (int)(i - r * width);
    }
    // gate and up of column c: side by side halves of the row, or (pairs) neighbours 2c, 2c + 1
    const T* row = gu + (size_t)r * 2 * width;
    const float g = to_f(pairs ? row[2 * c] : row[c]), u = to_f(pairs ? row[2 * c + 1] : row[width + c]);
    out[i] = from_f<T>(to_f(from_f<T>(g / (1.0f + __expf(-g)))) * u);  // the SiLU is rounded to T before the product, as two separate operators would
}

// The end of a greedy decode step as one launch: token[b] = index of the largest of row b's logits (the first of equal
// ones, a NaN counted as larger than any number, as torch.argmax has it); the first workgroup then moves the position
// on by one, held at max_pos, and marks it in the mask of valid cache slots when there is one.
template <typename T>
__global__ __launch_bounds__(1024) void tl_greedy_advance_k(const T* __restrict__ logits, int vocab, long long* __restrict__ token,
                                                            long long* __restrict__ pos, long long max_pos, unsigned char* __restrict__ mask)
{
    __shared__ float best_v[16];
    __shared__ int best_i[16];
    const T* row = logits + (size_t)blockIdx.x * vocab;
    const int tid = threadIdx.x;
    float bv = 0.f;
    int bi = -1;
    auto better = [](float v, int i, float w, int j) {  // (v, i) before (w, j)?
        if (j < 0) return true;
        const bool vn = v != v, wn = w != w;
        if (vn || wn) return vn && (!wn || i < j);
        return v > w || (v == w && i < j);
    };
    constexpr int VE = 16 / (int)sizeof(T), U = 4;
    if (vocab % VE == 0 && reinterpret_cast<uintptr_t>(logits) % 16 == 0) {
        // 16-byte pieces, U of them asked for before the first is looked at (one value per trip to memory is what
        // makes a plain loop over a row of 32000 take 15 µs)
        const int pieces_n = vocab / VE;
        const uint4* vec = reinterpret_cast<const uint4*>(row);
        for (int first = tid; first < pieces_n; first += 1024 * U) {
            uint4 piece[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int at = first + u * 1024;
                piece[u] = vec[at < pieces_n ? at : first];
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int at = first + u * 1024;
                if (at >= pieces_n) break;
                const T* e = reinterpret_cast<const T*>(&piece[u]);
#pragma unroll
                for (int k = 0; k < VE; ++k)
                    if (better(to_f(e[k]), at * VE + k, bv, bi)) {
                        bv = to_f(e[k]);
                        bi = at * VE + k;
                    }
            }
        }
    } else {
        for (int i = tid; i < vocab; i += 1024) {
            const float v = to_f(row[i]);
            if (better(v, i, bv, bi)) {
                bv = v;
                bi = i;
            }
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, 64);
        const int oi = __shfl_xor(bi, off, 64);
        if (oi >= 0 && better(ov, oi, bv, bi)) {
            bv = ov;
            bi = oi;
        }
    }
    if ((tid & 63) == 0) {
        best_v[tid >> 6] = bv;
        best_i[tid >> 6] = bi;
    }
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < 16; ++w)
            if (best_i[w] >= 0 && better(best_v[w], best_i[w], bv, bi)) {
                bv = best_v[w];
                bi = best_i[w];
            }
        token[blockIdx.x] = bi;
        if (blockIdx.x == 0 && pos) {
            long long p = *pos + 1;
            if (p > max_pos) p = max_pos;
            *pos = p;
            if (mask && p >= 0) mask[p] = 1;
        }
    }
}

int check_common(int dtype, int64_t batch, int heads, int head_dim, int64_t max_seq, const void* pos_dev)
{
    if (dtype != TL_F16 && dtype != TL_F32) return fail(TL_ERR_DTYPE, "dtype code %d unknown", dtype);
    if (batch <= 0 || heads <= 0 || max_seq <= 0 || batch * heads > (1ll << 30)) return fail(TL_ERR_SHAPE, "batch, heads and max_seq must be positive");
    if (head_dim <= 0 || head_dim % 2) return fail(TL_ERR_SHAPE, "head_dim=%d must be positive and even", head_dim);
    if (!pos_dev) return fail(TL_ERR_ARG, "position pointer is null");
    return TL_OK;
}

// Compute units of the current device, read once per device.
int device_units()
{
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 64;
    int units = cached[dev].load(std::memory_order_relaxed);
    if (units == 0) {
        if (hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || units <= 0) units = 64;
        cached[dev].store(units, std::memory_order_relaxed);
    }
    return units;
}

int launched()
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(TL_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString(e));
    return TL_OK;
}

// q|k|v of the token and the rotary tables for the fused form of the attention (all null otherwise)
struct FreshArgs {
    const void* qkv;
    const void* cos_table;
    const void* sin_table;
};

template <typename T, int HD>
int attn_launch(dim3 grid, size_t lds, hipStream_t st, const void* q, const void* k, const void* v, const long long* pos, void* out,
                long long out_kld, int heads, long long max_seq, float scale, int splits, float* partial, unsigned* arrivals, const FreshArgs& f)
{
    // more workgroups than compute units: the kernel of which two fit a compute unit (built for fp16 heads of up to 128 values)
    constexpr bool kPacked = sizeof(T) == 2 && HD <= 128;
    auto kernel = tl_decode_attn<T, HD>;
    if constexpr (kPacked) {
        if ((int64_t)grid.x * splits > device_units()) kernel = tl_decode_attn_packed<T, HD>;
    }
    FreshToken<T> fresh{static_cast<const T*>(f.qkv), static_cast<const T*>(f.cos_table), static_cast<const T*>(f.sin_table),
                        f.qkv ? static_cast<T*>(const_cast<void*>(k)) : nullptr, f.qkv ? static_cast<T*>(const_cast<void*>(v)) : nullptr};
    hipLaunchKernelGGL(kernel, dim3(grid.x, (unsigned)splits), dim3(kAttnThreads), lds, st, static_cast<const T*>(q), static_cast<const T*>(k),
                       static_cast<const T*>(v), pos, static_cast<T*>(out), out_kld, heads, max_seq, scale, splits, partial, arrivals, fresh);
    if (partial && out && !arrivals) {
        auto combine = tl_attn_combine<T, HD>;
        hipLaunchKernelGGL(combine, grid, dim3(HD), 0, st, partial, splits, static_cast<T*>(out), out_kld, heads);
    }
    return TL_OK;
}

template <typename T>
int attn_dispatch(int head_dim, dim3 grid, size_t lds, hipStream_t st, const void* q, const void* k, const void* v,
                  const long long* pos, void* out, long long out_kld, int heads, long long max_seq, float scale, int splits, float* partial,
                  unsigned* arrivals, const FreshArgs& f)
{
    switch (head_dim) {
        case 64: return attn_launch<T, 64>(grid, lds, st, q, k, v, pos, out, out_kld, heads, max_seq, scale, splits, partial, arrivals, f);
        case 128: return attn_launch<T, 128>(grid, lds, st, q, k, v, pos, out, out_kld, heads, max_seq, scale, splits, partial, arrivals, f);
        case 256: return attn_launch<T, 256>(grid, lds, st, q, k, v, pos, out, out_kld, heads, max_seq, scale, splits, partial, arrivals, f);
        default: return fail(TL_ERR_UNSUPPORTED, "head_dim=%d (64, 128 or 256 supported)", head_dim);
    }
}

}  // namespace

extern "C" int tl_rope_cache_update(const void* qkv, int dtype, int64_t batch, int heads, int head_dim,
                                    const void* cos_table, const void* sin_table, const int64_t* pos_dev,
                                    void* q_out, void* k_cache, void* v_cache, int64_t max_seq, void* stream)
{
    if (int rc = check_common(dtype, batch, heads, head_dim, max_seq, pos_dev)) return rc;
    if (!qkv || !cos_table || !sin_table || !q_out || !k_cache || !v_cache) return fail(TL_ERR_ARG, "device pointer is null");
    const int64_t total = batch * heads * head_dim;
    if (ceil_div(total, 256) > INT32_MAX) return fail(TL_ERR_SHAPE, "batch x heads x head_dim = %lld is more than one launch takes", (long long)total);
    dim3 grid((unsigned)ceil_div(total, 256));
    hipStream_t st = static_cast<hipStream_t>(stream);
    const long long* pos = reinterpret_cast<const long long*>(pos_dev);
    if (dtype == TL_F16)
        hipLaunchKernelGGL(tl_rope_cache<__half>, grid, dim3(256), 0, st, static_cast<const __half*>(qkv),
                           static_cast<const __half*>(cos_table), static_cast<const __half*>(sin_table), pos,
                           static_cast<__half*>(q_out), static_cast<__half*>(k_cache), static_cast<__half*>(v_cache), (int)batch, heads,
                           head_dim, (long long)max_seq);
    else
        hipLaunchKernelGGL(tl_rope_cache<float>, grid, dim3(256), 0, st, static_cast<const float*>(qkv),
                           static_cast<const float*>(cos_table), static_cast<const float*>(sin_table), pos,
                           static_cast<float*>(q_out), static_cast<float*>(k_cache), static_cast<float*>(v_cache), (int)batch, heads,
                           head_dim, (long long)max_seq);
    return launched();
}

namespace {
constexpr int kAttnMaxSplits = 8;

int attention(const void* q, const FreshArgs& fresh, const void* k_cache, const void* v_cache, int dtype, int64_t batch, int heads, int head_dim,
              int64_t max_seq, const int64_t* pos_dev, void* out, int64_t out_kmajor_ld, int splits, void* workspace, int64_t workspace_bytes,
              void* stream, uint32_t* arrivals = nullptr)
{
    if (int rc = check_common(dtype, batch, heads, head_dim, max_seq, pos_dev)) return rc;
    if (!(q || fresh.qkv) || !k_cache || !v_cache || (!out && !workspace)) return fail(TL_ERR_ARG, "device pointer is null");
    if (fresh.qkv && (!fresh.cos_table || !fresh.sin_table)) return fail(TL_ERR_ARG, "rotary table pointer is null");
    if (out_kmajor_ld && out_kmajor_ld < batch) return fail(TL_ERR_SHAPE, "out_kmajor_ld=%lld is less than the batch", (long long)out_kmajor_ld);
    const size_t lds = 0;
    if (reinterpret_cast<uintptr_t>(k_cache) % 16 || reinterpret_cast<uintptr_t>(v_cache) % 16 || reinterpret_cast<uintptr_t>(q) % 16)
        return fail(TL_ERR_ALIGN, "q and the caches must be 16-byte aligned");
    if (max_seq * head_dim * (dtype == TL_F16 ? 2 : 4) >= (1ll << 31)) return fail(TL_ERR_UNSUPPORTED, "a head's cache of %lld rows is 2 GiB or more", (long long)max_seq);
    if (reinterpret_cast<uintptr_t>(fresh.qkv) % 16 || reinterpret_cast<uintptr_t>(fresh.cos_table) % 16 || reinterpret_cast<uintptr_t>(fresh.sin_table) % 16)
        return fail(TL_ERR_ALIGN, "qkv and the rotary tables must be 16-byte aligned");
    if (splits < 1 || splits > kAttnMaxSplits) return fail(TL_ERR_ARG, "splits=%d (1 to %d expected)", splits, kAttnMaxSplits);
    const bool leaves_pieces = splits > 1 || !out;
    if (leaves_pieces) {
        const int64_t need = batch * heads * splits * (int64_t)(head_dim + 4) * (int64_t)sizeof(float);
        if (!workspace || workspace_bytes < need || reinterpret_cast<uintptr_t>(workspace) % 16)
            return fail(TL_ERR_SIZE, "%d splits need a 16-byte aligned workspace of %lld bytes", splits, (long long)need);
    }
    dim3 grid((unsigned)(batch * heads));
    hipStream_t st = static_cast<hipStream_t>(stream);
    const long long* pos = reinterpret_cast<const long long*>(pos_dev);
    const float scale = 1.0f / sqrtf((float)head_dim);
    float* partial = leaves_pieces ? static_cast<float*>(workspace) : nullptr;
    if (arrivals && (!out || splits < 2 || reinterpret_cast<uintptr_t>(arrivals) % 4))
        return fail(TL_ERR_ARG, "the fold inside the kernel is for 2 or more splits, an output and 4-byte aligned counters");
    int rc;
    if (dtype == TL_F16) rc = attn_dispatch<__half>(head_dim, grid, lds, st, q, k_cache, v_cache, pos, out, (long long)out_kmajor_ld, heads,
                                                    (long long)max_seq, scale, splits, partial, arrivals, fresh);
    else rc = attn_dispatch<float>(head_dim, grid, lds, st, q, k_cache, v_cache, pos, out, (long long)out_kmajor_ld, heads, (long long)max_seq,
                                   scale, splits, partial, arrivals, fresh);
    if (rc) return rc;
    return launched();
}
}  // namespace

extern "C" int tl_decode_attention(const void* q, const void* k_cache, const void* v_cache, int dtype, int64_t batch, int heads,
                                   int head_dim, int64_t max_seq, const int64_t* pos_dev, void* out, int64_t out_kmajor_ld, void* stream)
{
    return attention(q, FreshArgs{nullptr, nullptr, nullptr}, k_cache, v_cache, dtype, batch, heads, head_dim, max_seq, pos_dev, out, out_kmajor_ld,
                     1, nullptr, 0, stream);
}

extern "C" int tl_decode_attention_split(const void* q, const void* k_cache, const void* v_cache, int dtype, int64_t batch, int heads,
                                         int head_dim, int64_t max_seq, const int64_t* pos_dev, void* out, int64_t out_kmajor_ld,
                                         int splits, void* workspace, int64_t workspace_bytes, void* stream)
{
    return attention(q, FreshArgs{nullptr, nullptr, nullptr}, k_cache, v_cache, dtype, batch, heads, head_dim, max_seq, pos_dev, out, out_kmajor_ld,
                     splits, workspace, workspace_bytes, stream);
}

extern "C" int tl_decode_attention_rope(const void* qkv, const void* cos_table, const void* sin_table, void* k_cache, void* v_cache, int dtype,
                                        int64_t batch, int heads, int head_dim, int64_t max_seq, const int64_t* pos_dev, void* out,
                                        int64_t out_kmajor_ld, int splits, void* workspace, int64_t workspace_bytes, void* stream)
{
    if (!qkv) return fail(TL_ERR_ARG, "device pointer is null");
    return attention(nullptr, FreshArgs{qkv, cos_table, sin_table}, k_cache, v_cache, dtype, batch, heads, head_dim, max_seq, pos_dev, out,
                     out_kmajor_ld, splits, workspace, workspace_bytes, stream);
}

extern "C" int tl_add_rmsnorm(const void* x, const void* y, const void* weight, int dtype, int64_t rows, int width, float eps,
                              void* x_out, void* h_out, int64_t h_kmajor_ld, void* stream)
{
    if (dtype != TL_F16 && dtype != TL_F32) return fail(TL_ERR_DTYPE, "dtype code %d unknown", dtype);
    if (!x || !weight || !h_out) return fail(TL_ERR_ARG, "device pointer is null");
    if (rows <= 0 || width <= 0 || rows > (1ll << 30)) return fail(TL_ERR_SHAPE, "rows and width must be positive");
    if (y && !x_out) return fail(TL_ERR_ARG, "x_out is needed when y is given");
    if (h_kmajor_ld && h_kmajor_ld < rows) return fail(TL_ERR_SHAPE, "h_kmajor_ld=%lld is less than the rows", (long long)h_kmajor_ld);
    const long long kld = (long long)h_kmajor_ld;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int ve = dtype == TL_F16 ? 8 : 4;
    auto aligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
    if (width % ve == 0 && width / ve <= 4 * 512 && aligned(x) && aligned(y) && aligned(weight) && aligned(x_out) && aligned(h_out)) {
        // workgroups per row: as many as spread a small launch over the chip, at most 8
        const int units = device_units();
        const unsigned parts = (unsigned)std::max<int64_t>(1, std::min<int64_t>(8, units / (4 * rows)));
        if (dtype == TL_F16)
            hipLaunchKernelGGL(tl_add_rmsnorm_vec<__half>, dim3((unsigned)rows, parts), dim3(512), 0, st, static_cast<const __half*>(x),
                               static_cast<const __half*>(y), static_cast<const __half*>(weight), static_cast<__half*>(x_out),
                               static_cast<__half*>(h_out), kld, width, eps);
        else
            hipLaunchKernelGGL(tl_add_rmsnorm_vec<float>, dim3((unsigned)rows, parts), dim3(512), 0, st, static_cast<const float*>(x),
                               static_cast<const float*>(y), static_cast<const float*>(weight), static_cast<float*>(x_out),
                               static_cast<float*>(h_out), kld, width, eps);
        return launched();
    }
    if (dtype == TL_F16)
        hipLaunchKernelGGL(tl_add_rmsnorm_k<__half>, dim3((unsigned)rows), dim3(256), 0, st, static_cast<const __half*>(x),
                           static_cast<const __half*>(y), static_cast<const __half*>(weight), static_cast<__half*>(x_out),
                           static_cast<__half*>(h_out), kld, width, eps);
    else
        hipLaunchKernelGGL(tl_add_rmsnorm_k<float>, dim3((unsigned)rows), dim3(256), 0, st, static_cast<const float*>(x),
                           static_cast<const float*>(y), static_cast<const float*>(weight), static_cast<float*>(x_out),
                           static_cast<float*>(h_out), kld, width, eps);
    return launched();
}

namespace {
int silu_mul_call(const void* gate_up, int dtype, int64_t rows, int width, void* out, int64_t out_kmajor_ld, void* stream, int pairs)
{
    if (dtype != TL_F16 && dtype != TL_F32) return fail(TL_ERR_DTYPE, "dtype code %d unknown", dtype);
    if (!gate_up || !out) return fail(TL_ERR_ARG, "device pointer is null");
    if (rows <= 0 || width <= 0 || rows * width > (1ll << 40)) return fail(TL_ERR_SHAPE, "rows and width must be positive");
    if (out_kmajor_ld && out_kmajor_ld < rows) return fail(TL_ERR_SHAPE, "out_kmajor_ld=%lld is less than the rows", (long long)out_kmajor_ld);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (out_kmajor_ld > (1ll << 40) / width || ceil_div((out_kmajor_ld ? out_kmajor_ld : rows) * width, 256) > INT32_MAX)
        return fail(TL_ERR_SHAPE, "rows x width is more than one launch takes");
    const unsigned blocks = (unsigned)ceil_div((out_kmajor_ld ? out_kmajor_ld : rows) * width, 256);
    if (dtype == TL_F16)
        hipLaunchKernelGGL(tl_silu_mul_k<__half>, dim3(blocks), dim3(256), 0, st, static_cast<const __half*>(gate_up), static_cast<__half*>(out),
                           (long long)out_kmajor_ld, (long long)rows, width, pairs);
    else
        hipLaunchKernelGGL(tl_silu_mul_k<float>, dim3(blocks), dim3(256), 0, st, static_cast<const float*>(gate_up), static_cast<float*>(out),
                           (long long)out_kmajor_ld, (long long)rows, width, pairs);
    return launched();
}
}  // namespace

extern "C" int tl_silu_mul(const void* gate_up, int dtype, int64_t rows, int width, void* out, int64_t out_kmajor_ld, void* stream)
{
    return silu_mul_call(gate_up, dtype, rows, width, out, out_kmajor_ld, stream, 0);
}

extern "C" int tl_silu_mul_pairs(const void* gate_up, int dtype, int64_t rows, int width, void* out, int64_t out_kmajor_ld, void* stream)
{
    return silu_mul_call(gate_up, dtype, rows, width, out, out_kmajor_ld, stream, 1);
}

extern "C" int tl_decode_attention_fold(const void* q, const void* qkv, const void* cos_table, const void* sin_table, void* k_cache, void* v_cache,
                                        int dtype, int64_t batch, int heads, int head_dim, int64_t max_seq, const int64_t* pos_dev, void* out,
                                        int64_t out_kmajor_ld, int splits, void* workspace, int64_t workspace_bytes, uint32_t* arrivals,
                                        void* stream)
{
    if (!arrivals) return fail(TL_ERR_ARG, "arrivals is null");
    if ((q != nullptr) == (qkv != nullptr)) return fail(TL_ERR_ARG, "give q, or qkv with the rotary tables");
    return attention(q, FreshArgs{qkv, qkv ? cos_table : nullptr, qkv ? sin_table : nullptr}, k_cache, v_cache, dtype, batch, heads, head_dim, max_seq,
                     pos_dev, out, out_kmajor_ld, splits, workspace, workspace_bytes, stream, arrivals);
}

extern "C" int tl_greedy_advance(const void* logits, int dtype, int64_t batch, int vocab, int64_t* token, int64_t* pos_dev, int64_t max_pos,
                                 void* mask, void* stream)
{
    if (dtype != TL_F16 && dtype != TL_F32) return fail(TL_ERR_DTYPE, "dtype code %d unknown", dtype);
    if (!logits || !token) return fail(TL_ERR_ARG, "device pointer is null");
    if (batch <= 0 || batch > INT32_MAX || vocab <= 0) return fail(TL_ERR_SHAPE, "batch and vocab must be positive");
    if (reinterpret_cast<uintptr_t>(token) % 8 || reinterpret_cast<uintptr_t>(pos_dev) % 8) return fail(TL_ERR_ALIGN, "token and pos must be 8-byte aligned");
    if (pos_dev && max_pos < 0) return fail(TL_ERR_ARG, "max_pos=%lld is negative", (long long)max_pos);
    hipStream_t st = static_cast<hipStream_t>(stream);
    long long* tok = reinterpret_cast<long long*>(token);
    long long* pos = reinterpret_cast<long long*>(pos_dev);
    if (dtype == TL_F16)
        hipLaunchKernelGGL(tl_greedy_advance_k<__half>, dim3((unsigned)batch), dim3(1024), 0, st, static_cast<const __half*>(logits), vocab, tok, pos,
                           (long long)max_pos, static_cast<unsigned char*>(mask));
    else
        hipLaunchKernelGGL(tl_greedy_advance_k<float>, dim3((unsigned)batch), dim3(1024), 0, st, static_cast<const float*>(logits), vocab, tok, pos,
                           (long long)max_pos, static_cast<unsigned char*>(mask));
    return launched();
}
