// TEST / BASELINE INFRASTRUCTURE ONLY -- this repository's port of the
// reference's CPU SIMD kernels, timed by bench.py as the `cpu_baseline` leg
// (kind "port") where the reference's own build is not usable, and checked
// against the exact product before it is timed.  The shipped library never
// links or calls it.
//
// Format restated: "min"-grouped merged TCSC
//   (ternaryLLM_CPU/src/TCSC.hpp:6-34 naive TCSC, :99-174 grouping).
//   For a group of G columns, A = min over the group of min(#pos, #neg).
//   The first A (+,-) pairs of every column are stored together
//   (interleaved: p0 n0 p1 n1 ... per k for the GEMM kernel;
//    blocked: G pos then G neg per k for the GEMV kernel), then per column
//   its leftover +1 rows and its leftover -1 rows.  Metadata per group:
//   [pair_start, pair_end, then (pos_end, neg_end) per column] = 2 + 2G ints.
// Kernels restated (same register blocking and loop order, unaligned loads):
//   GEMM  32 rows x 8 columns, AVX2, OpenMP over column groups
//         (GEMM_CPU_FP32.cpp:2956-3221); X is [K][M], result is [N][M].
//   GEMV  64 columns per group, AVX2 i32 gathers on the paired part, scalar
//         leftovers (GEMM_CPU_FP32.cpp:15008-15081); x row-major, int32 indices;
//         and its AVX-512 sibling (:15684-15729).
#include <immintrin.h>
#include <omp.h>

#include <algorithm>
#include <cstdint>
#include <vector>

namespace {

struct Grouped {
    int G;
    bool interleaved;
    std::vector<int32_t> meta;
    std::vector<int16_t> idx16;
    std::vector<int32_t> idx32;
};

struct ColumnLists {
    std::vector<int32_t> pos_ptr, neg_ptr;
    std::vector<int32_t> pos_row, neg_row;
};

ColumnLists scan_columns(const int8_t* W, int K, int N)
{
    ColumnLists c;
    c.pos_ptr.assign(N + 1, 0);
    c.neg_ptr.assign(N + 1, 0);
    for (int k = 0; k < K; ++k)
        for (int n = 0; n < N; ++n) {
            int8_t v = W[(size_t)k * N + n];
            if (v >= 1) c.pos_ptr[n + 1]++;
            else if (v <= -1) c.neg_ptr[n + 1]++;
        }
    for (int n = 0; n < N; ++n) {
        c.pos_ptr[n + 1] += c.pos_ptr[n];
        c.neg_ptr[n + 1] += c.neg_ptr[n];
    }
    c.pos_row.resize(c.pos_ptr[N]);
    c.neg_row.resize(c.neg_ptr[N]);
    std::vector<int32_t> pc(c.pos_ptr.begin(), c.pos_ptr.end() - 1), nc(c.neg_ptr.begin(), c.neg_ptr.end() - 1);
    for (int k = 0; k < K; ++k)
        for (int n = 0; n < N; ++n) {
            int8_t v = W[(size_t)k * N + n];
            if (v >= 1) c.pos_row[pc[n]++] = k;
            else if (v <= -1) c.neg_row[nc[n]++] = k;
        }
    return c;
}

Grouped* build_grouped(const int8_t* W, int K, int N, int G, bool interleaved)
{
    ColumnLists c = scan_columns(W, K, N);
    Grouped* g = new Grouped;
    g->G = G;
    g->interleaved = interleaved;
    std::vector<int32_t> stream;
    stream.reserve(c.pos_row.size() + c.neg_row.size());
    int32_t cursor = 0;
    for (int n0 = 0; n0 < N; n0 += G) {
        int A = INT32_MAX;
        for (int i = 0; i < G; ++i) {
            int p = c.pos_ptr[n0 + i + 1] - c.pos_ptr[n0 + i];
            int q = c.neg_ptr[n0 + i + 1] - c.neg_ptr[n0 + i];
            A = std::min(A, std::min(p, q));
        }
        for (int k = 0; k < A; ++k) {
            if (interleaved) {
                for (int i = 0; i < G; ++i) {
                    stream.push_back(c.pos_row[c.pos_ptr[n0 + i] + k]);
                    stream.push_back(c.neg_row[c.neg_ptr[n0 + i] + k]);
                }
            } else {
                for (int i = 0; i < G; ++i) stream.push_back(c.pos_row[c.pos_ptr[n0 + i] + k]);
                for (int i = 0; i < G; ++i) stream.push_back(c.neg_row[c.neg_ptr[n0 + i] + k]);
            }
        }
        g->meta.push_back(cursor);
        cursor += A * G * 2;
        g->meta.push_back(cursor);
        for (int i = 0; i < G; ++i) {
            for (int k = c.pos_ptr[n0 + i] + A; k < c.pos_ptr[n0 + i + 1]; ++k) stream.push_back(c.pos_row[k]);
            cursor += c.pos_ptr[n0 + i + 1] - c.pos_ptr[n0 + i] - A;
            g->meta.push_back(cursor);
            for (int k = c.neg_ptr[n0 + i] + A; k < c.neg_ptr[n0 + i + 1]; ++k) stream.push_back(c.neg_row[k]);
            cursor += c.neg_ptr[n0 + i + 1] - c.neg_ptr[n0 + i] - A;
            g->meta.push_back(cursor);
        }
    }
    g->idx32 = stream;
    g->idx16.assign(stream.begin(), stream.end());
    return g;
}

}  // namespace

extern "C" {

void* port_group_build(const int8_t* W, int K, int N, int G, int interleaved)
{
    if (N % G != 0) return nullptr;
    return build_grouped(W, K, N, G, interleaved != 0);
}
void port_group_free(void* h) { delete static_cast<Grouped*>(h); }
int64_t port_group_index_count(void* h) { return (int64_t) static_cast<Grouped*>(h)->idx32.size(); }
int64_t port_group_meta_count(void* h) { return (int64_t) static_cast<Grouped*>(h)->meta.size(); }
const int32_t* port_group_meta(void* h) { return static_cast<Grouped*>(h)->meta.data(); }
const int16_t* port_group_index16(void* h) { return static_cast<Grouped*>(h)->idx16.data(); }
int port_threads(void) { return omp_get_max_threads(); }

// X: [K][M] floats, result: [N][M] floats, M % 32 == 0, format built with G = 8, interleaved.
void port_gemm_32xg8_avx2(const float* X, void* h, float* result, int M, int N, int K)
{
    (void)K;
    const Grouped* g = static_cast<const Grouped*>(h);
    const int16_t* idx = g->idx16.data();
    const int32_t* meta = g->meta.data();
#pragma omp parallel for schedule(static)
    for (int j = 0; j < N / 8; ++j) {
        const int32_t* gd = meta + (size_t)j * 18;
        for (int i = 0; i < M; i += 32) {
            __m256 acc[8][4];
            for (int c = 0; c < 8; ++c)
                for (int q = 0; q < 4; ++q) acc[c][q] = _mm256_setzero_ps();
            for (int k = gd[0]; k < gd[1]; k += 16) {
                for (int c = 0; c < 8; ++c) {
                    const float* xp = X + (size_t)idx[k + 2 * c] * M + i;
                    const float* xn = X + (size_t)idx[k + 2 * c + 1] * M + i;
                    for (int q = 0; q < 4; ++q)
                        acc[c][q] = _mm256_add_ps(acc[c][q],
                                                  _mm256_sub_ps(_mm256_loadu_ps(xp + 8 * q), _mm256_loadu_ps(xn + 8 * q)));
                }
            }
            for (int c = 0; c < 8; ++c) {
                for (int k = gd[1 + 2 * c]; k < gd[2 + 2 * c]; ++k) {
                    const float* xp = X + (size_t)idx[k] * M + i;
                    for (int q = 0; q < 4; ++q) acc[c][q] = _mm256_add_ps(acc[c][q], _mm256_loadu_ps(xp + 8 * q));
                }
                for (int k = gd[2 + 2 * c]; k < gd[3 + 2 * c]; ++k) {
                    const float* xn = X + (size_t)idx[k] * M + i;
                    for (int q = 0; q < 4; ++q) acc[c][q] = _mm256_sub_ps(acc[c][q], _mm256_loadu_ps(xn + 8 * q));
                }
            }
            for (int c = 0; c < 8; ++c)
                for (int q = 0; q < 4; ++q)
                    _mm256_storeu_ps(result + (size_t)(j * 8 + c) * M + i + 8 * q, acc[c][q]);
        }
    }
}

// x: [K] floats, result: [N] floats, format built with G = 64, blocked (not interleaved), int32 indices.
void port_gemv_g64_avx2(const float* x, void* h, float* result, int N, int K)
{
    (void)K;
    const Grouped* g = static_cast<const Grouped*>(h);
    const int32_t* idx = g->idx32.data();
    const int32_t* meta = g->meta.data();
#pragma omp parallel for schedule(static)
    for (int j = 0; j < N / 64; ++j) {
        const int32_t* gd = meta + (size_t)j * 130;
        __m256 acc[8];
        for (int q = 0; q < 8; ++q) acc[q] = _mm256_setzero_ps();
        for (int k = gd[0]; k < gd[1]; k += 128) {
            for (int q = 0; q < 8; ++q) {
                __m256i ip = _mm256_loadu_si256(reinterpret_cast<const __m256i*>(idx + k + 8 * q));
                __m256i in = _mm256_loadu_si256(reinterpret_cast<const __m256i*>(idx + k + 64 + 8 * q));
                acc[q] = _mm256_add_ps(acc[q], _mm256_sub_ps(_mm256_i32gather_ps(x, ip, 4), _mm256_i32gather_ps(x, in, 4)));
            }
        }
        float* y = result + (size_t)j * 64;
        for (int q = 0; q < 8; ++q) _mm256_storeu_ps(y + 8 * q, acc[q]);
        for (int c = 0; c < 64; ++c) {
            float s = y[c];
            for (int k = gd[1 + 2 * c]; k < gd[2 + 2 * c]; ++k) s += x[idx[k]];
            for (int k = gd[2 + 2 * c]; k < gd[3 + 2 * c]; ++k) s -= x[idx[k]];
            y[c] = s;
        }
    }
}

// The same with 16-lane gathers (GEMM_CPU_FP32.cpp:15684-15729): four accumulators of 16 columns.
__attribute__((target("avx512f"))) void port_gemv_g64_avx512(const float* x, void* h, float* result, int N, int K)
{
    (void)K;
    const Grouped* g = static_cast<const Grouped*>(h);
    const int32_t* idx = g->idx32.data();
    const int32_t* meta = g->meta.data();
#pragma omp parallel for schedule(static)
    for (int j = 0; j < N / 64; ++j) {
        const int32_t* gd = meta + (size_t)j * 130;
        __m512 acc[4];
        for (int q = 0; q < 4; ++q) acc[q] = _mm512_setzero_ps();
        for (int k = gd[0]; k < gd[1]; k += 128) {
            for (int q = 0; q < 4; ++q) {
                __m512i ip = _mm512_loadu_si512(idx + k + 16 * q);
                __m512i in = _mm512_loadu_si512(idx + k + 64 + 16 * q);
                acc[q] = _mm512_add_ps(acc[q], _mm512_sub_ps(_mm512_i32gather_ps(ip, x, 4), _mm512_i32gather_ps(in, x, 4)));
            }
        }
        float* y = result + (size_t)j * 64;
        for (int q = 0; q < 4; ++q) _mm512_storeu_ps(y + 16 * q, acc[q]);
        for (int c = 0; c < 64; ++c) {
            float s = y[c];
            for (int k = gd[1 + 2 * c]; k < gd[2 + 2 * c]; ++k) s += x[idx[k]];
            for (int k = gd[2 + 2 * c]; k < gd[3 + 2 * c]; ++k) s -= x[idx[k]];
            y[c] = s;
        }
    }
}

}  // extern "C"
