// TEST INFRASTRUCTURE ONLY -- C-ABI shim around the reference's own CPU kernels.
//
// This file holds no kernel code.  It is compiled together with the
// reference's ternaryLLM_CPU/src/GEMM_CPU_FP32.cpp and includes the reference's
// TCSC.hpp, both read in place from the reference checkout (see Makefile: the
// include path points there, nothing is copied), into oracle/_ref/libref_cpu.so.
// The shim only (1) builds the reference's grouped merged-TCSC format from a
// dense int8 W and (2) forwards to the two kernels the reference's own
// benchmark uses as its headline choices:
//   GEMM_CPU_FP32_colMajor_TCSC_Merged_GroupMin_32xG8_AVX2_OpenMP
//       (GEMM_CPU_FP32.cpp:2956, called at main.cpp:1088)
//   GEMM_CPU_FP32_colMajor_TCSC_Merged_GroupMin_32xG16_AVX512_OpenMP
//       (GEMM_CPU_FP32.cpp:8365)
// Both use 32-byte/64-byte *aligned* loads on X and on the result, so callers
// must hand in 64-byte aligned buffers and M % 32 == 0.  The reference's GEMV
// kernels are not exported: they issue aligned index loads at offsets that are
// not 32-byte multiples (GEMM_CPU_FP32.cpp:15021) and fault when built with
// GCC, so the M = 1 baseline is timed with this repository's own port instead.
#include <algorithm>
#include <cstdint>
#include <cstring>
#include <string>
#include <vector>
#include <iostream>

#include "TCSC.hpp"
#include "GEMM_CPU_FP32.hpp"

namespace {
struct GroupFormat {
    MergedTCSC_Group* fmt;
};
}  // namespace

extern "C" {

// W: row-major int8 [K][N].  group = 8 (AVX2 kernel) or 16 (AVX-512 kernel),
// grouping method "min", interleaved indices, as at main.cpp:1030-1034.
void* ref_group_build(const int8_t* W, int K, int N, int group)
{
    SparseFormat naive(W, K, N);
    GroupFormat* g = new GroupFormat;
    g->fmt = new MergedTCSC_Group(naive, K, N, group, "min", true);
    return g;
}

void ref_group_free(void* h)
{
    GroupFormat* g = static_cast<GroupFormat*>(h);
    if (!g) return;
    delete g->fmt;
    delete g;
}

int64_t ref_group_index_count(void* h) { return (int64_t) static_cast<GroupFormat*>(h)->fmt->row_index.size(); }
int64_t ref_group_meta_count(void* h) { return (int64_t) static_cast<GroupFormat*>(h)->fmt->metadata.size(); }
const int16_t* ref_group_index(void* h) { return static_cast<GroupFormat*>(h)->fmt->row_index.data(); }
const int32_t* ref_group_meta(void* h) { return static_cast<GroupFormat*>(h)->fmt->metadata.data(); }

// X: [K][M] floats (64-byte aligned), result: [N][M] floats (64-byte aligned).
void ref_gemm_32xg8_avx2(const float* X, void* h, float* result, int M, int N, int K)
{
    GroupFormat* g = static_cast<GroupFormat*>(h);
    GEMM_CPU_FP32_colMajor_TCSC_Merged_GroupMin_32xG8_AVX2_OpenMP(
        X, g->fmt->metadata.data(), g->fmt->row_index.data(), result, M, N, K);
}

void ref_gemm_32xg16_avx512(const float* X, void* h, float* result, int M, int N, int K)
{
    GroupFormat* g = static_cast<GroupFormat*>(h);
    GEMM_CPU_FP32_colMajor_TCSC_Merged_GroupMin_32xG16_AVX512_OpenMP(
        X, g->fmt->metadata.data(), g->fmt->row_index.data(), result, M, N, K);
}

}  // extern "C"
