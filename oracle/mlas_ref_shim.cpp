// TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
//
// C entry points over the MLAS library that ships (as source) inside the nnfusion tree at
// thirdparty/mlas.  This file is compiled together with those sources, where they lie, into
// oracle/_ref/libmlas_ref.so (see oracle/Makefile); no reference source is copied.  It exposes
// exactly the routine cpu::DotMlas emits (src/nnfusion/core/kernels/cpu/mlas/dot.cpp:89-100):
//   MlasGemm(TransA, TransB, M, N, K, 1.0, A, lda, B, ldb, 0.0, C, ldc, thread_pool)
// and the u8 x s8 -> s32 MlasGemm (thirdparty/mlas/inc/mlas.h:147-163) used to cross-check the
// int8 accumulators.
#include <chrono>
#include <cstddef>
#include <cstdint>
#include "mlas.h"

extern "C" {

void mlas_ref_sgemm(int transA, int transB, size_t M, size_t N, size_t K,
                    const float* A, size_t lda, const float* B, size_t ldb, float* C, size_t ldc)
{
    MlasGemm(transA ? CblasTrans : CblasNoTrans, transB ? CblasTrans : CblasNoTrans,
             M, N, K, 1.0f, A, lda, B, ldb, 0.0f, C, ldc, nullptr);
}

// A is u8 [M,K] with zero point offa, B is s8 [K,N] (row-major, ldb = N) with zero point offb.
void mlas_ref_qgemm_u8s8(size_t M, size_t N, size_t K, const uint8_t* A, size_t lda, uint8_t offa,
                         const int8_t* B, size_t ldb, int8_t offb, int32_t* C, size_t ldc)
{
    MlasGemm(M, N, K, A, lda, offa, B, ldb, offb, C, ldc, nullptr);
}

// Timing loop in the shape of the generated CPU main_test
// (src/nnfusion/engine/pass/codegen/cpu_codegen_pass.cpp:301-335): warm-ups, then timed
// iterations with std::chrono, mean in ms; weights are [N,K] (transB form, ldb = K).
double mlas_ref_time_sgemm_nt(size_t M, size_t N, size_t K, const float* A, const float* Bt, float* C,
                              int warmup, int iters, double* min_ms)
{
    for (int i = 0; i < warmup; ++i)
        MlasGemm(CblasNoTrans, CblasTrans, M, N, K, 1.0f, A, K, Bt, K, 0.0f, C, N, nullptr);
    double total = 0.0, best = 1e300;
    for (int i = 0; i < iters; ++i)
    {
        auto t0 = std::chrono::high_resolution_clock::now();
        MlasGemm(CblasNoTrans, CblasTrans, M, N, K, 1.0f, A, K, Bt, K, 0.0f, C, N, nullptr);
        auto t1 = std::chrono::high_resolution_clock::now();
        double ms = std::chrono::duration<double, std::milli>(t1 - t0).count();
        total += ms;
        if (ms < best)
            best = ms;
    }
    if (min_ms)
        *min_ms = best;
    return iters > 0 ? total / iters : 0.0;
}

} // extern "C"
