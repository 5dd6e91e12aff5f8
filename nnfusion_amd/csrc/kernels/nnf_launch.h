// Internal launch functions behind the C ABI (one per kernel family).  Each validates nothing:
// nnf_api.hip checks shapes, alignment and workspace before calling in.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace nnf
{
    // largest dynamic LDS a workgroup may ask for on gfx950 (160 KiB per CU)
    constexpr size_t MAX_LDS_BYTES = 160 * 1024;

    hipError_t launch_w4a16_gemv(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y,
                                 int M, int N, int K, int zp, int num_cu);
    // true when launch_w4a16_gemv can stage the activations of one pass in LDS
    bool w4a16_gemv_supported(int M, int K);

    // one activation row (M = 1): the row-streaming kernel
    hipError_t launch_w4a16_gemv_rows(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int N,
                                      int K, int zp, int num_cu);
    bool w4a16_gemv_rows_supported(int M, int N, int K, int num_cu);

    // 2 <= M <= 16, K = 1024 / 2048 / 4096 / 8192: weights streamed through LDS rings, activations in registers
    hipError_t launch_w4a16_mrows(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M, int N,
                                  int K, int zp, int num_cu);
    bool w4a16_mrows_supported(int M, int N, int K, int num_cu);
    bool w4a16_mrows_preferred(int M, int N, int K, int num_cu); // where the library picks it without being told
    // K above 8192: the same kernel over ranges of K, fp32 sums to partial[ranges][M][N] for the reduction pass
    int w4a16_mrows_ksplits(int M, int N, int K, int num_cu); // 0: does not apply
    hipError_t launch_w4a16_mrows_split(hipStream_t stream, const void* A, const void* Wq, const void* S, float* partial,
                                        int M, int N, int K, int zp, int num_cu);

    hipError_t launch_w4a16_skinny(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M,
                                   int N, int K, int zp, int num_cu);
    // true when one workgroup can hold the activations (M <= 16 rows of K) in LDS
    bool w4a16_skinny_supported(int M, int N, int K);
    int& skinny_direct_min_rows(); // experiments: see w4a16_skinny.hip

    // M <= 16 with activations too large for LDS: the same kernel over `ksplits` ranges of K, fp32 partial sums
    // [ksplits][M][N] (to be added by the GEMM's reduction pass); w4a16_skinny_ksplits returns 0 when not applicable
    int w4a16_skinny_ksplits(int M, int N, int K);
    hipError_t launch_w4a16_skinny_split(hipStream_t stream, const void* A, const void* Wq, const void* S, float* partial,
                                         int M, int N, int K, int zp, int ksplits, int num_cu);

    // MFMA GEMM (any M) with the RMSNorm prologue and bias / residual / SiLU-gate epilogues.
    // rms_ws: nnf::workspace::rms_rows(M, K) bytes, needed when rms_gamma != nullptr;
    // partial_ws: nnf::workspace::gemm_partial_bytes(...) for the plan of the shape (may be 0 bytes).
    // M <= 16 shapes that the GEMV kernel can serve go through it (plus an element-wise epilogue kernel),
    // unless gemm_only asks for the MFMA GEMM tiles whatever M is.
    hipError_t launch_w4a16_gemm(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M,
                                 int N, int K, int zp, const void* rms_gamma, float rms_eps, const void* bias,
                                 const void* residual, int act, void* rms_ws, void* partial_ws, int num_cu,
                                 bool gemm_only = false);

    // W8A8: acc != nullptr writes the raw int32 accumulators, otherwise Y = fp16(acc * s_tok * s_ch).
    // partial_ws: nnf::workspace::w8a8_gemm(M, N, K) bytes (0 for the M <= 16 kernel)
    hipError_t launch_w8a8(hipStream_t stream, const void* A, const void* s_tok, const void* W, const void* s_ch,
                           void* Y, void* acc, int M, int N, int K, int num_cu, void* partial_ws);
    // the MFMA GEMM behind launch_w8a8 (any M)
    hipError_t launch_w8a8_gemm(hipStream_t stream, const void* A, const void* s_tok, const void* W, const void* s_ch,
                                void* Y, void* acc, int M, int N, int K, void* partial_ws);
    bool w8a8_skinny_supported(int M, int K);
    // one activation row (M = 1): the row-streaming kernel; acc != nullptr writes the raw int32 sums
    hipError_t launch_w8a8_gemv_rows(hipStream_t stream, const void* A, const void* s_tok, const void* W, const void* s_ch,
                                     void* Y, void* acc, int N, int K, int num_cu);
    bool w8a8_gemv_rows_supported(int M, int N, int K, int num_cu);
    // 2 <= M <= 32, K = 2048, 4096, 6144 or 8192: the row-streaming MFMA kernel (w8a8_mrows.hip)
    hipError_t launch_w8a8_mrows(hipStream_t stream, const void* A, const void* s_tok, const void* W, const void* s_ch,
                                 void* Y, void* acc, int M, int N, int K, int num_cu);
    bool w8a8_mrows_supported(int M, int N, int K, int num_cu);
    bool w8a8_mrows_preferred(int M, int N, int K, int num_cu); // where the library picks it without being told

    // Tuning knobs for experiments (not part of the public ABI): 0 = automatic.
    struct Tuning
    {
        int force_path = 0;  // 1 = VALU GEMV, 2 = MFMA skinny, 3 = MFMA GEMM, 4 = row-streaming GEMV (M = 1),
                             // 5 = row-streaming MFMA kernel (2 <= M <= 16) where it applies
        int skinny_cps = 0;  // chunks (groups of 128) per wavefront
        int skinny_wg_per_cu = 0;
        int gemm_tile = 0;   // 1 + nnf::workspace::GemmTile
        int gemm_splits = 0; // K ranges of the mid / small tile kernels
    };
    extern Tuning g_tuning;
} // namespace nnf
