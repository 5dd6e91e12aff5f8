// Scratch-memory sizes of the launcher entry points: pure host arithmetic, shared by the library
// (nnf_*_workspace_bytes) and by the emitters, which reserve the scratch tensor at compile time.
#pragma once

#include <stddef.h>

namespace nnf
{
    namespace workspace
    {
        inline size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }
        // per-row statistics of the RMSNorm prologue
        inline size_t rms_rows(int M) { return M > 0 ? align256((size_t)M * sizeof(float)) : 0; }
        inline size_t w4a16_gemm(int, int, int, int) { return 0; }
        inline size_t w4a16_gemm_fused(int M, int, int, int, int) { return rms_rows(M); }
        inline size_t w8a8_gemm(int, int, int) { return 0; }
        // [ rstd: M floats ][ h: M x I fp16 ]
        inline size_t fused_mlp_w4a16(int M, int, int I, int)
        {
            return (M > 0 && I > 0) ? rms_rows(M) + align256((size_t)M * I * 2) : 0;
        }
    } // namespace workspace
} // namespace nnf
