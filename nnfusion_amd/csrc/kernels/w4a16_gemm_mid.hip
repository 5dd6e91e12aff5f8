// The 128 x 128 and 64 x 256 tile instantiations of the fp16 x int4 MFMA GEMM kernel template
// (w4a16_gemm_dl.h): shapes whose 256 x 256 tiles would leave most of the GPU idle.  With
// p.partial set the kernels write fp32 partial sums of their K range and the caller runs the
// reduction pass; the small tile always does.
#include "w4a16_gemm_dl.h"

namespace nnf
{
    // 128 x 128 (GATE: 128 x (128 + 128)): wavefronts 2 (M) x 4 (N), each 2 x 1 (GATE: 2 x 2) MFMA tiles
    hipError_t launch_gemm_mid(hipStream_t stream, const GemmParams& p, bool gate, bool hb, bool hr)
    {
        if (p.partial)
        {
            if (gate)
                return launch_gemm_dl<2, 4, 2, 2, true, false, false, true, 4>(stream, p);
            return launch_gemm_dl<2, 4, 2, 1, false, false, false, true, 4>(stream, p);
        }
        if (gate)
            return launch_gemm_dl<2, 4, 2, 2, true, false, false, false, 4>(stream, p);
        if (hb && hr)
            return launch_gemm_dl<2, 4, 2, 1, false, true, true, false, 4>(stream, p);
        if (hb)
            return launch_gemm_dl<2, 4, 2, 1, false, true, false, false, 4>(stream, p);
        if (hr)
            return launch_gemm_dl<2, 4, 2, 1, false, false, true, false, 4>(stream, p);
        return launch_gemm_dl<2, 4, 2, 1, false, false, false, false, 4>(stream, p);
    }

    // 64 x 256 (GATE: 64 x (256 + 256)): wavefronts 1 (M) x 8 (N), each 2 x 1 (GATE: 2 x 2) MFMA tiles
    hipError_t launch_gemm_small(hipStream_t stream, const GemmParams& p, bool gate, bool, bool)
    {
        if (!p.partial)
            return hipErrorInvalidValue;
        if (gate)
            return launch_gemm_dl<1, 8, 2, 2, true, false, false, true, 4>(stream, p);
        return launch_gemm_dl<1, 8, 2, 1, false, false, false, true, 4>(stream, p);
    }

    // 32 x 256 (GATE: 32 x (256 + 256)): wavefronts 1 (M) x 8 (N), each 1 x 1 (GATE: 1 x 2) MFMA tiles; for
    // M <= 32, where a 64-row tile would fetch as many (repeated) activation rows as weights
    hipError_t launch_gemm_tiny(hipStream_t stream, const GemmParams& p, bool gate, bool, bool)
    {
        if (!p.partial)
            return hipErrorInvalidValue;
        if (gate)
            return launch_gemm_dl<1, 8, 1, 2, true, false, false, true, 4>(stream, p);
        return launch_gemm_dl<1, 8, 1, 1, false, false, false, true, 4>(stream, p);
    }
} // namespace nnf
