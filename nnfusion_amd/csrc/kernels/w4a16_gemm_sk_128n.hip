// fp16 x int4 tile GEMM, tiles of 128 x 128 (one column tile per wavefront): the instantiations of w4a16_gemm_sk.h.
#include "w4a16_gemm_sk_launch.h"

namespace nnf
{
    hipError_t launch_gemm_sk_128_narrow(hipStream_t stream, const SkGemmParams& p, int grid)
    {
        return gemm_sk::launch_tile_height_plain<4, 1>(stream, p, grid);
    }
} // namespace nnf
