// fp16 x int4 tile GEMM, tiles of 32 x 256: the instantiations of w4a16_gemm_sk.h for this tile height.
#include "w4a16_gemm_sk_launch.h"

namespace nnf
{
    hipError_t launch_gemm_sk_32(hipStream_t stream, const SkGemmParams& p, int grid, bool gate)
    {
        return gemm_sk::launch_tile_height<1, 2>(stream, p, grid, gate);
    }
} // namespace nnf
