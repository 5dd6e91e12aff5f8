// fp16 x int4 tile GEMM with groups of 32 and a scalar zero point or one per (row, group): the instantiations of
// w4a16_gemm_sk.h.
#include "w4a16_gemm_sk_launch.h"

namespace nnf
{
    hipError_t launch_gemm_sk_q5(hipStream_t stream, const SkGemmParams& p, int grid, int tile_rows, int tile_cols)
    {
        return gemm_sk::launch_tiles_q<5>(stream, p, grid, tile_rows, tile_cols);
    }
} // namespace nnf
