// Host side of one tile height of the fp16 x int4 tile GEMM (w4a16_gemm_sk.h): picks the instantiation for the
// epilogue asked for and launches it.  Included by one translation unit per tile height, so that they compile in
// parallel.
#pragma once

#include "w4a16_gemm_sk.h"

namespace nnf
{
    namespace gemm_sk
    {
        template <int TM, int TN, bool GATE, bool BIAS, bool RESID, bool RMS>
        hipError_t launch_instance(hipStream_t stream, const SkGemmParams& p, int grid)
        {
            using T = Tile<TM, TN>;
            auto kernel = &w4a16_gemm_sk_kernel<TM, TN, GATE, BIAS, RESID, RMS>;
            if (T::LDS_BYTES > 48 * 1024)
            {
                static LdsGrant granted;
                const hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), granted, T::LDS_BYTES);
                if (e != hipSuccess)
                    return e;
            }
            launch_sk_kernel(kernel, grid, T::LDS_BYTES, stream, p);
            hipError_t e = hipGetLastError();
            if (e != hipSuccess || !p.partial || p.sync)
                return e;
            // tiles shared by several workgroups: their parts are added and finished by a second launch (unless the
            // workgroups did it themselves: p.sync)
            constexpr int ROUNDS = TM; // blocks of 32 rows
            hipLaunchKernelGGL((w4a16_gemm_sk_fixup_kernel<TM, TN, GATE, BIAS, RESID, RMS>), dim3(p.tiles_m * p.tiles_n * ROUNDS * WAVES),
                               dim3(64), 0, stream, p, grid);
            return hipGetLastError();
        }

        template <int TM, int TN>
        hipError_t launch_tile_height(hipStream_t stream, const SkGemmParams& p, int grid, bool gate)
        {
            const bool hb = p.bias != nullptr, hr = p.residual != nullptr, rms = p.gamma != nullptr;
            if (gate)
                return rms ? launch_instance<TM, TN, true, false, false, true>(stream, p, grid)
                           : launch_instance<TM, TN, true, false, false, false>(stream, p, grid);
            if (hb && hr)
                return rms ? launch_instance<TM, TN, false, true, true, true>(stream, p, grid)
                           : launch_instance<TM, TN, false, true, true, false>(stream, p, grid);
            if (hb)
                return rms ? launch_instance<TM, TN, false, true, false, true>(stream, p, grid)
                           : launch_instance<TM, TN, false, true, false, false>(stream, p, grid);
            if (hr)
                return rms ? launch_instance<TM, TN, false, false, true, true>(stream, p, grid)
                           : launch_instance<TM, TN, false, false, true, false>(stream, p, grid);
            return rms ? launch_instance<TM, TN, false, false, false, true>(stream, p, grid)
                       : launch_instance<TM, TN, false, false, false, false>(stream, p, grid);
        }
        // the forms without SiLU-gate (tiles one column tile per wavefront wide have no gate | up pairs)
        template <int TM, int TN>
        hipError_t launch_tile_height_plain(hipStream_t stream, const SkGemmParams& p, int grid)
        {
            const bool hb = p.bias != nullptr, hr = p.residual != nullptr, rms = p.gamma != nullptr;
            if (hb && hr)
                return rms ? launch_instance<TM, TN, false, true, true, true>(stream, p, grid)
                           : launch_instance<TM, TN, false, true, true, false>(stream, p, grid);
            if (hb)
                return rms ? launch_instance<TM, TN, false, true, false, true>(stream, p, grid)
                           : launch_instance<TM, TN, false, true, false, false>(stream, p, grid);
            if (hr)
                return rms ? launch_instance<TM, TN, false, false, true, true>(stream, p, grid)
                           : launch_instance<TM, TN, false, false, true, false>(stream, p, grid);
            return rms ? launch_instance<TM, TN, false, false, false, true>(stream, p, grid)
                       : launch_instance<TM, TN, false, false, false, false>(stream, p, grid);
        }
        // other block parameters (QG = log2 of the group size; zero points per (row, group) when p.zps is set): the
        // plain product; the second launch does not depend on them
        template <int TM, int TN, int QG>
        hipError_t launch_instance_q(hipStream_t stream, const SkGemmParams& p, int grid)
        {
            using T = Tile<TM, TN>;
            auto kernel = &w4a16_gemm_sk_kernel<TM, TN, false, false, false, false, QG>;
            if (T::LDS_BYTES > 48 * 1024)
            {
                static LdsGrant granted;
                const hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), granted, T::LDS_BYTES);
                if (e != hipSuccess)
                    return e;
            }
            launch_sk_kernel(kernel, grid, T::LDS_BYTES, stream, p);
            hipError_t e = hipGetLastError();
            if (e != hipSuccess || !p.partial || p.sync)
                return e;
            hipLaunchKernelGGL((w4a16_gemm_sk_fixup_kernel<TM, TN, false, false, false, false>), dim3(p.tiles_m * p.tiles_n * TM * WAVES),
                               dim3(64), 0, stream, p, grid);
            return hipGetLastError();
        }
        // tile_rows x tile_cols as sk_tile_shape chooses them for a plain product
        template <int QG>
        hipError_t launch_tiles_q(hipStream_t stream, const SkGemmParams& p, int grid, int tile_rows, int tile_cols)
        {
            if (tile_cols == 128)
                return tile_rows == 256   ? launch_instance_q<8, 1, QG>(stream, p, grid)
                       : tile_rows == 128 ? launch_instance_q<4, 1, QG>(stream, p, grid)
                       : tile_rows == 64  ? launch_instance_q<2, 1, QG>(stream, p, grid)
                                          : hipErrorInvalidValue;
            return tile_rows == 256   ? launch_instance_q<8, 2, QG>(stream, p, grid)
                   : tile_rows == 128 ? launch_instance_q<4, 2, QG>(stream, p, grid)
                   : tile_rows == 32  ? launch_instance_q<1, 2, QG>(stream, p, grid)
                                      : hipErrorInvalidValue;
        }
    } // namespace gemm_sk

    // groups of 32 / 64 / 128 with p.zps or p.zp (w4a16_gemm_sk_q5.hip ... _q7.hip)
    hipError_t launch_gemm_sk_q5(hipStream_t stream, const SkGemmParams& p, int grid, int tile_rows, int tile_cols);
    hipError_t launch_gemm_sk_q6(hipStream_t stream, const SkGemmParams& p, int grid, int tile_rows, int tile_cols);
    hipError_t launch_gemm_sk_q7(hipStream_t stream, const SkGemmParams& p, int grid, int tile_rows, int tile_cols);
    // one per tile height (w4a16_gemm_sk_32.hip ... _256.hip); narrow: 128 x 128 tiles, plain product, bias, residual, RMSNorm
    hipError_t launch_gemm_sk_64_narrow(hipStream_t stream, const SkGemmParams& p, int grid);
    hipError_t launch_gemm_sk_128_narrow(hipStream_t stream, const SkGemmParams& p, int grid);
    hipError_t launch_gemm_sk_256_narrow(hipStream_t stream, const SkGemmParams& p, int grid);
    hipError_t launch_gemm_sk_32(hipStream_t stream, const SkGemmParams& p, int grid, bool gate);
    hipError_t launch_gemm_sk_64(hipStream_t stream, const SkGemmParams& p, int grid, bool gate);
    hipError_t launch_gemm_sk_128(hipStream_t stream, const SkGemmParams& p, int grid, bool gate);
    hipError_t launch_gemm_sk_256(hipStream_t stream, const SkGemmParams& p, int grid, bool gate);
} // namespace nnf
