// fp16 x int4 (g128) GEMV for a single activation row (M = 1) on gfx950:  y[N] = ((Wq - zp) * S) . a
//
// With one activation row there is nothing for the matrix cores to amortise, and the kernel that is
// closest to "just read the weights once" wins.  This one is built like a streaming read:
//   * a wavefront works on whole weight rows (for long rows: on a fixed K segment of them, 2..8 wavefronts
//     sharing a row): each wavefront-wide load takes 1 KiB of one row, in memory order, so the weight
//     matrix is read as long sequential runs;
//   * the loads go global -> LDS without passing through registers (global_load_lds_dwordx4) into a
//     private ring of D rows per wavefront, D rows ahead of their use, and are waited for with explicit
//     s_waitcnt counts; no register is held by data in flight;
//   * a workgroup owns a contiguous run of rows; its wavefronts take the next row from a counter in LDS
//     whenever they have room for one.  (The hardware issues the oldest wavefront first: with a fixed
//     split the youngest wavefront of a CU finishes its rows 20 % later than the oldest, and decides.)
//     There is no barrier between the prologue and the final flush;
//   * the group scales of all the workgroup's rows (a contiguous block of S) are fetched into LDS in the
//     prologue, so that a row can go to any wavefront;
//   * a lane always meets the same 32 (x SEG) activations, whatever the row: they live in registers for
//     the whole kernel, already paired for the nibble trick below, and nothing but the
//     weights is read per row (plus two bytes of scale per lane and load, from LDS);
//   * nibbles become fp16 with one v_and_or_b32 per pair: (q | 0x6400) = 1024 + q (0x6400 is 1024 with an ulp
//     of 1) and, for a nibble four bits up, (16 q | 0x5400) = 64 + q (0x5400 is 64 with an ulp of 1/16): both
//     exact, whatever the activations are; the dot products run on v_dot2_f32_f16 (fp32 accumulate) against
//     (a_even, a_odd), and the constant part  (1024 + zp) sum a_even + (64 + zp) sum a_odd  of a lane's sum is
//     the same for every row: it is computed once and used as the negative initial accumulator;
//   * the 32 weights of a lane and load share one group scale (a group of 128 is 4 lanes); the lane's
//     partial sum is multiplied by it in fp32, the 64 lanes are added with DPP row rotations, and the
//     row's result is parked in LDS; outputs are written once, after the last row.
// Every instruction of a wavefront costs the CU the same issue time whether sixteen wavefronts share the rows
// or eight: eight pay the per-wavefront parts (address set-up, activations into registers, flush) half as often.
#include "w4a16_gemv_rows.h"

namespace nnf
{

    // The plain kernel keeps its arguments within the sixteen dwords that are preloaded into scalar registers at launch
    // (measured with FETCH_SIZE / WRITE_SIZE: with the fused kernel's longer argument list the same code wrote its
    // outputs as 16-byte pieces, 8 x the bytes, and fetched 3 % more).
    template <int SEG, int D, int WAVES>
    __global__ __launch_bounds__(WAVES * 64) void w4a16_gemv_rows_kernel(const half_t* __restrict__ A,
                                                                         const uint8_t* __restrict__ Wq,
                                                                         const half_t* __restrict__ S,
                                                                         half_t* __restrict__ Y, int N, int K,
                                                                         int rows_q, int rows_r, int pack)
    {
        gemv_rows_body<SEG, D, WAVES, 0>(A, Wq, S, Y, N, K, rows_q, rows_r, pack, GemvFusionArgs{nullptr, nullptr, nullptr, nullptr, 0.f});
    }
    // (the RMSNorm weight's pointer, which the kernel needs for its first loads, as an argument of its own ahead of `f`,
    // and K in the top byte of `pack`, in units of 256: fourteen dwords of scalar arguments arrive in registers with the
    // wavefront, a structure passed by value does not)
    template <int SEG, int D, int WAVES, int EPI>
    __global__ __launch_bounds__(WAVES * 64) void w4a16_gemv_rows_fused_kernel(const half_t* __restrict__ A,
                                                                               const uint8_t* __restrict__ Wq,
                                                                               const half_t* __restrict__ S,
                                                                               half_t* __restrict__ Y, int N, int rows_q,
                                                                               int rows_r, int pack, const half_t* gamma,
                                                                               GemvFusionArgs f)
    {
        static_assert(EPI == 1 || EPI == 2, "the plain kernel is w4a16_gemv_rows_kernel");
        const GemvFusionArgs g = {gamma, f.rstd, f.bias, f.residual, f.rms_eps};
        gemv_rows_body<SEG, D, WAVES, EPI>(A, Wq, S, Y, N, (int)((unsigned)pack >> 24) << 8, rows_q, rows_r, pack & 0xffffff, g);
    }

    // Other block parameters (EPI 4: group size; 3: a zero point per (row, group) as well; BITS: 4 or 8).  Sixteen dwords
    // of arguments, like the plain kernel.
    template <int SEG, int D, int WAVES, int EPI, int BITS>
    __global__ __launch_bounds__(WAVES * 64) void w4a16_gemv_rows_q_kernel(const half_t* __restrict__ A,
                                                                           const uint8_t* __restrict__ Wq,
                                                                           const half_t* __restrict__ S,
                                                                           half_t* __restrict__ Y, int N, int K,
                                                                           int rows_q, int rows_r, int pack,
                                                                           const uint8_t* __restrict__ zps)
    {
        static_assert(EPI == 3 || EPI == 4, "the plain kernel is w4a16_gemv_rows_kernel");
        gemv_rows_body<SEG, D, WAVES, EPI, BITS>(A, Wq, S, Y, N, K, rows_q, rows_r, pack, GemvFusionArgs{nullptr, nullptr, nullptr, nullptr, 0.f}, zps);
    }

    namespace
    {
        using workspace::RowsPlan;

        template <int SEG, int D, int WAVES, int EPI, int BITS>
        hipError_t launch_rows_q(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int N, int K,
                                 int zp, int group_shift, const void* zps, const RowsPlan& p, int grid)
        {
            const size_t lds_total = p.lds_bytes(N, K, grid, false, group_shift, EPI == 3);
            if (lds_total > MAX_LDS_BYTES)
                return hipErrorInvalidValue;
            if (lds_total > 64 * 1024)
            {
                static LdsGrant granted;
                const hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(&w4a16_gemv_rows_q_kernel<SEG, D, WAVES, EPI, BITS>),
                                                       granted, (int)MAX_LDS_BYTES);
                if (e != hipSuccess)
                    return e;
            }
            hipLaunchKernelGGL((w4a16_gemv_rows_q_kernel<SEG, D, WAVES, EPI, BITS>), dim3(grid), dim3(WAVES * 64), lds_total, stream,
                               (const half_t*)A, (const uint8_t*)Wq, (const half_t*)S, (half_t*)Y, N, K, N / grid, N % grid,
                               zp | (p.kshift << 8) | (group_shift << 16), (const uint8_t*)zps);
            return hipGetLastError();
        }

        template <int SEG, int D, int WAVES, int EPI>
        hipError_t launch_rows(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int N, int K,
                               int zp, const RowsPlan& p, int grid, const GemvFusion& fusion)
        {
            const size_t lds_total = p.lds_bytes(N, K, grid, EPI == 2);
            const GemvFusionArgs f = {(const half_t*)fusion.gamma, fusion.rstd, (const half_t*)fusion.bias,
                                      (const half_t*)fusion.residual, fusion.rms_eps};
            if (lds_total > MAX_LDS_BYTES)
                return hipErrorInvalidValue;
            const void* kernel;
            if constexpr (EPI == 0)
                kernel = reinterpret_cast<const void*>(&w4a16_gemv_rows_kernel<SEG, D, WAVES>);
            else
                kernel = reinterpret_cast<const void*>(&w4a16_gemv_rows_fused_kernel<SEG, D, WAVES, EPI>);
            if (lds_total > 64 * 1024)
            {
                static LdsGrant granted;
                const hipError_t e = allow_dynamic_lds(kernel, granted, (int)MAX_LDS_BYTES);
                if (e != hipSuccess)
                    return e;
            }
            if constexpr (EPI == 0)
                hipLaunchKernelGGL((w4a16_gemv_rows_kernel<SEG, D, WAVES>), dim3(grid), dim3(WAVES * 64), lds_total, stream,
                                   (const half_t*)A, (const uint8_t*)Wq, (const half_t*)S, (half_t*)Y, N, K, N / grid, N % grid,
                                   zp | (p.kshift << 8));
            else
                hipLaunchKernelGGL((w4a16_gemv_rows_fused_kernel<SEG, D, WAVES, EPI>), dim3(grid), dim3(WAVES * 64), lds_total,
                                   stream, (const half_t*)A, (const uint8_t*)Wq, (const half_t*)S, (half_t*)Y, N, N / grid,
                                   N % grid, zp | (p.kshift << 8) | ((K >> 8) << 24), f.gamma, f); // (K: a multiple of 256 up to 16384)
            return hipGetLastError();
        }
    } // namespace

    bool w4a16_gemv_rows_supported(int M, int N, int K, int num_cu, bool gate)
    {
        return workspace::plan_w4a16_rows(M, N, K, num_cu, 0, gate).seg != 0;
    }

    hipError_t launch_w4a16_gemv_rows(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int N,
                                      int K, int zp, int num_cu, const GemvFusion& fusion)
    {
        const RowsPlan p = workspace::plan_w4a16_rows(1, N, K, num_cu, 0, fusion.gate);
        const int grid = workspace::rows_grid(N, num_cu);
        if (fusion.gate && (fusion.bias || fusion.residual))
            return hipErrorInvalidValue;
        const int epi = fusion.gate ? 2 : fusion.any() ? 1 : 0;
        switch (p.seg * 10 + p.depth)
        {
#define NNF_ROWS_CASE(SEG, D)                                                                                          \
    case SEG * 10 + D:                                                                                                 \
        return epi == 0   ? launch_rows<SEG, D, workspace::ROWS_WAVES, 0>(stream, A, Wq, S, Y, N, K, zp, p, grid, fusion)  \
               : epi == 1 ? launch_rows<SEG, D, workspace::ROWS_WAVES, 1>(stream, A, Wq, S, Y, N, K, zp, p, grid, fusion)  \
                          : launch_rows<SEG, D, workspace::ROWS_WAVES, 2>(stream, A, Wq, S, Y, N, K, zp, p, grid, fusion);
            NNF_ROWS_CASE(1, 1)
            NNF_ROWS_CASE(1, 2)
            NNF_ROWS_CASE(1, 3)
            NNF_ROWS_CASE(1, 4)
            NNF_ROWS_CASE(2, 1)
            NNF_ROWS_CASE(2, 2)
            NNF_ROWS_CASE(2, 3)
            NNF_ROWS_CASE(2, 4)
            NNF_ROWS_CASE(3, 1)
            NNF_ROWS_CASE(3, 2)
#undef NNF_ROWS_CASE
        default: return hipErrorInvalidValue;
        }
    }

    bool w4a16_gemv_rows_q_supported(int M, int N, int K, int group_shift, bool zero_points, int num_cu, int bits)
    {
        return workspace::plan_w4a16_rows(M, N, K, num_cu, 0, false, group_shift, zero_points, bits).seg != 0;
    }

    hipError_t launch_w4a16_gemv_rows_q(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int N,
                                        int K, int group_shift, int zp, const void* zero_points, int num_cu, int bits)
    {
        const RowsPlan p = workspace::plan_w4a16_rows(1, N, K, num_cu, 0, false, group_shift, zero_points != nullptr, bits);
        const int grid = workspace::rows_grid(N, num_cu);
        switch (p.seg * 10 + p.depth)
        {
#define NNF_ROWS_Q(SEG, D, EPI, BITS, ZPS)                                                                             \
    launch_rows_q<SEG, D, workspace::ROWS_WAVES, EPI, BITS>(stream, A, Wq, S, Y, N, K, zp, group_shift, ZPS, p, grid)
#define NNF_ROWS_CASE(SEG, D)                                                                                          \
    case SEG * 10 + D:                                                                                                 \
        if (bits == 8)                                                                                                 \
            return zero_points ? NNF_ROWS_Q(SEG, D, 3, 8, zero_points) : NNF_ROWS_Q(SEG, D, 4, 8, nullptr);            \
        return zero_points ? NNF_ROWS_Q(SEG, D, 3, 4, zero_points) : NNF_ROWS_Q(SEG, D, 4, 4, nullptr);
            NNF_ROWS_CASE(1, 1)
            NNF_ROWS_CASE(1, 2)
            NNF_ROWS_CASE(1, 3)
            NNF_ROWS_CASE(1, 4)
            NNF_ROWS_CASE(2, 1)
            NNF_ROWS_CASE(2, 2)
            NNF_ROWS_CASE(2, 3)
            NNF_ROWS_CASE(2, 4)
            NNF_ROWS_CASE(3, 1)
            NNF_ROWS_CASE(3, 2)
#undef NNF_ROWS_CASE
#undef NNF_ROWS_Q
        default: return hipErrorInvalidValue;
        }
    }
} // namespace nnf
