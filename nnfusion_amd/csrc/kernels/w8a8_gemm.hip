// W8A8: int8 x int8 -> int32 GEMM on the gfx950 int8 matrix cores, exact accumulators.
//
//   acc[M,N] = A[M,K] . W[N,K]^T  (int32, bit exact);  Y = fp16((float)acc * s_tok[m] * s_ch[n])
//
// This file: the M <= 16 kernel and the dispatcher (larger M: w8a8_gemm_dl.hip).
//
// M <= 16: bandwidth-bound skinny kernel on v_mfma_i32_16x16x64_i8: a wavefront owns 16 weight rows
// and a K-slice, one 128-bit load per lane brings 16 rows x 64 B, the K-slices of a workgroup meet
// in LDS (integer adds: the result does not depend on the order).
#include "nnf_device.h"
#include "nnf_launch.h"

#include "../nnf_workspace.h"

#include <algorithm>

namespace nnf
{
    struct W8A8Params
    {
        const int8_t* A;
        const int8_t* W;
        const float* s_tok;
        const float* s_ch;
        half_t* Y;
        int32_t* acc;
        int M, N, K;
    };

    template <int CPS, bool RAW_ACC>
    __global__ __launch_bounds__(1024) void w8a8_skinny_kernel(W8A8Params p, int n_tiles)
    {
        extern __shared__ uintx4 lds[];
        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = tid >> 6;
        const int KS = blockDim.x >> 6;
        const int col = lane & 15;
        const int kq = lane >> 4;
        const int M = p.M, N = p.N, K = p.K;
        const int C = K >> 6; // 64-byte chunks per row
        const int n_units = C * 4 * M;
        int32_t* red = reinterpret_cast<int32_t*>(lds + n_units);
        int32_t* outb = red + 2 * KS * 256;
        const int chunk0 = wave * CPS;

        auto load_tile = [&](int tile, uintx4* w) {
            int n = min(tile * 16 + col, N - 1);
            const int8_t* wrow = p.W + (size_t)n * K + kq * 16;
#pragma unroll
            for (int c = 0; c < CPS; ++c)
                w[c] = *reinterpret_cast<const uintx4*>(wrow + (size_t)min(chunk0 + c, C - 1) * 64);
        };

        uintx4 w0[CPS], w1[CPS];
        int tile = blockIdx.x;
        load_tile(tile, w0);

        for (int u = tid; u < n_units; u += blockDim.x)
        {
            int m = u % M;
            int rest = u / M; // c*4 + kq
            lds[u] = *reinterpret_cast<const uintx4*>(p.A + (size_t)m * K + (size_t)rest * 16);
        }
        __syncthreads();

        const int m_rd = min(col, M - 1);
        int a_unit[CPS];
        int valid[CPS];
#pragma unroll
        for (int c = 0; c < CPS; ++c)
        {
            a_unit[c] = (min(chunk0 + c, C - 1) * 4 + kq) * M + m_rd;
            valid[c] = (chunk0 + c < C) ? -1 : 0;
        }

        int buf = 0, local_tile = 0;
        auto compute_store = [&](const uintx4* wt) {
            intx4 acc = {0, 0, 0, 0};
#pragma unroll
            for (int c = 0; c < CPS; ++c)
            {
                uintx4 a = lds[a_unit[c]];
                uintx4 w = wt[c];
                // chunks past the end of K contribute nothing
                w.x &= valid[c];
                w.y &= valid[c];
                w.z &= valid[c];
                w.w &= valid[c];
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(intx4, a), __builtin_bit_cast(intx4, w),
                                                            acc, 0, 0, 0);
            }
            int32_t* rp = red + ((buf * KS + wave) * 16 + kq * 4) * 16 + col;
            rp[0] = acc.x;
            rp[16] = acc.y;
            rp[32] = acc.z;
            rp[48] = acc.w;
            lds_barrier();
            if (tid < M * 16)
            {
                const int32_t* rr = red + buf * KS * 256 + tid;
                int32_t v = 0;
                for (int w = 0; w < KS; ++w)
                    v += rr[w * 256];
                outb[local_tile * M * 16 + tid] = v;
            }
            buf ^= 1;
            ++local_tile;
        };

        const int stride = gridDim.x;
        const int my_tiles = (n_tiles - tile + stride - 1) / stride;
        const int last_tile = tile + (my_tiles - 1) * stride;
        for (int it = 0; it < (my_tiles >> 1); ++it)
        {
            load_tile(tile + stride, w1);
            __builtin_amdgcn_sched_barrier(0);
            compute_store(w0);
            load_tile(min(tile + 2 * stride, last_tile), w0);
            __builtin_amdgcn_sched_barrier(0);
            compute_store(w1);
            tile += 2 * stride;
        }
        if (my_tiles & 1)
            compute_store(w0);

        __syncthreads();
        const int per_tile = M * 16;
        for (int i = tid; i < local_tile * per_tile; i += blockDim.x)
        {
            int lt = i / per_tile;
            int r = i - lt * per_tile;
            int m = r >> 4;
            int n = ((int)blockIdx.x + lt * stride) * 16 + (r & 15);
            if (n < N)
            {
                if (RAW_ACC)
                {
                    p.acc[(size_t)m * N + n] = outb[i];
                }
                else
                {
                    float t = (float)outb[i] * p.s_tok[m];
                    p.Y[(size_t)m * N + n] = f32_to_f16_two_step(t * p.s_ch[n]);
                }
            }
        }
    }

    namespace
    {
        using Q8SkinnyPlan = workspace::Q8SkinnyPlan;
        Q8SkinnyPlan plan_q8_skinny(int M, int K) { return workspace::plan_w8a8_skinny(M, K); }

        template <int CPS, bool RAW_ACC>
        hipError_t launch_q8_skinny_cps(hipStream_t stream, const W8A8Params& p, const Q8SkinnyPlan& pl, int num_cu)
        {
            const int n_tiles = (p.N + 15) / 16;
            int grid = std::min(n_tiles, num_cu * (pl.ks >= 8 ? 1 : 2));
            int tiles_per_wg = (n_tiles + grid - 1) / grid;
            size_t lds_total = pl.lds + (size_t)tiles_per_wg * p.M * 16 * 4;
            while (lds_total > MAX_LDS_BYTES && grid < n_tiles)
            {
                grid = std::min(n_tiles, grid * 2);
                tiles_per_wg = (n_tiles + grid - 1) / grid;
                lds_total = pl.lds + (size_t)tiles_per_wg * p.M * 16 * 4;
            }
            if (lds_total > MAX_LDS_BYTES)
                return hipErrorInvalidValue;
            if (lds_total > 64 * 1024)
            {
                hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&w8a8_skinny_kernel<CPS, RAW_ACC>),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_total);
                if (e != hipSuccess)
                    return e;
            }
            hipLaunchKernelGGL((w8a8_skinny_kernel<CPS, RAW_ACC>), dim3(grid), dim3(pl.ks * 64), lds_total, stream, p,
                               n_tiles);
            return hipGetLastError();
        }

        template <bool RAW_ACC>
        hipError_t launch_q8_skinny(hipStream_t stream, const W8A8Params& p, int num_cu)
        {
            Q8SkinnyPlan pl = plan_q8_skinny(p.M, p.K);
            switch (pl.cps)
            {
            case 1: return launch_q8_skinny_cps<1, RAW_ACC>(stream, p, pl, num_cu);
            case 2: return launch_q8_skinny_cps<2, RAW_ACC>(stream, p, pl, num_cu);
            case 4: return launch_q8_skinny_cps<4, RAW_ACC>(stream, p, pl, num_cu);
            case 8: return launch_q8_skinny_cps<8, RAW_ACC>(stream, p, pl, num_cu);
            case 16: return launch_q8_skinny_cps<16, RAW_ACC>(stream, p, pl, num_cu);
            default: return hipErrorInvalidValue;
            }
        }
    } // namespace

    bool w8a8_skinny_supported(int M, int K) { return workspace::w8a8_skinny_fits(M, K); }

    hipError_t launch_w8a8(hipStream_t stream, const void* A, const void* s_tok, const void* W, const void* s_ch,
                           void* Y, void* acc, int M, int N, int K, int num_cu, void* partial_ws)
    {
        W8A8Params p;
        p.A = (const int8_t*)A;
        p.W = (const int8_t*)W;
        p.s_tok = (const float*)s_tok;
        p.s_ch = (const float*)s_ch;
        p.Y = (half_t*)Y;
        p.acc = (int32_t*)acc;
        p.M = M;
        p.N = N;
        p.K = K;
        const bool raw = acc != nullptr;
        const bool skinny = g_tuning.force_path != 3 && w8a8_skinny_supported(M, K);
        if (skinny)
            return raw ? launch_q8_skinny<true>(stream, p, num_cu) : launch_q8_skinny<false>(stream, p, num_cu);
        return launch_w8a8_gemm(stream, A, s_tok, W, s_ch, Y, acc, M, N, K, partial_ws);
    }
} // namespace nnf
