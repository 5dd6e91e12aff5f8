// fp16 x int4 (g128) products beyond one activation row: the dispatcher between the row-streaming /
// split-K GEMV kernels (up to 40 rows) and the tile GEMM (w4a16_gemm_sk.h), the RMSNorm pre-passes, the
// reduction pass behind the GEMV kernels that run over ranges of K, and their element-wise epilogues.
//
//   Y[M,N] = epilogue( prologue(A)[M,K] . ((Wq - zp) * S)^T )
//
//   * prologue: RMSNorm.  The tile GEMM folds it in (a pre-pass computes rstd[m] only); the GEMV
//     kernels read normalised activations, fp16(x * rsqrt(mean(x^2) + eps) * gamma) written to scratch
//     memory by a pre-pass (the tensor of the unfused graph, at most 40 rows of it).
//   * epilogues: bias, residual add, SiLU(gate) * up with the gate and up projections as two halves of
//     the N tile -- in the tile GEMM's epilogue, in the reduction pass, or in an element-wise kernel
//     behind a GEMV kernel.
//   * tile height and split of the work over the CUs follow nnf::workspace::plan_w4a16_sk.
#include "w4a16_gemm_sk_launch.h"

#include "../nnf_workspace.h"

#include <algorithm>

namespace nnf
{
    // what the reduction pass behind the GEMV kernels that run over ranges of K needs to know
    struct GemmParams
    {
        half_t* Y;
        int M, N;               // N = output columns
        int ldy;                // row stride of Y
        const half_t* bias;     // BIAS: [N]
        const half_t* residual; // RESID: [M, ldy]
        const float* rstd;      // [M] or null: the sums of row m are scaled by rstd[m] (RMSNorm prologue)
        float* partial;         // [splits][M][ld_partial] fp32
        int splits;             // number of K ranges
        int ld_partial;         // N, or 2 N with GATE (gate columns, then up columns)
    };

    // one row per workgroup of four wavefronts: Xn[m, :] = fp16( x * rsqrt(mean_k(x^2) + eps) * gamma ).
    // The row is read once: a thread keeps its 16-byte units in registers between the two passes (up to K = 16384;
    // the units beyond that are read again).
    __global__ __launch_bounds__(256) void rms_norm_kernel(const half_t* __restrict__ X, const half_t* __restrict__ gamma,
                                                           half_t* __restrict__ Xn, int M, int K, float eps)
    {
        constexpr int KEEP = 8; // units per thread kept in registers
        __shared__ float part[4];
        const int tid = threadIdx.x;
        const int m = blockIdx.x;
        const int units = K >> 3;
        const uintx4* row = reinterpret_cast<const uintx4*>(X + (size_t)m * K);
        uintx4 kept[KEEP];
        float ss = 0.f;
        auto sq = [&](const uintx4& v) {
            const uint32_t vv[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int j = 0; j < 4; ++j)
            {
                half2_t h = as_half2(vv[j]);
                ss += (float)h.x * (float)h.x + (float)h.y * (float)h.y;
            }
        };
#pragma unroll
        for (int e = 0; e < KEEP; ++e)
        {
            const int i = tid + e * 256;
            kept[e] = i < units ? row[i] : uintx4{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int e = 0; e < KEEP; ++e)
            sq(kept[e]);
        for (int i = tid + KEEP * 256; i < units; i += 256)
            sq(row[i]);
        ss = wave_sum(ss);
        if ((tid & 63) == 0)
            part[tid >> 6] = ss;
        __syncthreads();
        ss = (part[0] + part[1]) + (part[2] + part[3]);
        const float rstd = 1.0f / __builtin_sqrtf(ss / (float)K + eps);
        const uintx4* grow = reinterpret_cast<const uintx4*>(gamma);
        uintx4* out = reinterpret_cast<uintx4*>(Xn + (size_t)m * K);
        auto norm = [&](const uintx4& v, const uintx4& g) {
            const uint32_t vv[4] = {v.x, v.y, v.z, v.w};
            const uint32_t gg[4] = {g.x, g.y, g.z, g.w};
            uint32_t oo[4];
#pragma unroll
            for (int j = 0; j < 4; ++j)
            {
                half2_t x = as_half2(vv[j]), w = as_half2(gg[j]), r;
                r.x = (half_t)((float)x.x * rstd * (float)w.x);
                r.y = (half_t)((float)x.y * rstd * (float)w.y);
                oo[j] = as_u32(r);
            }
            return uintx4{oo[0], oo[1], oo[2], oo[3]};
        };
#pragma unroll
        for (int e = 0; e < KEEP; ++e)
        {
            const int i = tid + e * 256;
            if (i < units)
                out[i] = norm(kept[e], grow[i]);
        }
        for (int i = tid + KEEP * 256; i < units; i += 256)
            out[i] = norm(row[i], grow[i]);
    }

    // RMSNorm for the tile GEMM, which never materialises the normalised activations: only
    // rstd[m] = rsqrt(mean_k(x[m,k]^2) + eps) is computed here (one workgroup of four wavefronts per row; same
    // summation order as rms_norm_kernel); gamma joins the weights inside the GEMM.
    __global__ __launch_bounds__(256) void rms_rstd_kernel(const half_t* __restrict__ X, float* __restrict__ rstd, int M, int K,
                                                           float eps)
    {
        __shared__ float part[4];
        const int tid = threadIdx.x;
        const int m = blockIdx.x;
        const int units = K >> 3;
        const uintx4* row = reinterpret_cast<const uintx4*>(X + (size_t)m * K);
        float ss = 0.f;
        for (int i = tid; i < units; i += 256)
        {
            const uintx4 v = row[i];
            const uint32_t vv[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int j = 0; j < 4; ++j)
            {
                const half2_t hh = as_half2(vv[j]);
                ss += (float)hh.x * (float)hh.x + (float)hh.y * (float)hh.y;
            }
        }
        ss = wave_sum(ss);
        if ((tid & 63) == 0)
            part[tid >> 6] = ss;
        __syncthreads();
        if (tid == 0)
            rstd[m] = 1.0f / __builtin_sqrtf(((part[0] + part[1]) + (part[2] + part[3])) / (float)K + eps);
    }

    // Y[m, n] = epilogue( sum_s partial[s][m][n] ); four consecutive columns per thread.
    // GATE: partial columns [0, N) are the gate, [N, 2N) the up projection.  rstd (or null): the sums of row m times
    // rstd[m] first (the kernel that wrote them multiplied the RMSNorm weight onto the activations).
    template <bool GATE, bool BIAS, bool RESID>
    __global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ partial, int splits, int M,
                                                                int N, int ld_partial, const half_t* __restrict__ bias,
                                                                const half_t* __restrict__ residual, half_t* __restrict__ Y,
                                                                int ldy, const float* __restrict__ rstd)
    {
        // grid: x over groups of four columns, y = row
        const int quads = (N + 3) >> 2;
        const int q = (int)blockIdx.x * 256 + (int)threadIdx.x;
        if (q >= quads)
            return;
        const int m = blockIdx.y;
        const int n = q * 4;
        const size_t plane = (size_t)M * ld_partial;
        const float* src = partial + (size_t)m * ld_partial + n;
        // ld_partial and n are multiples of 4 when N is; otherwise fall back to scalar accesses
        const bool vec = ((ld_partial | N) & 3) == 0;
        float a[4] = {0.f, 0.f, 0.f, 0.f}, u[4] = {0.f, 0.f, 0.f, 0.f};
        // (the ranges are added in order, whatever the unrolling: the sums do not depend on it)
#pragma unroll 4
        for (int s = 0; s < splits; ++s)
        {
            const float* ps = src + (size_t)s * plane;
            if (vec)
            {
                floatx4 v = *reinterpret_cast<const floatx4*>(ps);
                a[0] += v.x, a[1] += v.y, a[2] += v.z, a[3] += v.w;
                if (GATE)
                {
                    floatx4 w = *reinterpret_cast<const floatx4*>(ps + N);
                    u[0] += w.x, u[1] += w.y, u[2] += w.z, u[3] += w.w;
                }
            }
            else
            {
                for (int j = 0; j < 4; ++j)
                    if (n + j < N)
                    {
                        a[j] += ps[j];
                        if (GATE)
                            u[j] += ps[N + j];
                    }
            }
        }
        const float rs = rstd ? rstd[m] : 1.0f;
        half_t out[4];
        for (int j = 0; j < 4; ++j)
        {
            if (n + j >= N)
                break;
            float v = f32_product(a[j], rs);
            if (GATE)
            {
                float g = (float)(half_t)v;
                float up = (float)(half_t)f32_product(u[j], rs);
                v = g * (1.0f / (1.0f + __expf(-g))) * up;
            }
            if (BIAS)
                v = (float)(half_t)v + (float)bias[n + j];
            if (RESID)
                v = (float)(half_t)v + (float)residual[(size_t)m * ldy + n + j];
            out[j] = (half_t)v;
        }
        half_t* dst = Y + (size_t)m * ldy + n;
        if (vec && (ldy & 3) == 0)
        {
            *reinterpret_cast<uintx2*>(dst) = uintx2{as_u32(half2_t{out[0], out[1]}), as_u32(half2_t{out[2], out[3]})};
        }
        else
        {
            for (int j = 0; j < 4 && n + j < N; ++j)
                dst[j] = out[j];
        }
    }

    // Epilogues for the M <= 16 path, whose GEMV kernel writes plain fp16 products.
    // T [M, 2N] = (gate | up) products  ->  Y [M, N] = SiLU(gate) * up
    __global__ __launch_bounds__(256) void skinny_silu_gate_kernel(const half_t* __restrict__ T, half_t* __restrict__ Y,
                                                                   int M, int N)
    {
        const int i = blockIdx.x * 256 + threadIdx.x;
        if (i >= M * N)
            return;
        const int m = i / N, n = i - m * N;
        const float g = (float)T[(size_t)m * 2 * N + n];
        const float u = (float)T[(size_t)m * 2 * N + N + n];
        Y[i] = (half_t)(g * (1.0f / (1.0f + __expf(-g))) * u);
    }
    // Y [M, N] = T [M, N] + bias [N] (rounded to fp16), then + residual [M, N]; T may be Y, residual may be Y
    __global__ __launch_bounds__(256) void skinny_bias_residual_kernel(const half_t* T, half_t* Y, const half_t* bias,
                                                                       const half_t* residual, int M, int N)
    {
        const int i = blockIdx.x * 256 + threadIdx.x;
        if (i >= M * N)
            return;
        float v = (float)T[i];
        if (bias)
            v = (float)(half_t)(v + (float)bias[i % N]);
        if (residual)
            v = v + (float)residual[i];
        Y[i] = (half_t)v;
    }

    namespace
    {
        template <bool GATE, bool BIAS, bool RESID>
        hipError_t launch_reduce(hipStream_t stream, const GemmParams& p)
        {
            const int quads = (p.N + 3) >> 2;
            hipLaunchKernelGGL((splitk_reduce_kernel<GATE, BIAS, RESID>), dim3((unsigned)((quads + 255) / 256), (unsigned)p.M), dim3(256), 0,
                               stream, (const float*)p.partial, p.splits, p.M, p.N, p.ld_partial, p.bias, p.residual, p.Y,
                               p.ldy, p.rstd);
            return hipGetLastError();
        }

        hipError_t launch_reduce_any(hipStream_t stream, const GemmParams& p, bool gate, bool hb, bool hr)
        {
            if (gate)
                return launch_reduce<true, false, false>(stream, p);
            if (hb && hr)
                return launch_reduce<false, true, true>(stream, p);
            if (hb)
                return launch_reduce<false, true, false>(stream, p);
            if (hr)
                return launch_reduce<false, false, true>(stream, p);
            return launch_reduce<false, false, false>(stream, p);
        }
    } // namespace

    namespace
    {
        // one launch where the caller gave enough zeroed synchronisation words for the plan's tiles, else two
        // (and only where every workgroup of the grid has a CU: workgroups that wait for one another inside the launch
        // must all be running -- a forced plan with more workgroups than CUs would spin to its limit, some milliseconds)
        void set_sync(SkGemmParams& p, const workspace::SkPlan& plan, const LaunchChoice& choice, int num_cu)
        {
            p.partial_bytes = plan.bytes();
            p.trace = nullptr;
            // (the one-launch form addresses the parked tiles with 32-bit byte offsets)
            const bool one_launch = plan.slots && plan.grid <= num_cu && choice.sync_flags && choice.sync_bytes >= plan.sync_bytes() &&
                                    plan.bytes() < ((size_t)1 << 32);
            p.sync = one_launch ? (uint32_t*)choice.sync_flags + 2 : nullptr; // (the first two words: rstd_sync)
            p.spin_limit = choice.spin_limit > 0 ? choice.spin_limit : choice.spin_limit < 0 ? 0 : DEFAULT_SPIN_LIMIT;
            p.rstd_out = nullptr;
            p.rstd_sync = nullptr;
            p.rms_eps = 0.f;
        }
        // RMSNorm's rstd[] can be left to the GEMM launch itself: the caller gave (zeroed) synchronisation words
        bool rstd_inside_tile_gemm(const workspace::SkPlan& plan, const LaunchChoice& choice, int num_cu)
        {
            return plan.grid <= num_cu && choice.sync_flags && choice.sync_bytes >= plan.sync_bytes(true);
        }
    } // namespace

    hipError_t launch_w4a16_gemm(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M,
                                 int N, int K, int zp, const void* rms_gamma, float rms_eps, const void* bias,
                                 const void* residual, int act, void* rms_ws, void* partial_ws, int num_cu,
                                 const LaunchChoice& choice)
    {
        using workspace::W4A16Route;
        const bool rms = rms_gamma != nullptr, hb = bias != nullptr, hr = residual != nullptr, gate = act == 1;
        // the combinations the fused entry points use; anything else is composed by the caller
        if (gate && (hb || hr))
            return hipErrorInvalidValue;
        const int n_rows = gate ? 2 * N : N; // weight rows
        const W4A16Route route =
            workspace::route_w4a16(M, N, K, gate, rms, hr && residual == Y, num_cu, choice.path, choice.tile_rows, choice.k_parts, choice.tile_cols);
        if (route.kind == W4A16Route::NONE || (route.partial_bytes > 0 && !partial_ws) || (route.rms_bytes > 0 && !rms_ws))
            return hipErrorInvalidValue;
        // ---- RMSNorm pre-pass: rstd[m] for the kernels that multiply the weight in themselves, the normalised
        // activations for the MFMA GEMV kernel -------------------------------------------------------------------
        // (the row-streaming kernels add up the squares of the activations they hold themselves: no pre-pass; the form
        // with a run-time K keeps it)
        const bool normalised_copy = route.kind == W4A16Route::SKINNY || route.kind == W4A16Route::SKINNY_SPLIT;
        const bool rstd_in_tile_gemm = rms && route.kind == W4A16Route::TILE && rstd_inside_tile_gemm(route.plan, choice, num_cu);
        const bool rstd_in_kernel = route.kind == W4A16Route::ROWS ||
                                    (route.kind == W4A16Route::MROWS && workspace::w4a16_mrows_fixed_k(M, K)) || rstd_in_tile_gemm;
        if (rms && !rstd_in_kernel)
        {
            if (normalised_copy)
            {
                hipLaunchKernelGGL(rms_norm_kernel, dim3(M), dim3(256), 0, stream, (const half_t*)A, (const half_t*)rms_gamma,
                                   (half_t*)rms_ws, M, K, rms_eps);
                A = rms_ws;
            }
            else
                hipLaunchKernelGGL(rms_rstd_kernel, dim3(M), dim3(256), 0, stream, (const half_t*)A, (float*)rms_ws, M, K, rms_eps);
            const hipError_t e = hipGetLastError();
            if (e != hipSuccess)
                return e;
        }
        const float* rstd = (rms && !normalised_copy && !rstd_in_kernel) ? (const float*)rms_ws : nullptr;
        // ---- the row-streaming kernels (one row; up to 32 rows): prologue and epilogue inside the one launch ------
        if (route.kind == W4A16Route::ROWS || route.kind == W4A16Route::MROWS)
        {
            GemvFusion fusion;
            fusion.gamma = rms_gamma;
            fusion.rstd = rstd;
            fusion.rms_eps = rms_eps;
            fusion.bias = bias;
            fusion.residual = residual;
            fusion.gate = gate;
            return route.kind == W4A16Route::ROWS ? launch_w4a16_gemv_rows(stream, A, Wq, S, Y, N, K, zp, num_cu, fusion)
                                                  : launch_w4a16_mrows(stream, A, Wq, S, Y, M, N, K, zp, num_cu, fusion);
        }
        // ---- the MFMA GEMV kernel on the (normalised) activations, then a small element-wise kernel for whatever
        // epilogue is asked for ----------------------------------------------------------------------------------
        if (route.kind == W4A16Route::SKINNY)
        {
            void* y_gemv = route.via_scratch ? partial_ws : Y;
            hipError_t e = launch_w4a16_skinny(stream, A, Wq, S, y_gemv, M, n_rows, K, zp, num_cu);
            if (e != hipSuccess || (!gate && !hb && !hr))
                return e;
            const int blocks = (M * N + 255) / 256;
            if (gate)
                hipLaunchKernelGGL(skinny_silu_gate_kernel, dim3(blocks), dim3(256), 0, stream, (const half_t*)y_gemv,
                                   (half_t*)Y, M, N);
            else
                hipLaunchKernelGGL(skinny_bias_residual_kernel, dim3(blocks), dim3(256), 0, stream, (const half_t*)y_gemv,
                                   (half_t*)Y, (const half_t*)bias, (const half_t*)residual, M, N);
            return hipGetLastError();
        }
        // ---- more activations than one workgroup holds: a GEMV kernel over ranges of K, then the reduction pass
        // (which applies rstd and the epilogue) ------------------------------------------------------------------
        if (route.kind == W4A16Route::MROWS_SPLIT || route.kind == W4A16Route::SKINNY_SPLIT)
        {
            // (the row-streaming kernel adds its ranges up itself where the caller gave synchronisation words for it)
            if (route.kind == W4A16Route::MROWS_SPLIT && !gate && choice.sync_flags &&
                choice.sync_bytes >= w4a16_mrows_split_sync_bytes(num_cu) &&
                workspace::mrows_split_adds_in_launch(n_rows, route.ksplits, num_cu))
            {
                GemvFusion epilogue;
                epilogue.rstd = rstd;
                epilogue.bias = bias;
                epilogue.residual = residual;
                return launch_w4a16_mrows_split(stream, A, Wq, S, (float*)partial_ws, M, n_rows, K, zp, num_cu, rms_gamma, Y, &epilogue,
                                                (uint32_t*)choice.sync_flags);
            }
            hipError_t e = route.kind == W4A16Route::MROWS_SPLIT
                               ? launch_w4a16_mrows_split(stream, A, Wq, S, (float*)partial_ws, M, n_rows, K, zp, num_cu, rms_gamma)
                               : launch_w4a16_skinny_split(stream, A, Wq, S, (float*)partial_ws, M, n_rows, K, zp, route.ksplits,
                                                           num_cu);
            if (e != hipSuccess)
                return e;
            GemmParams p;
            p.Y = (half_t*)Y;
            p.M = M;
            p.N = N;
            p.ldy = N;
            p.bias = (const half_t*)bias;
            p.residual = (const half_t*)residual;
            p.rstd = rstd;
            p.partial = (float*)partial_ws;
            p.splits = route.ksplits;
            p.ld_partial = n_rows;
            return launch_reduce_any(stream, p, gate, hb, hr);
        }
        // ---- the tile GEMM ------------------------------------------------------------------------------------
        const workspace::SkPlan& plan = route.plan;
        if ((size_t)M * K * 2 + 8192 >= ((size_t)1 << 32) || (size_t)n_rows * (K >> 1) >= ((size_t)1 << 32))
            return hipErrorInvalidValue; // the kernel addresses its operands with 32-bit byte offsets
        SkGemmParams p;
        p.A = (const half_t*)A;
        p.Wq = (const uint8_t*)Wq;
        p.S = (const half_t*)S;
        p.Y = (half_t*)Y;
        p.M = M;
        p.N = N;
        p.K = K;
        p.zp = zp;
        p.ldy = N;
        p.up_row_offset = N; // gate rows [0,N), up rows [N,2N)
        p.bias = (const half_t*)bias;
        p.residual = (const half_t*)residual;
        p.gamma = rms ? (const half_t*)rms_gamma : nullptr;
        p.rstd = rms ? (const float*)rms_ws : nullptr;
        p.partial = plan.slots ? (float*)partial_ws : nullptr;
        p.tiles_m = plan.tiles_m;
        p.tiles_n = plan.tiles_n;
        p.supersteps = plan.supersteps;
        p.units = plan.units;
        p.zps = nullptr;
        set_sync(p, plan, choice, num_cu);
        if (rstd_in_tile_gemm)
        {
            p.rstd_out = (float*)rms_ws;
            p.rstd_sync = (uint32_t*)choice.sync_flags;
            p.rms_eps = rms_eps;
        }
        if (plan.tile_weight_rows == 128)
            return plan.tile_rows == 256 ? launch_gemm_sk_256_narrow(stream, p, plan.grid)
                   : plan.tile_rows == 128 ? launch_gemm_sk_128_narrow(stream, p, plan.grid)
                                           : launch_gemm_sk_64_narrow(stream, p, plan.grid);
        switch (plan.tile_rows)
        {
        case 256: return launch_gemm_sk_256(stream, p, plan.grid, gate);
        case 128: return launch_gemm_sk_128(stream, p, plan.grid, gate);
        case 64: return launch_gemm_sk_64(stream, p, plan.grid, gate);
        default: return launch_gemm_sk_32(stream, p, plan.grid, gate);
        }
    }

    hipError_t launch_rms_norm(hipStream_t stream, const void* X, const void* gamma, void* Xn, int M, int K, float eps)
    {
        hipLaunchKernelGGL(rms_norm_kernel, dim3(M), dim3(256), 0, stream, (const half_t*)X, (const half_t*)gamma, (half_t*)Xn, M, K, eps);
        return hipGetLastError();
    }
    hipError_t launch_silu_gate(hipStream_t stream, const void* T, void* Y, int M, int N)
    {
        hipLaunchKernelGGL(skinny_silu_gate_kernel, dim3((M * N + 255) / 256), dim3(256), 0, stream, (const half_t*)T, (half_t*)Y, M, N);
        return hipGetLastError();
    }
    hipError_t launch_bias_residual(hipStream_t stream, const void* T, void* Y, const void* bias, const void* residual, int M, int N)
    {
        hipLaunchKernelGGL(skinny_bias_residual_kernel, dim3((M * N + 255) / 256), dim3(256), 0, stream, (const half_t*)T, (half_t*)Y,
                           (const half_t*)bias, (const half_t*)residual, M, N);
        return hipGetLastError();
    }

    hipError_t launch_wna16_reduce(hipStream_t stream, const float* partial, int ranges, void* Y, int M, int N)
    {
        GemmParams p;
        p.Y = (half_t*)Y;
        p.M = M;
        p.N = N;
        p.ldy = N;
        p.bias = nullptr;
        p.residual = nullptr;
        p.rstd = nullptr;
        p.partial = const_cast<float*>(partial);
        p.splits = ranges;
        p.ld_partial = N;
        return launch_reduce_any(stream, p, false, false, false);
    }

    // ---- the tile GEMM with other block parameters ----------------------------------------------------------------------
    bool w4a16_gemm_q_supported(int M, int N, int K, int group_shift) { return workspace::w4a16_gemm_q_fits(M, N, K, group_shift); }
    hipError_t launch_w4a16_gemm_q(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M, int N,
                                   int K, int group_shift, int zp, const void* zero_points, void* partial_ws, int num_cu,
                                   const LaunchChoice& choice)
    {
        if (!w4a16_gemm_q_supported(M, N, K, group_shift))
            return hipErrorInvalidValue;
        const workspace::SkPlan plan = workspace::plan_w4a16_sk(M, N, K, false, num_cu);
        if (plan.slots && !partial_ws)
            return hipErrorInvalidValue;
        SkGemmParams p;
        p.A = (const half_t*)A;
        p.Wq = (const uint8_t*)Wq;
        p.S = (const half_t*)S;
        p.Y = (half_t*)Y;
        p.M = M;
        p.N = N;
        p.K = K;
        p.zp = zp;
        p.ldy = N;
        p.up_row_offset = N;
        p.bias = nullptr;
        p.residual = nullptr;
        p.gamma = nullptr;
        p.rstd = nullptr;
        p.partial = plan.slots ? (float*)partial_ws : nullptr;
        p.tiles_m = plan.tiles_m;
        p.tiles_n = plan.tiles_n;
        p.supersteps = plan.supersteps;
        p.units = plan.units;
        p.zps = (const uint8_t*)zero_points;
        set_sync(p, plan, choice, num_cu);
        switch (group_shift)
        {
        case 5: return launch_gemm_sk_q5(stream, p, plan.grid, plan.tile_rows, plan.tile_weight_rows);
        case 6: return launch_gemm_sk_q6(stream, p, plan.grid, plan.tile_rows, plan.tile_weight_rows);
        default: return launch_gemm_sk_q7(stream, p, plan.grid, plan.tile_rows, plan.tile_weight_rows);
        }
    }
} // namespace nnf
