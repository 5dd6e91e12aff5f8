// W8A8: int8 x int8 -> int32 GEMM on the gfx950 int8 matrix cores, exact accumulators.
//
//   acc[M,N] = A[M,K] . W[N,K]^T  (int32, bit exact);  Y = fp16((float)acc * s_tok[m] * s_ch[n])
//
// Large M: v_mfma_i32_32x32x32_i8, workgroup tile 256 x 256 x 128, four wavefronts of 128 x 128
// (4 x 4 MFMA tiles, 256 int32 accumulators per lane), register-staged double-buffered LDS with
// the same 16-byte XOR swizzle as the fp16 x int4 kernel.  Both operands are K-contiguous int8, so a
// lane's MFMA operand is 16 consecutive bytes of a row: K index in a 128-wide tile = 32*s + 16*h + e.
//
// M <= 16: bandwidth-bound skinny kernel on v_mfma_i32_16x16x64_i8: a wavefront owns 16 weight rows
// and a K-slice, one 128-bit load per lane brings 16 rows x 64 B, the K-slices of a workgroup meet
// in LDS (integer adds: the result does not depend on the order).
#include "nnf_device.h"
#include "nnf_launch.h"

#include <algorithm>

namespace nnf
{
    namespace q8
    {
        constexpr int BM = 256, BN = 256, BK = 128;
        constexpr int TILE_BYTES = BM * BK; // 32 KiB per operand
        constexpr int STAGE_BYTES = 2 * TILE_BYTES;
        constexpr int LDS_BYTES = 2 * STAGE_BYTES; // 128 KiB

        __device__ __forceinline__ int t_off(int r, int p)
        {
            return r * 128 + ((p ^ ((r >> 1) & 7)) << 4);
        }
    } // namespace q8

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

    template <bool RAW_ACC>
    __global__ __launch_bounds__(256) void w8a8_gemm_kernel(W8A8Params p)
    {
        using namespace q8;
        extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = tid >> 6;
        const int wm = wave >> 1, wn = wave & 1;
        const int l32 = lane & 31, h = lane >> 5;
        const int K = p.K;

        const int tiles_m = (p.M + BM - 1) / BM;
        const int tiles_n = (p.N + BN - 1) / BN;
        const int n_wg = tiles_m * tiles_n;
        int pid = blockIdx.x;
        {
            // contiguous run of tiles per XCD (workgroup ids are dealt round-robin to the 8 XCDs)
            const int per_xcd = (n_wg + 7) >> 3;
            const int full = n_wg - (per_xcd - 1) * 8;
            const int xcd = pid & 7, idx = pid >> 3;
            pid = (xcd < full) ? xcd * per_xcd + idx : full * per_xcd + (xcd - full) * (per_xcd - 1) + idx;
        }
        const int tm = pid % tiles_m, tn = pid / tiles_m;
        const int m0 = tm * BM, n0 = tn * BN;

        // staging: each operand tile is 2048 pieces of 16 B, 8 per thread: row = i*32 + tid/8, piece = tid%8
        const int s_p = tid & 7;
        const int8_t* a_src[8];
        const int8_t* w_src[8];
        int dst[8];
#pragma unroll
        for (int i = 0; i < 8; ++i)
        {
            int r = i * 32 + (tid >> 3);
            a_src[i] = p.A + (size_t)min(m0 + r, p.M - 1) * K + s_p * 16;
            w_src[i] = p.W + (size_t)min(n0 + r, p.N - 1) * K + s_p * 16;
            dst[i] = t_off(r, s_p);
        }
        int a_frag[4], a_swz[4], w_frag[4], w_swz[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
        {
            int ra = wm * 128 + i * 32 + l32;
            a_frag[i] = ra * 128;
            a_swz[i] = (ra >> 1) & 7;
            int rw = wn * 128 + i * 32 + l32;
            w_frag[i] = TILE_BYTES + rw * 128;
            w_swz[i] = (rw >> 1) & 7;
        }

        intx16 acc[4][4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    acc[i][j][e] = 0;

        uintx4 a_reg[8], w_reg[8];
        auto load_global = [&](int kt) {
            const int k0 = kt * BK;
#pragma unroll
            for (int i = 0; i < 8; ++i)
                a_reg[i] = *reinterpret_cast<const uintx4*>(a_src[i] + k0);
#pragma unroll
            for (int i = 0; i < 8; ++i)
                w_reg[i] = *reinterpret_cast<const uintx4*>(w_src[i] + k0);
        };
        auto store_lds = [&](int stage) {
            uint8_t* base = smem + stage * STAGE_BYTES;
#pragma unroll
            for (int i = 0; i < 8; ++i)
            {
                *reinterpret_cast<uintx4*>(base + dst[i]) = a_reg[i];
                *reinterpret_cast<uintx4*>(base + TILE_BYTES + dst[i]) = w_reg[i];
            }
        };

        const int KT = K / BK;
        load_global(0);
        store_lds(0);
        __syncthreads();
        for (int kt = 0; kt < KT; ++kt)
        {
            const int stage = kt & 1;
            if (kt + 1 < KT)
                load_global(kt + 1);
            const uint8_t* base = smem + stage * STAGE_BYTES;
#pragma unroll
            for (int s = 0; s < 4; ++s)
            {
                intx4 af[4], wf[4];
                const int pc = s * 2 + h;
#pragma unroll
                for (int i = 0; i < 4; ++i)
                {
                    af[i] = *reinterpret_cast<const intx4*>(base + a_frag[i] + ((pc ^ a_swz[i]) << 4));
                    wf[i] = *reinterpret_cast<const intx4*>(base + w_frag[i] + ((pc ^ w_swz[i]) << 4));
                }
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], wf[j], acc[i][j], 0, 0, 0);
            }
            if (kt + 1 < KT)
                store_lds(stage ^ 1);
            __syncthreads();
        }

        // D layout of a 32x32 tile: lane (col = l32, h), element e: row = 8*(e/4) + 4*h + (e%4)
#pragma unroll
        for (int j = 0; j < 4; ++j)
        {
            const int n = n0 + wn * 128 + j * 32 + l32;
            if (n >= p.N)
                continue;
            float sch = 0.f;
            if (!RAW_ACC)
                sch = p.s_ch[n];
#pragma unroll
            for (int i = 0; i < 4; ++i)
            {
#pragma unroll
                for (int e = 0; e < 16; ++e)
                {
                    const int m = m0 + wm * 128 + i * 32 + 8 * (e >> 2) + 4 * h + (e & 3);
                    if (m >= p.M)
                        continue;
                    if (RAW_ACC)
                    {
                        p.acc[(size_t)m * p.N + n] = acc[i][j][e];
                    }
                    else
                    {
                        float t = (float)acc[i][j][e] * p.s_tok[m];
                        p.Y[(size_t)m * p.N + n] = f32_to_f16_two_step(t * sch);
                    }
                }
            }
        }
    }

    // ---- skinny path ------------------------------------------------------------------------------
    // LDS: activations as 16-byte units  unit(c, kq, m) = (c*4 + kq)*M + m = a[m][c*64 + kq*16 .. +16);
    // then red[2][KS][16 m][16 n] int32 and the output parking area [tiles][M][16] int32.
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
        struct Q8SkinnyPlan
        {
            int cps = 0, ks = 0;
            size_t lds = 0;
        };

        Q8SkinnyPlan plan_q8_skinny(int M, int K)
        {
            Q8SkinnyPlan pl;
            const int C = K >> 6;
            static const int options[] = {1, 2, 4, 8, 16};
            for (int cps : options)
            {
                int ks = (C + cps - 1) / cps;
                if (ks <= 16)
                {
                    pl.cps = cps;
                    pl.ks = ks;
                    break;
                }
            }
            if (pl.cps)
                pl.lds = (size_t)C * 4 * M * 16 + (size_t)2 * pl.ks * 256 * 4;
            return pl;
        }

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

        template <bool RAW_ACC>
        hipError_t launch_q8_gemm(hipStream_t stream, const W8A8Params& p)
        {
            using namespace q8;
            const int tiles_m = (p.M + BM - 1) / BM;
            const int tiles_n = (p.N + BN - 1) / BN;
            static bool attr_set = false;
            if (!attr_set)
            {
                hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&w8a8_gemm_kernel<RAW_ACC>),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
                if (e != hipSuccess)
                    return e;
                attr_set = true;
            }
            hipLaunchKernelGGL((w8a8_gemm_kernel<RAW_ACC>), dim3(tiles_m * tiles_n), dim3(256), LDS_BYTES, stream, p);
            return hipGetLastError();
        }
    } // namespace

    bool w8a8_skinny_supported(int M, int K)
    {
        if (M < 1 || M > 16 || (K & 63))
            return false;
        Q8SkinnyPlan pl = plan_q8_skinny(M, K);
        return pl.cps != 0 && pl.lds + 16 * 1024 <= MAX_LDS_BYTES;
    }

    hipError_t launch_w8a8(hipStream_t stream, const void* A, const void* s_tok, const void* W, const void* s_ch,
                           void* Y, void* acc, int M, int N, int K, int num_cu)
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
        return raw ? launch_q8_gemm<true>(stream, p) : launch_q8_gemm<false>(stream, p);
    }
} // namespace nnf
