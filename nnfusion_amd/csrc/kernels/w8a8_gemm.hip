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

    // CPS: 64-byte chunks of K per wavefront and pass; KH: passes over K per tile (the weights of a
    // pass sit in one of two register buffers that take turns; 1 or even).
    template <int CPS, int KH, bool RAW_ACC>
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
        const int C = K >> 6;            // 64-byte chunks per row
        const int c_pad = KS * CPS * KH; // chunks the workgroup walks; activations past C are zero
        const int rows_c4 = C * 4, rows_pad = c_pad * 4;
        int32_t* red = reinterpret_cast<int32_t*>(lds + rows_pad * M);
        int32_t* outb = red + 2 * KS * 256;

        // A tile index past the end of the matrix loads one cache line over and over (the loads stay
        // unconditional so that the loop's wait counts do not depend on a branch; the values are unused).
        // Chunks past the end of K read the last chunk again and meet zero activations.
        auto load_seq = [&](int seq, uintx4* w) {
            const int tile = (int)blockIdx.x + (seq / KH) * (int)gridDim.x;
            const int h = seq % KH;
            const bool real = tile < n_tiles;
            const int n = min(tile * 16 + col, N - 1);
            const int8_t* wrow = real ? p.W + (size_t)n * K + kq * 16 : p.W;
            const size_t step = real ? 64 : 0;
            const int chunk0 = (h * KS + wave) * CPS;
#pragma unroll
            for (int c = 0; c < CPS; ++c)
                w[c] = *reinterpret_cast<const uintx4*>(wrow + (size_t)min(chunk0 + c, C - 1) * step);
        };

        // Activations first (a few loads, needed by the first product), then two buffers of weights:
        // everything a workgroup with two passes needs is requested before the first wait.
        const uintx4 zero = {0u, 0u, 0u, 0u};
        uintx4 a_first[4];
        {
            const int r = min(tid, rows_c4 - 1);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                a_first[j] = *reinterpret_cast<const uintx4*>(p.A + (size_t)min(j, M - 1) * K + (size_t)r * 16);
        }

        uintx4 w0[CPS], w1[CPS];
        load_seq(0, w0);
        load_seq(1, w1);

        if (tid < rows_pad)
        {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (j < M)
                    lds[tid * M + j] = tid < rows_c4 ? a_first[j] : zero;
        }
        // rows 4.. of the activations and the part of a row past the workgroup's width
        for (int m0 = 0; m0 < M; m0 += 4)
        {
            for (int r = tid + (m0 == 0 ? (int)blockDim.x : 0); r < rows_pad; r += blockDim.x)
            {
                const int rl = min(r, rows_c4 - 1);
                uintx4 t[4];
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    t[j] = *reinterpret_cast<const uintx4*>(p.A + (size_t)min(m0 + j, M - 1) * K + (size_t)rl * 16);
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (m0 + j < M)
                        lds[r * M + m0 + j] = r < rows_c4 ? t[j] : zero;
            }
        }
        __syncthreads();

        const int a_base = (wave * CPS * 4 + kq) * M + min(col, M - 1);
        const int a_chunk = 4 * M;          // units between the chunks of a wavefront
        const int a_pass = KS * CPS * 4 * M; // units between the passes

        int buf = 0, local_tile = 0;
        auto accumulate = [&](const uintx4* wt, int h, intx4 acc) {
#pragma unroll
            for (int c = 0; c < CPS; ++c)
            {
                uintx4 a = lds[a_base + h * a_pass + c * a_chunk];
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(intx4, a),
                                                            __builtin_bit_cast(intx4, wt[c]), acc, 0, 0, 0);
            }
            return acc;
        };
        auto reduce_store = [&](intx4 acc) {
            int32_t* rp = red + ((buf * KS + wave) * 16 + kq * 4) * 16 + col;
            rp[0] = acc.x;
            rp[16] = acc.y;
            rp[32] = acc.z;
            rp[48] = acc.w;
            lds_barrier();
            // (K = 128: two wavefronts, fewer threads than the M x 16 outputs of a tile from 9 rows on)
            for (int o = tid; o < M * 16; o += (int)blockDim.x)
            {
                const int32_t* rr = red + buf * KS * 256 + o;
                int32_t v = 0;
                for (int w = 0; w < KS; ++w)
                    v += rr[w * 256];
                outb[local_tile * M * 16 + o] = v;
            }
            buf ^= 1;
            ++local_tile;
        };

        const intx4 acc0 = {0, 0, 0, 0};
        const int stride = gridDim.x;
        const int my_tiles = (n_tiles - (int)blockIdx.x + stride - 1) / stride;
        int seq = 0;
        if (KH >= 2)
        {
            for (int it = 0; it < my_tiles; ++it)
            {
                intx4 acc = acc0;
#pragma unroll
                for (int h = 0; h < KH; h += 2)
                {
                    acc = accumulate(w0, h, acc);
                    load_seq(seq + 2, w0);
                    __builtin_amdgcn_sched_barrier(0);
                    acc = accumulate(w1, h + 1, acc);
                    load_seq(seq + 3, w1);
                    __builtin_amdgcn_sched_barrier(0);
                    seq += 2;
                }
                reduce_store(acc);
            }
        }
        else
        {
            for (int it = 0; it < (my_tiles >> 1); ++it)
            {
                reduce_store(accumulate(w0, 0, acc0));
                load_seq(seq + 2, w0);
                __builtin_amdgcn_sched_barrier(0);
                reduce_store(accumulate(w1, 0, acc0));
                load_seq(seq + 3, w1);
                __builtin_amdgcn_sched_barrier(0);
                seq += 2;
            }
            if (my_tiles & 1)
                reduce_store(accumulate(w0, 0, acc0));
        }

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
        Q8SkinnyPlan plan_q8_skinny(int M, int K) { return workspace::plan_w8a8_skinny(M, K, 0); }

        template <int CPS, int KH, bool RAW_ACC>
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
                static LdsGrant granted;
                const hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(&w8a8_skinny_kernel<CPS, KH, RAW_ACC>),
                                                       granted, (int)MAX_LDS_BYTES);
                if (e != hipSuccess)
                    return e;
            }
            hipLaunchKernelGGL((w8a8_skinny_kernel<CPS, KH, RAW_ACC>), dim3(grid), dim3(pl.ks * 64), lds_total, stream, p,
                               n_tiles);
            return hipGetLastError();
        }

        template <bool RAW_ACC>
        hipError_t launch_q8_skinny(hipStream_t stream, const W8A8Params& p, int num_cu)
        {
            Q8SkinnyPlan pl = plan_q8_skinny(p.M, p.K);
            switch (pl.cps * 16 + pl.kh)
            {
#define NNF_Q8_CASE(CPS, KH)                                                                                           \
    case CPS * 16 + KH: return launch_q8_skinny_cps<CPS, KH, RAW_ACC>(stream, p, pl, num_cu);
                NNF_Q8_CASE(1, 1)
                NNF_Q8_CASE(2, 1)
                NNF_Q8_CASE(4, 1)
                NNF_Q8_CASE(8, 1)
                NNF_Q8_CASE(1, 2)
                NNF_Q8_CASE(2, 2)
                NNF_Q8_CASE(4, 2)
                NNF_Q8_CASE(8, 2)
                NNF_Q8_CASE(1, 4)
                NNF_Q8_CASE(2, 4)
                NNF_Q8_CASE(4, 4)
                NNF_Q8_CASE(1, 8)
                NNF_Q8_CASE(2, 8)
#undef NNF_Q8_CASE
            default: return hipErrorInvalidValue;
            }
        }
    } // namespace

    bool w8a8_skinny_supported(int M, int K) { return workspace::w8a8_skinny_fits(M, K); }

    namespace
    {
        enum Q8Kind { Q8_NONE = -1, Q8_ROWS, Q8_MROWS, Q8_SKINNY, Q8_TILE };
        // the kernel family that serves a call: the caller's choice where it made one (Q8_NONE: that family cannot
        // serve the shape), otherwise by shape
        Q8Kind pick_w8a8(int M, int N, int K, int num_cu, int path)
        {
            switch (path)
            {
            case 0:
                if (w8a8_gemv_rows_supported(M, N, K, num_cu))
                    return Q8_ROWS;
                if (w8a8_mrows_preferred(M, N, K, num_cu))
                    return Q8_MROWS;
                return w8a8_skinny_supported(M, K) ? Q8_SKINNY : Q8_TILE;
            case 2: return w8a8_skinny_supported(M, K) ? Q8_SKINNY : Q8_NONE;
            case 3: return Q8_TILE;
            case 4:
                if (M == 1)
                    return w8a8_gemv_rows_supported(M, N, K, num_cu) ? Q8_ROWS : Q8_NONE;
                return w8a8_mrows_supported(M, N, K, num_cu) ? Q8_MROWS : Q8_NONE;
            default: return Q8_NONE;
            }
        }
    } // namespace

    bool w8a8_path_supported(int M, int N, int K, int num_cu, int path)
    {
        return pick_w8a8(M, N, K, num_cu, path) != Q8_NONE;
    }

    size_t w8a8_partial_bytes(int M, int N, int K, int num_cu, const LaunchChoice& choice)
    {
        const Q8Kind kind = pick_w8a8(M, N, K, num_cu, choice.path);
        if (kind == Q8_MROWS) // (two ranges of K, their sums added up in the launch: with synchronisation words only)
            return choice.sync_flags && choice.sync_bytes >= workspace::mrows_split_sync_bytes(num_cu)
                       ? workspace::w8a8_mrows_ranges_bytes(M, N, K, num_cu)
                       : 0;
        if (kind != Q8_TILE)
            return 0;
        const int tile = workspace::w8a8_forced_tile(choice.tile_rows, choice.tile_cols);
        return workspace::gemm_partial_bytes(M, N, false, workspace::plan_w8a8_gemm(M, N, K, tile, choice.k_parts));
    }

    bool w8a8_partial_optional(int M, int N, int K, int num_cu, const LaunchChoice& choice)
    {
        return pick_w8a8(M, N, K, num_cu, choice.path) == Q8_MROWS;
    }

    hipError_t launch_w8a8(hipStream_t stream, const void* A, const void* s_tok, const void* W, const void* s_ch,
                           void* Y, void* acc, int M, int N, int K, int num_cu, void* partial_ws, size_t partial_bytes,
                           const LaunchChoice& choice)
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
        switch (pick_w8a8(M, N, K, num_cu, choice.path))
        {
        case Q8_ROWS: return launch_w8a8_gemv_rows(stream, A, s_tok, W, s_ch, Y, acc, N, K, num_cu);
        case Q8_MROWS:
            return launch_w8a8_mrows(stream, A, s_tok, W, s_ch, Y, acc, M, N, K, num_cu, partial_ws, partial_bytes,
                                     (uint32_t*)choice.sync_flags, choice.sync_bytes);
        case Q8_SKINNY: return raw ? launch_q8_skinny<true>(stream, p, num_cu) : launch_q8_skinny<false>(stream, p, num_cu);
        case Q8_TILE: return launch_w8a8_gemm(stream, A, s_tok, W, s_ch, Y, acc, M, N, K, partial_ws, choice);
        default: return hipErrorInvalidValue;
        }
    }
} // namespace nnf
