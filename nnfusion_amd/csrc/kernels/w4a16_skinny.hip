// fp16 x int4 (g128) decode GEMV / skinny GEMM for M <= 16 on gfx950, on the matrix cores.
//
//   Y[M,N] = A[M,K] . ((Wq - zp) * S)^T
//
// The kernel is bound by the one pass over Wq (N*K/2 bytes) and S; everything else is arranged so
// that this pass runs at memory speed:
//   * one wavefront owns a tile of 16 weight rows and a K-slice of CPS groups of 128; one
//     128-bit load per lane fetches a whole group for the tile (16 rows x 64 B per instruction),
//     and the next tile's loads are issued before the current tile is computed;
//   * the dot products run on v_mfma_f32_16x16x32_f16 with the weight tile as the B operand
//     (columns = n) and the M <= 16 activation rows as the A operand (rows = m), so the cost per
//     weight byte does not depend on M;
//   * nibbles are turned into fp16 with one v_and_or_b32 per pair: (q | 0x6400) = 1024 + q, and a
//     nibble four bits up gives 1024 + 16 q.  Instead of subtracting the 1024 / zero point from
//     every weight, the activations of the "16 q" slots are pre-divided by 16 and the constant part
//         corr[m, group] = (1024 + zp) * sum_even a + (64 + zp) * 16 * sum_odd (a / 16)
//     is computed once per workgroup (by one MFMA against a constant operand) and used as the
//     negative initial accumulator of each group.  Products are exact in fp32, the sum of a group
//     is of order 1e4 at fp32 precision, i.e. an absolute error of ~1e-3 on a group sum of order 50;
//   * the group scale multiplies the fp32 group sum (4 FMAs per group and lane);
//   * the KS wavefronts of a workgroup split K; their partial tiles meet in LDS.
#include "nnf_device.h"
#include "nnf_launch.h"

#include <algorithm>

namespace nnf
{
    // LDS: activations as 16-byte units  unit(c, j, kq, m) = ((c*4 + j)*4 + kq)*M + m  holding the
    // eight fp16  a[m][c*128 + kq*32 + j*8 + {0,4,1,5,2,6,3,7}]  with slots 2,3,6,7 (odd k) times 1/16;
    // followed by the reduction buffer  red[2][KS][16 m][16 n]  fp32.
    template <int CPS>
    __global__ __launch_bounds__(1024) void w4a16_skinny_kernel(const half_t* __restrict__ A,
                                                                const uint8_t* __restrict__ Wq,
                                                                const half_t* __restrict__ S,
                                                                half_t* __restrict__ Y,
                                                                int M, int N, int K, int zp, int n_tiles)
    {
        extern __shared__ uintx4 lds[];
        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = tid >> 6;
        const int KS = blockDim.x >> 6;
        const int col = lane & 15; // n within the tile (B operand / D column), m for the A operand
        const int kq = lane >> 4;  // K quarter of the MFMA (A/B operands), row quad of D
        const int G = K >> 7;
        const int n_units = G * 16 * M;
        float* red = reinterpret_cast<float*>(lds + n_units);   // [2][KS][16][16]
        float* outb = red + 2 * KS * 256;                       // [tiles of this workgroup][M][16]
        const int chunk0 = wave * CPS;
        const size_t row_bytes = (size_t)(K >> 1);

        // Loads of one tile: unconditional (indices clamped to valid memory, scales of chunks past
        // the end of K forced to zero) so that no branch separates a load from its use and the
        // next tile's loads stay in flight while the current tile is computed.
        auto load_tile = [&](int tile, uintx4* w, uint32_t* s) {
            int n = min(tile * 16 + col, N - 1);
            const uint8_t* wrow = Wq + (size_t)n * row_bytes + kq * 16;
            const uint32_t* s32 = reinterpret_cast<const uint32_t*>(S);
            const size_t srow = (size_t)n * G;
#pragma unroll
            for (int c = 0; c < CPS; ++c)
            {
                int cc = min(chunk0 + c, G - 1);
                // plain (temporal) load: each instruction touches half of 16 cache lines, the next
                // chunk the other half; a non-temporal hint drops the line in between
                w[c] = *reinterpret_cast<const uintx4*>(wrow + (size_t)cc * 64);
                // The aligned 32-bit word that holds the fp16 scale; the half is picked at use.
                // (A 16-bit load makes the compiler carry a 16-bit value around the loop and
                // re-extend it at the latch, which waits for the prefetch to land.)
                s[c] = s32[(srow + cc) >> 1];
            }
        };

        uintx4 w0[CPS], w1[CPS];
        uint32_t s0[CPS], s1[CPS];
        float s_mask[CPS]; // 0 for chunks past the end of K
#pragma unroll
        for (int c = 0; c < CPS; ++c)
            s_mask[c] = (chunk0 + c < G) ? 1.0f : 0.0f;
        int tile = blockIdx.x; // the grid never exceeds n_tiles
        load_tile(tile, w0, s0);

        // ---- stage the activations -------------------------------------------------------------
        const half2_t sixteenth = half2_t{(half_t)0.0625f, (half_t)0.0625f};
        for (int u = tid; u < n_units; u += blockDim.x)
        {
            int m = u % M;
            int rest = u / M;
            int q = rest & 3;
            int j = (rest >> 2) & 3;
            int c = rest >> 4;
            uintx4 a = *reinterpret_cast<const uintx4*>(A + (size_t)m * K + (c << 7) + (q << 5) + (j << 3));
            a = permute_a8(a);
            a.y = as_u32(as_half2(a.y) * sixteenth);
            a.w = as_u32(as_half2(a.w) * sixteenth);
            lds[u] = a;
        }
        __syncthreads();

        const int m_rd = min(col, M - 1); // rows >= M read a valid row; their D rows are never stored
        // LDS unit index of this lane's A operand for chunk c, word j:  a_base + (c*16 + j*4) * M
        int a_unit[CPS];
#pragma unroll
        for (int c = 0; c < CPS; ++c)
            a_unit[c] = (min(chunk0 + c, G - 1) * 16 + kq) * M + m_rd;

        // ---- constant part of every group sum, negated: ncorr[c][r] for m = 4*kq + r ----------------
        floatx4 ncorr[CPS];
        {
            const half_t ce = (half_t)(-(1024.0f + (float)zp));
            const half_t co = (half_t)(-16.0f * (64.0f + (float)zp));
            const half8_t bconst = {ce, ce, co, co, ce, ce, co, co};
#pragma unroll
            for (int c = 0; c < CPS; ++c)
            {
                floatx4 t = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int j = 0; j < 4; ++j)
                {
                    uintx4 a = lds[a_unit[c] + j * 4 * M];
                    t = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a), bconst, t, 0, 0, 0);
                }
                ncorr[c] = t;
            }
        }

        // 0x64006400 in a scalar register, so that (w & mask) | magic is a single v_and_or_b32
        // (an instruction can carry only one 32-bit literal)
        uint32_t MAGIC;
        asm("s_mov_b32 %0, 0x64006400" : "=s"(MAGIC));

        int buf = 0;
        int local_tile = 0;
        auto compute_store = [&](int tile_id, const uintx4* wt, const uint32_t* st) {
            const int n_row = min(tile_id * 16 + col, N - 1);
            floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < CPS; ++c)
            {
                floatx4 t = ncorr[c];
                const uint32_t ww[4] = {wt[c].x, wt[c].y, wt[c].z, wt[c].w};
#pragma unroll
                for (int j = 0; j < 4; ++j)
                {
                    uint32_t w = ww[j];
                    uint32_t w8 = w >> 8;
                    uintx4 b;
                    b.x = (w & 0x000F000Fu) | MAGIC;  // 1024 + (q0, q4)
                    b.y = (w & 0x00F000F0u) | MAGIC;  // 1024 + 16 (q1, q5)
                    b.z = (w8 & 0x000F000Fu) | MAGIC; // 1024 + (q2, q6)
                    b.w = (w8 & 0x00F000F0u) | MAGIC; // 1024 + 16 (q3, q7)
                    uintx4 a = lds[a_unit[c] + j * 4 * M];
                    t = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a),
                                                               __builtin_bit_cast(half8_t, b), t, 0, 0, 0);
                }
                const int s_idx = n_row * G + min(chunk0 + c, G - 1);
                const uint32_t sbits = st[c] >> ((s_idx & 1) << 4);
                float sc = (float)__builtin_bit_cast(half2_t, sbits).x * s_mask[c];
                acc.x = __builtin_fmaf(t.x, sc, acc.x);
                acc.y = __builtin_fmaf(t.y, sc, acc.y);
                acc.z = __builtin_fmaf(t.z, sc, acc.z);
                acc.w = __builtin_fmaf(t.w, sc, acc.w);
            }

            // partial tile -> LDS: red[buf][wave][m = 4*kq + r][col]
            float* rp = red + ((buf * KS + wave) * 16 + kq * 4) * 16 + col;
            rp[0] = acc.x;
            rp[16] = acc.y;
            rp[32] = acc.z;
            rp[48] = acc.w;
            lds_barrier(); // LDS only: the prefetched global loads stay in flight
            // The sums are parked in LDS and written to Y after the last tile: a global store inside
            // the loop would make the next tile's address arithmetic wait for it, and with it for
            // every prefetched load issued before it (one in-order counter covers both).
            if (tid < M * 16)
            {
                const float* rr = red + buf * KS * 256 + tid; // tid = m*16 + n
                float v = 0.f;
                for (int w = 0; w < KS; ++w)
                    v += rr[w * 256];
                outb[local_tile * M * 16 + tid] = v;
            }
            buf ^= 1;
            ++local_tile;
        };

        // ---- tiles, software pipelined over two register sets -------------------------------------
        // A loop without early exits: a break between the two halves would merge, in the compiler's
        // control-flow graph, a path with loads still in flight into the loop header and force a
        // full vmcnt(0) wait there on every iteration.
        const int stride = gridDim.x;
        const int my_tiles = (n_tiles - tile + stride - 1) / stride;
        const int last_tile = tile + (my_tiles - 1) * stride;
        for (int p = 0; p < (my_tiles >> 1); ++p)
        {
            load_tile(tile + stride, w1, s1);
            __builtin_amdgcn_sched_barrier(0); // keep the prefetch ahead of the compute
            compute_store(tile, w0, s0);
            load_tile(min(tile + 2 * stride, last_tile), w0, s0);
            __builtin_amdgcn_sched_barrier(0);
            compute_store(tile + stride, w1, s1);
            tile += 2 * stride;
        }
        if (my_tiles & 1)
            compute_store(tile, w0, s0);

        // ---- write Y ----------------------------------------------------------------------------
        __syncthreads();
        const int per_tile = M * 16;
        for (int i = tid; i < local_tile * per_tile; i += blockDim.x)
        {
            int lt = i / per_tile;
            int r = i - lt * per_tile;
            int m = r >> 4;
            int n = ((int)blockIdx.x + lt * stride) * 16 + (r & 15);
            if (n < N)
                Y[(size_t)m * N + n] = (half_t)outb[i];
        }
    }

    namespace
    {
        struct SkinnyPlan
        {
            int cps = 0, ks = 0;
            size_t lds = 0;
        };

        // chunks-per-wave and waves-per-workgroup so that one workgroup spans all of K
        SkinnyPlan plan_skinny(int M, int K)
        {
            SkinnyPlan p;
            const int G = K >> 7;
            static const int cps_options[] = {1, 2, 3, 4, 6, 8};
            for (int cps : cps_options)
            {
                int ks = (G + cps - 1) / cps;
                if (g_tuning.skinny_cps != 0 && cps != g_tuning.skinny_cps)
                    continue;
                if (ks <= 16)
                {
                    p.cps = cps;
                    p.ks = ks;
                    break;
                }
            }
            if (p.cps == 0)
                return p;
            // activations + reduction buffers; the per-tile output parking area is added at launch
            p.lds = (size_t)G * 16 * M * 16 + (size_t)2 * p.ks * 256 * 4;
            return p;
        }

        template <int CPS>
        hipError_t launch_cps(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M, int N,
                              int K, int zp, const SkinnyPlan& p, int num_cu)
        {
            const int n_tiles = (N + 15) / 16;
            // persistent workgroups: one per CU when it has >= 8 wavefronts, else two
            int per_cu = p.ks >= 8 ? 1 : 2;
            if (g_tuning.skinny_wg_per_cu > 0)
                per_cu = g_tuning.skinny_wg_per_cu;
            int grid = std::min(n_tiles, num_cu * per_cu);
            int tiles_per_wg = (n_tiles + grid - 1) / grid;
            size_t lds_total = p.lds + (size_t)tiles_per_wg * M * 16 * 4;
            while (lds_total > MAX_LDS_BYTES && grid < n_tiles)
            {
                // a very large N: more, shorter workgroups so that the parked outputs fit
                grid = std::min(n_tiles, grid * 2);
                tiles_per_wg = (n_tiles + grid - 1) / grid;
                lds_total = p.lds + (size_t)tiles_per_wg * M * 16 * 4;
            }
            if (lds_total > MAX_LDS_BYTES)
                return hipErrorInvalidValue;
            if (lds_total > 64 * 1024)
            {
                hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&w4a16_skinny_kernel<CPS>),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_total);
                if (e != hipSuccess)
                    return e;
            }
            hipLaunchKernelGGL(w4a16_skinny_kernel<CPS>, dim3(grid), dim3(p.ks * 64), lds_total, stream,
                               (const half_t*)A, (const uint8_t*)Wq, (const half_t*)S, (half_t*)Y, M, N, K, zp,
                               n_tiles);
            return hipGetLastError();
        }
    } // namespace

    bool w4a16_skinny_supported(int M, int K)
    {
        if (M < 1 || M > 16 || (K & 127))
            return false;
        SkinnyPlan p = plan_skinny(M, K);
        // leave room for the output parking area (a few tiles of M x 16 floats)
        return p.cps != 0 && p.lds + 16 * 1024 <= MAX_LDS_BYTES;
    }

    hipError_t launch_w4a16_skinny(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M,
                                   int N, int K, int zp, int num_cu)
    {
        SkinnyPlan p = plan_skinny(M, K);
        switch (p.cps)
        {
        case 1: return launch_cps<1>(stream, A, Wq, S, Y, M, N, K, zp, p, num_cu);
        case 2: return launch_cps<2>(stream, A, Wq, S, Y, M, N, K, zp, p, num_cu);
        case 3: return launch_cps<3>(stream, A, Wq, S, Y, M, N, K, zp, p, num_cu);
        case 4: return launch_cps<4>(stream, A, Wq, S, Y, M, N, K, zp, p, num_cu);
        case 6: return launch_cps<6>(stream, A, Wq, S, Y, M, N, K, zp, p, num_cu);
        case 8: return launch_cps<8>(stream, A, Wq, S, Y, M, N, K, zp, p, num_cu);
        default: return hipErrorInvalidValue;
        }
    }
} // namespace nnf
