// fp16 x int4 (g128) decode GEMV / skinny GEMM for M <= 16 on gfx950, on the matrix cores.
//
//   Y[M,N] = A[M,K] . ((Wq - zp) * S)^T
//
// The kernel is bound by the one pass over Wq (N*K/2 bytes) and S; everything else is arranged so
// that this pass runs at memory speed:
//   * persistent workgroups (one per CU) walk tiles of 16 weight rows; the KS wavefronts of a
//     workgroup split K: a wavefront owns CPS groups of 128 in each of H passes over K (H = 1 for
//     K <= 8192, 2 above).  One 128-bit load per lane fetches a whole group for the tile; loads run
//     one to two tiles ahead of the MFMAs (two register sets, reloaded as soon as consumed);
//   * the group scales of a tile (16 rows x K/128 fp16, contiguous in memory) are fetched once per
//     workgroup with one coalesced 16-byte load per thread, two tiles ahead, and shared through LDS
//     -- per-lane scale loads would double the number of memory requests of the kernel;
//   * the dot products run on v_mfma_f32_16x16x32_f16 with the weight tile as the B operand
//     (columns = n) and the M <= 16 activation rows as the A operand (rows = m), so the cost per
//     weight byte does not depend on M.  The A operand is staged once per workgroup in LDS (already
//     permuted and pre-scaled); with up to two groups per wavefront it is then kept in registers;
//   * nibbles are turned into fp16 with one v_and_or_b32 per pair: (q | 0x6400) = 1024 + q, and a
//     nibble four bits up gives 1024 + 16 q.  Instead of subtracting the 1024 / zero point from
//     every weight, the activations of the "16 q" slots are pre-divided by 16 and the constant part
//         corr[m, group] = (1024 + zp) * sum_even a + (64 + zp) * 16 * sum_odd (a / 16)
//     is computed once per wavefront (one MFMA chain against a constant operand) and used as the
//     negative initial accumulator of each group.  Products are exact in fp32, the sum of a group
//     is of order 1e4 at fp32 precision, i.e. an absolute error of ~1e-3 on a group sum of order 50;
//   * the group scale multiplies the fp32 group sum (4 FMAs per group and lane);
//   * the partial tiles of the KS wavefronts meet in LDS (one LDS-only barrier per tile, so the
//     prefetched global loads stay in flight); results are parked in LDS and written once at the end.
#include "nnf_device.h"
#include "nnf_launch.h"

#include <algorithm>
#include <type_traits>

namespace nnf
{
    // LDS, in this order:
    //   activations as 16-byte units  unit(c, j, kq, m) = ((c*4 + j)*4 + kq)*M + m  holding
    //       the eight fp16  a[m][c*128 + kq*32 + j*8 + {0,4,1,5,2,6,3,7}]  with slots 2,3,6,7 (odd k) times 1/16
    //   scales   sc[2][16 rows][G] fp16 (as in memory), each copy padded to 16 bytes
    //   red      [2][KS][16 m][16 n] fp32 partial tiles
    //   outb     [tiles of this workgroup][M][16] fp32
    // Group (chunk) index of wavefront w, pass h, slot c:  (h*KS + w)*CPS + c.
    template <int CPS, bool A_REGS, int H>
    __global__ __launch_bounds__(1024) void w4a16_skinny_kernel(const half_t* __restrict__ A,
                                                                const uint8_t* __restrict__ Wq,
                                                                const half_t* __restrict__ S,
                                                                half_t* __restrict__ Y,
                                                                int M, int N, int K, int zp, int n_tiles)
    {
        static_assert(H == 1 || H == 2, "one or two passes over K");
        static_assert(!A_REGS || H == 1, "register-resident activations only with one pass");
        extern __shared__ uintx4 lds[];
        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = tid >> 6;
        const int KS = blockDim.x >> 6;
        const int col = lane & 15; // n within the tile (B operand / D column), m for the A operand
        const int kq = lane >> 4;  // K quarter of the MFMA (A/B operands), row quad of D
        const int G = K >> 7;
        const int a_units = G * 16 * M;
        const int sc_units = (16 * G * 2 + 15) >> 4; // 16-byte units of one scale copy
        uintx4* sc_lds = lds + a_units;
        float* red = reinterpret_cast<float*>(sc_lds + 2 * sc_units); // [2][KS][16][16]
        float* outb = red + 2 * KS * 256;
        const size_t row_bytes = (size_t)(K >> 1);
        const int m_rd = min(col, M - 1); // rows >= M read a valid row; their D rows are never stored
        int chunk_of[H][CPS];             // clamped to valid memory; chunks past the end of K are masked at use
        float s_mask[H][CPS];
#pragma unroll
        for (int h = 0; h < H; ++h)
#pragma unroll
            for (int c = 0; c < CPS; ++c)
            {
                int ch = (h * KS + wave) * CPS + c;
                chunk_of[h][c] = min(ch, G - 1);
                s_mask[h][c] = ch < G ? 1.0f : 0.0f;
            }

        // ---- loads: unconditional, so that no branch separates a load from its use ---------------------
        auto load_w = [&](int tile, int h, uintx4* w) {
            int n = min(tile * 16 + col, N - 1);
            const uint8_t* wrow = Wq + (size_t)n * row_bytes + kq * 16;
#pragma unroll
            for (int c = 0; c < CPS; ++c)
                w[c] = *reinterpret_cast<const uintx4*>(wrow + (size_t)chunk_of[h][c] * 64);
        };
        // scale block of a tile: bytes [tile*16*G*2, +16*G*2) of S; thread t carries bytes [16t, 16t+16)
        const size_t s_total = (size_t)N * G * 2;
        const bool s_loader = tid < sc_units;
        auto load_s = [&](int tile) -> uintx4 {
            size_t off = (size_t)tile * 16 * G * 2 + (size_t)tid * 16;
            off = min(off, s_total - 16); // rows past N (last tile) are never stored
            return *reinterpret_cast<const uintx4*>(reinterpret_cast<const uint8_t*>(S) + off);
        };

        const int stride = gridDim.x;
        const int tile0 = blockIdx.x; // the grid never exceeds n_tiles
        const int T = (n_tiles - tile0 + stride - 1) / stride;
        auto tile_at = [&](int k) { return tile0 + k * stride; };

        // register set 0 / 1: H == 1: even / odd tiles;  H == 2: first / second pass of the current tile
        uintx4 w0[CPS], w1[CPS], sreg = {0, 0, 0, 0};
        load_w(tile_at(0), 0, w0);
        if (s_loader)
            sreg = load_s(tile_at(0));
        if (H == 2)
            load_w(tile_at(0), H - 1, w1);
        else if (T > 1)
            load_w(tile_at(1), 0, w1);

        // ---- activations ---------------------------------------------------------------------------
        const half2_t sixteenth = half2_t{(half_t)0.0625f, (half_t)0.0625f};
        auto prep_a = [&](uintx4 a) {
            a = permute_a8(a);
            a.y = as_u32(as_half2(a.y) * sixteenth);
            a.w = as_u32(as_half2(a.w) * sixteenth);
            return a;
        };
        // Staged once per workgroup (one coalesced 16-byte load per thread and unit); every wavefront
        // loading its own operand straight from global memory would cost 8 load instructions per
        // wavefront, almost all of whose lanes are redundant.
        for (int u = tid; u < a_units; u += blockDim.x)
        {
            int m = u % M;
            int rest = u / M;
            int q = rest & 3;
            int j = (rest >> 2) & 3;
            int c = rest >> 4;
            lds[u] = prep_a(*reinterpret_cast<const uintx4*>(A + (size_t)m * K + (c << 7) + (q << 5) + (j << 3)));
        }
        int a_unit[H][CPS];
#pragma unroll
        for (int h = 0; h < H; ++h)
#pragma unroll
            for (int c = 0; c < CPS; ++c)
                a_unit[h][c] = (chunk_of[h][c] * 16 + kq) * M + m_rd;
        // scales of the first tile -> LDS copy 0, then fetch the second tile's
        if (s_loader)
        {
            sc_lds[tid] = sreg;
            if (T > 1)
                sreg = load_s(tile_at(1));
        }
        lds_barrier();

        // A_REGS: this wavefront's operand is read from LDS once and kept (16 VGPRs per group)
        uintx4 areg[A_REGS ? CPS : 1][4];
        if (A_REGS)
        {
#pragma unroll
            for (int c = 0; c < CPS; ++c)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    areg[A_REGS ? c : 0][j] = lds[a_unit[0][c] + j * 4 * M];
        }

        auto a_op = [&](int h, int c, int j) -> uintx4 {
            if (A_REGS)
                return areg[A_REGS ? c : 0][j];
            return lds[a_unit[h][c] + j * 4 * M];
        };

        // ---- constant part of every group sum, negated: ncorr[h][c][r] for m = 4*kq + r ---------------
        floatx4 ncorr[H][CPS];
        {
            const half_t ce = (half_t)(-(1024.0f + (float)zp));
            const half_t co = (half_t)(-16.0f * (64.0f + (float)zp));
            const half8_t bconst = {ce, ce, co, co, ce, ce, co, co};
#pragma unroll
            for (int h = 0; h < H; ++h)
#pragma unroll
                for (int c = 0; c < CPS; ++c)
                {
                    floatx4 t = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        t = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a_op(h, c, j)), bconst, t,
                                                                   0, 0, 0);
                    ncorr[h][c] = t;
                }
        }

        // 0x64006400 in a scalar register, so that (w & mask) | magic is a single v_and_or_b32
        // (an instruction can carry only one 32-bit literal)
        uint32_t MAGIC;
        asm("s_mov_b32 %0, 0x64006400" : "=s"(MAGIC));

        int local_tile = 0;
        // MFMAs of one pass h of a tile from register set wt, scales from LDS copy `par`, added to acc
        auto compute = [&](floatx4 acc, const uintx4* wt, auto hh, int par) -> floatx4 {
            constexpr int h = decltype(hh)::value;
            const half_t* sc = reinterpret_cast<const half_t*>(sc_lds + par * sc_units);
            // The A operand is re-read from LDS for every tile: hoisted out of the tile loop it would
            // occupy 16 VGPRs per group and spill.
            if (!A_REGS)
                asm volatile("" ::: "memory");
#pragma unroll
            for (int c = 0; c < CPS; ++c)
            {
                floatx4 t = ncorr[h][c];
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
                    t = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a_op(h, c, j)),
                                                               __builtin_bit_cast(half8_t, b), t, 0, 0, 0);
                }
                float s = (float)sc[col * G + chunk_of[h][c]] * s_mask[h][c];
                acc.x = __builtin_fmaf(t.x, s, acc.x);
                acc.y = __builtin_fmaf(t.y, s, acc.y);
                acc.z = __builtin_fmaf(t.z, s, acc.z);
                acc.w = __builtin_fmaf(t.w, s, acc.w);
                // keep the scheduler from pulling every group's LDS reads to the front (16 VGPRs each)
                if (!A_REGS)
                    __builtin_amdgcn_sched_barrier(0);
            }
            return acc;
        };
        // After the MFMAs of a tile: partial tile -> LDS; the scales of the next tile (in sreg) -> the
        // other LDS copy [put_s]; fetch the scales of the tile after it [get_s]; reload the freed weight
        // register set [get_w]; barrier; reduction.  The flags are compile-time so that the steady-state
        // loop has no branch around a load (a load on one side of a branch makes the compiler wait for
        // all loads at the join).
        auto finish = [&](floatx4 acc, int par, auto put_s, auto get_s, int tile_s, auto get_w, int tile_w, int h_w,
                          uintx4* w_free) {
            float* rp = red + ((par * KS + wave) * 16 + kq * 4) * 16 + col;
            rp[0] = acc.x;
            rp[16] = acc.y;
            rp[32] = acc.z;
            rp[48] = acc.w;
            // Order matters for the in-order load counter: the scale registers (loaded one tile ago) are
            // consumed first, then reloaded, and only then is the freed weight register set reloaded --
            // so waiting for the scales next time does not also wait for these weight loads.
            if (s_loader)
            {
                if (decltype(put_s)::value)
                    sc_lds[(par ^ 1) * sc_units + tid] = sreg;
                if (decltype(get_s)::value)
                    sreg = load_s(tile_s);
            }
            if (decltype(get_w)::value)
            {
                load_w(tile_w, h_w, w_free);
                __builtin_amdgcn_sched_barrier(0);
            }
            lds_barrier(); // LDS only: the prefetched global loads stay in flight
            // The sums are parked in LDS and written to Y after the last tile: a global store inside
            // the loop would make later address arithmetic wait for it, and with it for every
            // prefetched load issued before it (one in-order counter covers both).
            if (tid < M * 16)
            {
                const float* rr = red + par * KS * 256 + tid; // tid = m*16 + n
                float v = 0.f;
                for (int w = 0; w < KS; w += 4)
                {
                    // four independent reads per step (clamped: a repeated slot is not added)
                    float p0 = rr[w * 256];
                    float p1 = rr[min(w + 1, KS - 1) * 256];
                    float p2 = rr[min(w + 2, KS - 1) * 256];
                    float p3 = rr[min(w + 3, KS - 1) * 256];
                    v += p0;
                    v += (w + 1 < KS) ? p1 : 0.f;
                    v += (w + 2 < KS) ? p2 : 0.f;
                    v += (w + 3 < KS) ? p3 : 0.f;
                }
                outb[local_tile * M * 16 + tid] = v;
            }
            ++local_tile;
        };
        const std::true_type yes;
        const std::false_type no;
        const std::integral_constant<int, 0> h0;
        const std::integral_constant<int, H - 1> h1;
        const floatx4 zero = {0.f, 0.f, 0.f, 0.f};

        if (H == 1)
        {
            // tiles k = 0 .. T-1: even tiles use register set w0 / scale copy 0, odd tiles w1 / copy 1.
            // Steady state (both k+2 and k+3 exist), then the last one to three tiles without useless loads.
            int k = 0;
            for (; k + 3 < T; k += 2)
            {
                floatx4 acc = compute(zero, w0, h0, 0);
                finish(acc, 0, yes, yes, tile_at(k + 2), yes, tile_at(k + 2), 0, w0);
                acc = compute(zero, w1, h0, 1);
                finish(acc, 1, yes, yes, tile_at(k + 3), yes, tile_at(k + 3), 0, w1);
            }
            const int rest = T - k; // 1, 2 or 3
            if (rest == 3)
            {
                floatx4 acc = compute(zero, w0, h0, 0);
                finish(acc, 0, yes, yes, tile_at(k + 2), yes, tile_at(k + 2), 0, w0);
                acc = compute(zero, w1, h0, 1);
                finish(acc, 1, yes, no, 0, no, 0, 0, w1);
                acc = compute(zero, w0, h0, 0);
                finish(acc, 0, no, no, 0, no, 0, 0, w0);
            }
            else if (rest == 2)
            {
                floatx4 acc = compute(zero, w0, h0, 0);
                finish(acc, 0, yes, no, 0, no, 0, 0, w0);
                acc = compute(zero, w1, h0, 1);
                finish(acc, 1, no, no, 0, no, 0, 0, w1);
            }
            else
            {
                floatx4 acc = compute(zero, w0, h0, 0);
                finish(acc, 0, no, no, 0, no, 0, 0, w0);
            }
        }
        else
        {
            // two passes per tile: w0 holds the first pass, w1 the second; after pass h of tile k its set
            // is reloaded with pass h of tile k+1.  Scale copy k & 1.
            int k = 0;
            for (; k + 2 < T; ++k)
            {
                floatx4 acc = compute(zero, w0, h0, k & 1);
                load_w(tile_at(k + 1), 0, w0);
                __builtin_amdgcn_sched_barrier(0);
                acc = compute(acc, w1, h1, k & 1);
                finish(acc, k & 1, yes, yes, tile_at(k + 2), yes, tile_at(k + 1), H - 1, w1);
            }
            if (T - k == 2)
            {
                floatx4 acc = compute(zero, w0, h0, k & 1);
                load_w(tile_at(k + 1), 0, w0);
                __builtin_amdgcn_sched_barrier(0);
                acc = compute(acc, w1, h1, k & 1);
                finish(acc, k & 1, yes, no, 0, yes, tile_at(k + 1), H - 1, w1);
                ++k;
            }
            floatx4 acc = compute(zero, w0, h0, k & 1);
            acc = compute(acc, w1, h1, k & 1);
            finish(acc, k & 1, no, no, 0, no, 0, 0, w1);
        }

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
            int cps = 0, ks = 0, h = 0;
            bool a_regs = false;
            size_t lds = 0; // without the output parking area
        };

        // groups per wavefront and pass, wavefronts per workgroup, passes: one workgroup spans all of K
        SkinnyPlan plan_skinny(int M, int K)
        {
            SkinnyPlan p;
            const int G = K >> 7;
            struct Option
            {
                int cps, h;
            };
            // fewest groups per wavefront first (more wavefronts in flight); two passes beyond 16 * 4 groups
            static const Option options[] = {{1, 1}, {2, 1}, {3, 1}, {4, 1}, {3, 2}, {4, 2}};
            for (const Option& o : options)
            {
                int ks = (G + o.cps * o.h - 1) / (o.cps * o.h);
                if (g_tuning.skinny_cps != 0 && o.cps != g_tuning.skinny_cps)
                    continue;
                if (ks <= 16)
                {
                    p.cps = o.cps;
                    p.h = o.h;
                    p.ks = ks;
                    break;
                }
            }
            if (p.cps == 0)
                return p;
            // the A operand fits in registers up to two groups per wavefront (32 VGPRs)
            p.a_regs = p.cps <= 2 && p.h == 1;
            const size_t a_bytes = (size_t)G * 16 * M * 16;
            const size_t sc_bytes = 2 * (((size_t)16 * G * 2 + 15) & ~(size_t)15);
            p.lds = a_bytes + sc_bytes + (size_t)2 * p.ks * 256 * 4;
            return p;
        }

        template <int CPS, bool A_REGS, int H>
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
                hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&w4a16_skinny_kernel<CPS, A_REGS, H>),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_total);
                if (e != hipSuccess)
                    return e;
            }
            hipLaunchKernelGGL((w4a16_skinny_kernel<CPS, A_REGS, H>), dim3(grid), dim3(p.ks * 64), lds_total, stream,
                               (const half_t*)A, (const uint8_t*)Wq, (const half_t*)S, (half_t*)Y, M, N, K, zp, n_tiles);
            return hipGetLastError();
        }
    } // namespace

    bool w4a16_skinny_supported(int M, int N, int K)
    {
        if (M < 1 || M > 16 || (K & 127))
            return false;
        // the scale block of a tile is fetched in whole 16-byte pieces
        if (((size_t)N * (K >> 7) * 2) % 16 != 0 || (size_t)N * (K >> 7) * 2 < 16)
            return false;
        SkinnyPlan p = plan_skinny(M, K);
        // leave room for the output parking area (a few tiles of M x 16 floats)
        return p.cps != 0 && p.lds + 16 * 1024 <= MAX_LDS_BYTES;
    }

    hipError_t launch_w4a16_skinny(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M,
                                   int N, int K, int zp, int num_cu)
    {
        SkinnyPlan p = plan_skinny(M, K);
        switch (p.cps * 10 + p.h)
        {
        case 11: return launch_cps<1, true, 1>(stream, A, Wq, S, Y, M, N, K, zp, p, num_cu);
        case 21: return launch_cps<2, true, 1>(stream, A, Wq, S, Y, M, N, K, zp, p, num_cu);
        case 31: return launch_cps<3, false, 1>(stream, A, Wq, S, Y, M, N, K, zp, p, num_cu);
        case 41: return launch_cps<4, false, 1>(stream, A, Wq, S, Y, M, N, K, zp, p, num_cu);
        case 32: return launch_cps<3, false, 2>(stream, A, Wq, S, Y, M, N, K, zp, p, num_cu);
        case 42: return launch_cps<4, false, 2>(stream, A, Wq, S, Y, M, N, K, zp, p, num_cu);
        default: return hipErrorInvalidValue;
        }
    }
} // namespace nnf
