// fp16 x int4 (g128) MFMA GEMM kernel template for gfx950, shared by the translation units that
// instantiate its tile shapes.
//
//   Y[M,N] = epilogue( A[M,K] . ((Wq - zp) * S)^T )
//
// Replaces the cublasSgemm/cublasHgemm call that the reference's cuda::Dot emits
// (src/nnfusion/core/kernels/cuda_gpu/kernels/dot.cpp:128-205, 271-363) for a weight-quantized Dot
// with transpose_B, plus the element-wise kernels around it.
//
// Structure (8 wavefronts, WM x WN of them over a BM x BN tile, 32x32x16 MFMAs, BK = 64):
//   * Operands go global -> LDS asynchronously (global_load_lds_dwordx4: no register staging, no LDS
//     store instructions) into a three-stage ring, so that the operands of two K steps are in flight
//     while one is computed.  A wavefront-wide direct load fills 1 KiB of consecutive LDS; the XOR
//     swizzle that keeps the 16-byte fragment reads conflict-free is obtained by choosing which
//     16-byte piece of global memory each lane fetches.
//   * Nothing can be permuted on the way, so the activations stay in natural K order and the weights
//     are unpacked in natural order too: v_perm_b32 copies byte i of a word (nibbles 2i, 2i+1) into
//     bytes 0 and 2, one v_and_or_b32 makes (1024 + q_2i, 1024 + 16 q_2i+1), one packed fma with the
//     constants (1, 1/16) and (-(1024+zp), -(64+zp)) gives the exact (q - zp) pair, one packed multiply
//     applies the group scale: 16 VALU operations per 8 weights.
//   * One barrier per K step: after it, every wavefront's loads for this step have landed and every
//     wavefront has finished reading the stage that is about to be refilled.
//   * Tiles are numbered so that each XCD (own L2) works on a contiguous run of tiles, and within the
//     run four tile rows advance together along N: the 32 workgroups an XCD runs at a time share
//     4 A panels and 8 W panels instead of 16 and 2.
//   * SPLITK: the workgroup covers a range of quantization groups and writes raw fp32 partial sums
//     [split][m][column]; a small second kernel adds the splits and applies the epilogue.
//   * Epilogues round the way the unfused graph would: the GEMM result to fp16 first, then the
//     element-wise operation in fp32, then fp16 again.
#pragma once

#include "nnf_device.h"
#include "nnf_launch.h"

namespace nnf
{
    struct GemmParams
    {
        const half_t* A;
        const uint8_t* Wq;
        const half_t* S;
        half_t* Y;
        int M, N, K, zp;        // N = output columns
        int ldy;                // row stride of Y
        int up_row_offset;      // GATE: weight row of the up projection that pairs with gate row 0
        const half_t* bias;     // BIAS: [N]
        const half_t* residual; // RESID: [M, ldy]
        float* partial;         // SPLITK: [splits][M][ld_partial] fp32
        int splits;             // SPLITK: number of K ranges (1 otherwise)
        int ld_partial;         // SPLITK: N, or 2 N with GATE (gate columns, then up columns)
    };

    namespace gemm_dl
    {
        constexpr int BK = 64;
        constexpr int THREADS = 512; // 8 wavefronts
        constexpr int STAGES = 3;

        template <int WM, int WN, int TM, int TN>
        struct Tile
        {
            static_assert(WM * WN == 8, "eight wavefronts per workgroup");
            static constexpr int BM = WM * TM * 32;
            static constexpr int BN = WN * TN * 32;
            static_assert(BM >= 32 && BN >= 128, "a wavefront-wide load covers 8 A rows / 32 W rows");
            static constexpr int A_TILE_BYTES = BM * BK * 2;
            static constexpr int W_TILE_BYTES = BN * BK / 2;
            static constexpr int STAGE_BYTES = A_TILE_BYTES + W_TILE_BYTES;
            static constexpr int LDS_BYTES = STAGES * STAGE_BYTES;
            static constexpr int A_CHUNKS = BM / 8;    // wavefront-wide loads in one A tile
            static constexpr int A_LOADS = A_CHUNKS >= 8 ? A_CHUNKS / 8 : 1; // per wavefront
            static constexpr int W_CHUNKS = BN / 32;   // wavefront-wide loads in one W tile
            // every wavefront issues the same number of loads (the wait counts below rely on it): with
            // fewer than 8 chunks two wavefronts fetch the same chunk into the same place
            static constexpr int W_LOADS = W_CHUNKS >= 8 ? W_CHUNKS / 8 : 1;
            static constexpr int TILE_LOADS = A_LOADS + W_LOADS;
        };

        // s_waitcnt with only the vector-memory counter set (gfx9 encoding: vmcnt = bits 3:0 and 15:14)
        constexpr int vmcnt_imm(int n) { return (n & 0xF) | ((n >> 4) << 14) | (0x7 << 4) | (0xF << 8); }
    } // namespace gemm_dl

    // MINW: wavefronts per SIMD the register allocation has to leave room for (2 = one workgroup per CU)
    template <int WM, int WN, int TM, int TN, bool GATE, bool BIAS, bool RESID, bool SPLITK, int MINW>
    __global__ __launch_bounds__(512, MINW) void w4a16_gemm_dl_kernel(GemmParams p)
    {
        using namespace gemm_dl;
        using T = Tile<WM, WN, TM, TN>;
        static_assert(!GATE || TN == 2, "GATE pairs the two column tiles of a wavefront");
        constexpr int BM = T::BM, BN = T::BN;
        constexpr int A_LOADS = T::A_LOADS, W_LOADS = T::W_LOADS, TILE_LOADS = T::TILE_LOADS;
        constexpr int A_TILE_BYTES = T::A_TILE_BYTES, STAGE_BYTES = T::STAGE_BYTES;
        constexpr int BN_OUT = GATE ? BN / 2 : BN;
        extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
        // volatile: the vector move has to stay here, where every lane is active
        uint32_t MASK, MAGIC, SEL[4];
        asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(MAGIC));
        asm volatile("s_mov_b32 %0, 0x00F0000F" : "=s"(MASK));
        asm volatile("s_mov_b32 %0, 0x0c000c00" : "=s"(SEL[0]));
        asm volatile("s_mov_b32 %0, 0x0c010c01" : "=s"(SEL[1]));
        asm volatile("s_mov_b32 %0, 0x0c020c02" : "=s"(SEL[2]));
        asm volatile("s_mov_b32 %0, 0x0c030c03" : "=s"(SEL[3]));
        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int wm = wave / WN, wn = wave % WN;
        const int l32 = lane & 31, h = lane >> 5;
        const int K = p.K;
        const int G = K >> 7;

        const int tiles_m = (p.M + BM - 1) / BM;
        const int tiles_n = (p.N + BN_OUT - 1) / BN_OUT;
        const int n_wg = tiles_m * tiles_n;
        const int split = SPLITK ? (int)blockIdx.x / n_wg : 0;
        int pid = SPLITK ? (int)blockIdx.x - split * n_wg : (int)blockIdx.x;
        {
            // contiguous run of tiles per XCD (workgroup ids are dealt round-robin to the 8 XCDs)
            const int per_xcd = (n_wg + 7) >> 3;
            const int full = n_wg - (per_xcd - 1) * 8;
            const int xcd = pid & 7, idx = pid >> 3;
            pid = (xcd < full) ? xcd * per_xcd + idx : full * per_xcd + (xcd - full) * (per_xcd - 1) + idx;
        }
        int tm, tn;
        {
            // four tile rows advance together along N
            constexpr int GM = 4;
            const int per_group = GM * tiles_n;
            const int g = pid / per_group;
            const int first_m = g * GM;
            const int gm = min(GM, tiles_m - first_m);
            const int r = pid - g * per_group;
            tm = first_m + r % gm;
            tn = r / gm;
        }
        const int m0 = tm * BM, n0 = tn * BN_OUT;

        // this workgroup's range of quantization groups (all of them without SPLITK)
        const int g_begin = SPLITK ? (int)(((long long)split * G) / p.splits) : 0;
        const int g_end = SPLITK ? (int)(((long long)(split + 1) * G) / p.splits) : G;
        const int KT = 2 * (g_end - g_begin); // K steps of this workgroup: even, >= 2
        const int k_begin = g_begin * 128;

        // ---- direct-load maps -------------------------------------------------------------------------
        // A: chunk c fills LDS rows c*8 .. +7; lane l lands at (row = c*8 + l/8, slot = l%8) and therefore
        // fetches piece  slot ^ ((row >> 1) & 7)  of that row.
        const half_t* a_src[A_LOADS];
        int a_chunk[A_LOADS];
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i)
        {
            a_chunk[i] = (wave * A_LOADS + i) % T::A_CHUNKS;
            int row = a_chunk[i] * 8 + (lane >> 3);
            int piece = (lane & 7) ^ ((row >> 1) & 7);
            a_src[i] = p.A + (size_t)min(m0 + row, p.M - 1) * K + k_begin + piece * 8;
        }
        // W: chunk c fills LDS rows c*32 .. +31 (32 B each); lane l lands at (row = c*32 + l/2, slot = l%2)
        const uint8_t* w_src[W_LOADS];
        int w_chunk[W_LOADS];
#pragma unroll
        for (int i = 0; i < W_LOADS; ++i)
        {
            w_chunk[i] = (wave * W_LOADS + i) % T::W_CHUNKS;
            int row = w_chunk[i] * 32 + (lane >> 1);
            int piece = (lane & 1) ^ ((row >> 3) & 1);
            int gn;
            if (GATE)
            {
                gn = (row < BN / 2) ? (n0 + row) : (p.up_row_offset + n0 + (row - BN / 2));
                gn = min(gn, p.up_row_offset + p.N - 1);
            }
            else
            {
                gn = min(n0 + row, p.N - 1);
            }
            w_src[i] = p.Wq + (size_t)gn * (K >> 1) + (k_begin >> 1) + piece * 16;
        }
        auto issue_tile_loads = [&](int kt, int stage) {
            uint8_t* base = smem + stage * STAGE_BYTES;
            const int k0 = kt * BK;
#pragma unroll
            for (int i = 0; i < A_LOADS; ++i)
                __builtin_amdgcn_global_load_lds(
                    (const void __attribute__((address_space(1)))*)(a_src[i] + k0),
                    (void __attribute__((address_space(3)))*)(base + a_chunk[i] * 1024), 16, 0, 0);
#pragma unroll
            for (int i = 0; i < W_LOADS; ++i)
                __builtin_amdgcn_global_load_lds(
                    (const void __attribute__((address_space(1)))*)(w_src[i] + (k0 >> 1)),
                    (void __attribute__((address_space(3)))*)(base + A_TILE_BYTES + w_chunk[i] * 1024), 16, 0, 0);
        };

        // ---- per-lane fragment addresses in LDS ------------------------------------------------------
        int a_frag[TM], a_swz[TM];
#pragma unroll
        for (int i = 0; i < TM; ++i)
        {
            int r = wm * (TM * 32) + i * 32 + l32;
            a_frag[i] = r * 128;
            a_swz[i] = (r >> 1) & 7;
        }
        int w_frag[TN];
        size_t s_idx[TN];
#pragma unroll
        for (int j = 0; j < TN; ++j)
        {
            int r, gn;
            if (GATE)
            {
                int c = wn * 32 + l32;
                r = j * (BN / 2) + c; // j = 0: gate, 1: up
                gn = j ? (p.up_row_offset + n0 + c) : (n0 + c);
                gn = min(gn, p.up_row_offset + p.N - 1);
            }
            else
            {
                r = wn * (TN * 32) + j * 32 + l32;
                gn = min(n0 + r, p.N - 1);
            }
            w_frag[j] = A_TILE_BYTES + r * 32 + ((h ^ ((r >> 3) & 1)) << 4);
            s_idx[j] = (size_t)gn * G + g_begin;
        }

        floatx16 acc[TM][TN];
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    acc[i][j][e] = 0.f;

        const half2_t dq_mul = half2_t{(half_t)1.0f, (half_t)0.0625f};
        const half2_t dq_add = half2_t{(half_t)(-(1024.0f + (float)p.zp)), (half_t)(-(64.0f + (float)p.zp))};

        // group scales, fetched one group (two K steps) ahead as the aligned 32-bit word holding the fp16
        const uint32_t* s32 = reinterpret_cast<const uint32_t*>(p.S);
        const int n_groups = g_end - g_begin;
        uint32_t s_nxt[TN];
        auto load_scales = [&](int g) {
            g = min(g, n_groups - 1);
#pragma unroll
            for (int j = 0; j < TN; ++j)
                s_nxt[j] = s32[(s_idx[j] + g) >> 1];
        };
        half2_t sc[TN];
        auto take_scales = [&](int g) {
#pragma unroll
            for (int j = 0; j < TN; ++j)
            {
                uint32_t bits = s_nxt[j] >> ((((uint32_t)s_idx[j] + (uint32_t)g) & 1u) << 4);
                half_t s = as_half2(bits).x;
                sc[j] = half2_t{s, s};
            }
        };

        auto compute = [&](int stage) {
            const uint8_t* base = smem + stage * STAGE_BYTES;
            uintx4 wq[TN];
#pragma unroll
            for (int j = 0; j < TN; ++j)
                wq[j] = *reinterpret_cast<const uintx4*>(base + w_frag[j]);
#pragma unroll
            for (int s = 0; s < 4; ++s)
            {
                half8_t af[TM];
#pragma unroll
                for (int i = 0; i < TM; ++i)
                    af[i] = *reinterpret_cast<const half8_t*>(base + a_frag[i] + ((((h << 2) + s) ^ a_swz[i]) << 4));
#pragma unroll
                for (int j = 0; j < TN; ++j)
                {
                    const uint32_t w = (s == 0) ? wq[j].x : (s == 1) ? wq[j].y : (s == 2) ? wq[j].z : wq[j].w;
                    uint32_t bw[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                    {
                        uint32_t x = __builtin_amdgcn_perm(w, w, SEL[e]);        // bytes (b_e, 0, b_e, 0)
                        half2_t y = as_half2((x & MASK) | MAGIC);                // (1024 + q_2e, 1024 + 16 q_2e+1)
                        half2_t z = __builtin_elementwise_fma(y, dq_mul, dq_add); // (q_2e - zp, q_2e+1 - zp)
                        bw[e] = as_u32(z * sc[j]);
                    }
                    half8_t bf = __builtin_bit_cast(half8_t, uintx4{bw[0], bw[1], bw[2], bw[3]});
#pragma unroll
                    for (int i = 0; i < TM; ++i)
                        {
                            // fp16 results are written by rows (D[n][m]: four consecutive columns per lane);
                            // partial sums by columns (D[m][n]: 32 consecutive columns per store)
                            if (SPLITK)
                                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf, acc[i][j], 0, 0, 0);
                            else
                                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf, af[i], acc[i][j], 0, 0, 0);
                        }
                }
            }
        };

        // ---- K loop: stages kt % 3; loads run two K steps ahead -------------------------------------------
        load_scales(0);
        issue_tile_loads(0, 0);
        issue_tile_loads(1, 1);
        // Vector-memory operations complete in order.  Before the barrier of step kt a wavefront waits
        // until at most the operations it issued during step kt-1 are outstanding: then its own loads
        // for step kt (issued during step kt-2) have landed.  Even steps issue the scale loads (TN) and a
        // tile (TILE_LOADS), odd steps a tile only.
        int stage = 0;
        for (int kt = 0; kt < KT; kt += 2)
        {
            // even step
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(TILE_LOADS));
            __builtin_amdgcn_s_barrier();
            take_scales(kt >> 1);
            load_scales((kt >> 1) + 1);
            {
                const int nk = min(kt + 2, KT - 1); // past the end: reload a valid tile into the free stage
                int st = stage + 2;
                st = st >= STAGES ? st - STAGES : st;
                issue_tile_loads(nk, st);
            }
            compute(stage);
            stage = stage + 1 == STAGES ? 0 : stage + 1;
            // odd step
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(TILE_LOADS + TN));
            __builtin_amdgcn_s_barrier();
            {
                const int nk = min(kt + 3, KT - 1);
                int st = stage + 2;
                st = st >= STAGES ? st - STAGES : st;
                issue_tile_loads(nk, st);
            }
            compute(stage);
            stage = stage + 1 == STAGES ? 0 : stage + 1;
        }
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(0)); // drain the tail loads before the LDS goes away

        // ---- epilogue ---------------------------------------------------------------------------------
        const int m_wave = m0 + wm * (TM * 32);
        if (SPLITK)
        {
            // fp32 partial sums straight from the registers.  Here the activation fragment is the MFMA's first
            // operand: D[m][n], lane (n = l32, h), element e: row m = 8*(e/4) + 4*h + (e%4), so a store covers
            // 32 consecutive columns (128 bytes) of two rows.
            float* part = p.partial + (size_t)split * p.M * p.ld_partial;
#pragma unroll
            for (int j = 0; j < TN; ++j)
            {
                const int n = GATE ? n0 + wn * 32 + l32 : n0 + wn * (TN * 32) + j * 32 + l32;
                if (n >= p.N)
                    continue;
                const int pc = (GATE && j == 1) ? p.N + n : n; // up columns follow the N gate columns
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int e = 0; e < 16; ++e)
                    {
                        const int m = m_wave + i * 32 + 8 * (e >> 2) + 4 * h + (e & 3);
                        if (m < p.M)
                            part[(size_t)m * p.ld_partial + pc] = acc[i][j][e];
                    }
            }
            return;
        }
        // fp16 results.  The weight fragment is the MFMA's first operand, so a 32x32 result is D[n][m]: lane
        // (m = l32, h) holds, in element e, column n = 8*(e/4) + 4*h + (e%4) of its weight tile: four
        // consecutive columns per group of four elements.  They are rounded (GATE: combined) in registers,
        // turned through a private piece of LDS (the
        // ring is free after the barrier) and finished as whole rows of the wavefront's sub-tile, 16 bytes
        // (8 columns) per lane: bias, residual and the store.
        constexpr int OUT_TN = GATE ? 1 : TN;
        constexpr int ROUND_TM = TM >= 2 ? 2 : 1;      // 32-row blocks per pass through LDS
        constexpr int PITCH = OUT_TN * 64 + 16;        // bytes per staged row (padding spreads the banks)
        constexpr int REGION = ROUND_TM * 32 * PITCH;
        static_assert(8 * REGION <= T::LDS_BYTES, "the staging regions reuse the ring");
        constexpr int LANES_PER_ROW = OUT_TN * 4, ROWS_PER_READ = 64 / LANES_PER_ROW;
        __builtin_amdgcn_s_barrier(); // every wavefront has read its last fragments
        uint8_t* region = smem + wave * REGION;
        const int n_wave = GATE ? n0 + wn * 32 : n0 + wn * (TN * 32);
        const int piece = lane % LANES_PER_ROW;
        const int n_lane = n_wave + piece * 8; // first of this lane's 8 columns in the row phase
        bool vec = ((p.N & 7) == 0) && ((p.ldy & 7) == 0) && ((reinterpret_cast<uintptr_t>(p.Y) & 15) == 0);
        if (RESID)
            vec = vec && ((reinterpret_cast<uintptr_t>(p.residual) & 15) == 0);
        float bias[8];
        if (BIAS)
        {
#pragma unroll
            for (int k = 0; k < 8; ++k)
                bias[k] = (float)p.bias[min(n_lane + k, p.N - 1)];
        }
#pragma unroll
        for (int r = 0; r < TM / ROUND_TM; ++r)
        {
#pragma unroll
            for (int ii = 0; ii < ROUND_TM; ++ii)
            {
                const int i = r * ROUND_TM + ii;
#pragma unroll
                for (int j = 0; j < OUT_TN; ++j)
#pragma unroll
                    for (int g = 0; g < 4; ++g)
                    {
                        half4_t y;
#pragma unroll
                        for (int k = 0; k < 4; ++k)
                        {
                            if (GATE)
                            {
                                const float gt = (float)(half_t)acc[i][0][4 * g + k];
                                const float up = (float)(half_t)acc[i][1][4 * g + k];
                                y[k] = (half_t)(gt * (1.0f / (1.0f + __expf(-gt))) * up);
                            }
                            else
                            {
                                y[k] = (half_t)acc[i][j][4 * g + k];
                            }
                        }
                        *reinterpret_cast<half4_t*>(region + (ii * 32 + l32) * PITCH + (j * 32 + 8 * g + 4 * h) * 2) = y;
                    }
            }
            // LDS operations of one wavefront execute in order: no barrier around the private region
#pragma unroll
            for (int it = 0; it < ROUND_TM * 32 / ROWS_PER_READ; ++it)
            {
                const int row = it * ROWS_PER_READ + lane / LANES_PER_ROW;
                half8_t v = *reinterpret_cast<const half8_t*>(region + row * PITCH + piece * 16);
                const int m = m_wave + r * (ROUND_TM * 32) + row;
                if (m >= p.M || n_lane >= p.N)
                    continue;
                const size_t at = (size_t)m * p.ldy + n_lane;
                if (BIAS)
                {
#pragma unroll
                    for (int k = 0; k < 8; ++k)
                        v[k] = (half_t)((float)v[k] + bias[k]);
                }
                if (RESID)
                {
                    half8_t res;
                    if (vec)
                        res = *reinterpret_cast<const half8_t*>(p.residual + at);
                    else
                        for (int k = 0; k < 8; ++k)
                            res[k] = p.residual[n_lane + k < p.N ? at + k : at];
#pragma unroll
                    for (int k = 0; k < 8; ++k)
                        v[k] = (half_t)((float)v[k] + (float)res[k]);
                }
                if (vec)
                    *reinterpret_cast<half8_t*>(p.Y + at) = v;
                else
                    for (int k = 0; k < 8; ++k)
                        if (n_lane + k < p.N)
                            p.Y[at + k] = v[k];
            }
        }
    }

    template <int WM, int WN, int TM, int TN, bool GATE, bool BIAS, bool RESID, bool SPLITK, int MINW>
    hipError_t launch_gemm_dl(hipStream_t stream, const GemmParams& p)
    {
        using T = gemm_dl::Tile<WM, WN, TM, TN>;
        constexpr int BN_OUT = GATE ? T::BN / 2 : T::BN;
        const int tiles_m = (p.M + T::BM - 1) / T::BM;
        const int tiles_n = (p.N + BN_OUT - 1) / BN_OUT;
        auto kernel = &w4a16_gemm_dl_kernel<WM, WN, TM, TN, GATE, BIAS, RESID, SPLITK, MINW>;
        if (T::LDS_BYTES > 64 * 1024)
        {
            static bool attr_set = false;
            if (!attr_set)
            {
                hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, T::LDS_BYTES);
                if (e != hipSuccess)
                    return e;
                attr_set = true;
            }
        }
        const int splits = SPLITK ? p.splits : 1;
        hipLaunchKernelGGL(kernel, dim3(tiles_m * tiles_n * splits), dim3(gemm_dl::THREADS), T::LDS_BYTES, stream, p);
        return hipGetLastError();
    }

    // tile shapes (WM, WN, TM, TN) behind launch_w4a16_gemm
    //   big   256 x 256 (GATE: 256 x (128 + 128))    one workgroup per CU
    //   mid   128 x 128 (GATE: 128 x (128 + 128))    two per CU
    //   small  64 x 256 (GATE:  64 x (256 + 256))    two per CU
    //   tiny   32 x 256 (GATE:  32 x (256 + 256))    two per CU
    hipError_t launch_gemm_mid(hipStream_t stream, const GemmParams& p, bool gate, bool has_bias, bool has_resid);
    hipError_t launch_gemm_small(hipStream_t stream, const GemmParams& p, bool gate, bool has_bias, bool has_resid);
    hipError_t launch_gemm_tiny(hipStream_t stream, const GemmParams& p, bool gate, bool has_bias, bool has_resid);
} // namespace nnf
