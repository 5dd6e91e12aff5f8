// W8A8 for M > 16: int8 x int8 -> int32 GEMM on v_mfma_i32_32x32x32_i8, exact accumulators.
//
//   acc[M,N] = A[M,K] . W[N,K]^T  (int32, bit exact);  Y = fp16((float)acc * s_tok[m] * s_ch[n])
//
// Nothing in the reference computes this on a GPU; the nearest is MLAS's u8 x s8 MlasGemm
// (thirdparty/mlas/inc/mlas.h:147-163).
//
// Same skeleton as the fp16 x int4 GEMM: eight wavefronts (WM x WN) over a BM x BN tile, operands
// global -> LDS by asynchronous 1 KiB wavefront loads into a ring of stages (loads run STAGES-1 K steps
// ahead, one barrier per K step), tiles numbered so that an XCD works on a compact block of the output,
// optional split of K with int32 partial sums (added exactly by a reduction pass).  Both operands are
// K-contiguous int8 and need no unpacking: a K step is 64 bytes of every row, a lane's MFMA operand is
// 16 consecutive bytes (K index in the step = 32*s + 16*h + e), and the 16-byte pieces of a 64-byte row
// are XOR-swizzled with bits 2..3 of the row so that the 128-bit fragment reads are conflict free.
#include "nnf_device.h"
#include "nnf_launch.h"

#include "../nnf_workspace.h"

namespace nnf
{
    struct Q8GemmParams
    {
        const int8_t* A;
        const int8_t* W;
        const float* s_tok;
        const float* s_ch;
        half_t* Y;       // fp16 output, or
        int32_t* acc;    // raw accumulators (RAW)
        int32_t* partial; // SPLITK: [splits][M][N]
        int M, N, K, splits;
    };

    namespace q8dl
    {
        // BK: bytes (= int8 elements) of K per step, 64 or 128.  With 128 a wavefront-wide load fetches whole 128-byte
        // lines (8 rows); with 64 it fetches half of each of 16 lines, and the memory pipeline takes about as long over a
        // line it fetches half of as over a whole one.
        template <int WM, int WN, int TM, int TN, int STAGES_, int BK_ = 64>
        struct Tile
        {
            static constexpr int BK = BK_;
            static_assert(BK == 64 || BK == 128, "a K step is half a line or a line of every row");
            static constexpr int NSUB = BK / 32;          // sub-steps (one MFMA deep) per K step
            static constexpr int ROWS_PER_LOAD = 1024 / BK; // rows a wavefront-wide load covers
            static constexpr int WAVES = WM * WN;
            static_assert(WAVES == 8 || WAVES == 4, "eight wavefronts per workgroup, or four with one SIMD each");
            static constexpr int THREADS = WAVES * 64;
            static constexpr int STAGES = STAGES_;
            static constexpr int BM = WM * TM * 32;
            static constexpr int BN = WN * TN * 32;
            static constexpr int A_TILE_BYTES = BM * BK;
            static constexpr int W_TILE_BYTES = BN * BK;
            static constexpr int STAGE_BYTES = A_TILE_BYTES + W_TILE_BYTES;
            static constexpr int LDS_BYTES = STAGES * STAGE_BYTES;
            // a wavefront-wide load covers 16 rows of 64 bytes or 8 of 128; every wavefront issues the same number of loads
            // (with fewer chunks than wavefronts two wavefronts fetch the same chunk into the same place)
            static constexpr int A_CHUNKS = BM / ROWS_PER_LOAD;
            static constexpr int W_CHUNKS = BN / ROWS_PER_LOAD;
            static constexpr int A_LOADS = A_CHUNKS >= WAVES ? A_CHUNKS / WAVES : 1;
            static constexpr int W_LOADS = W_CHUNKS >= WAVES ? W_CHUNKS / WAVES : 1;
            static constexpr int TILE_LOADS = A_LOADS + W_LOADS;
        };

        constexpr int vmcnt_imm(int n) { return (n & 0xF) | ((n >> 4) << 14) | (0x7 << 4) | (0xF << 8); }
    } // namespace q8dl

    template <int WM, int WN, int TM, int TN, int STAGES, bool RAW, bool SPLITK, int MINW, int BK = 64>
    __global__ __launch_bounds__(WM * WN * 64, MINW) void w8a8_gemm_dl_kernel(const int8_t* __restrict__ A_first,
                                                                              const int8_t* __restrict__ W_first, int M_first,
                                                                              int N_first, int K_first, int splits_first,
                                                                              Q8GemmParams p_rest)
    {
        // (what the first loads need, once more as arguments of their own: scalar arguments arrive in registers with the
        // wavefront, a structure passed by value is loaded from memory -- the kernel began by waiting for it)
        Q8GemmParams p = p_rest;
        p.A = A_first;
        p.W = W_first;
        p.M = M_first;
        p.N = N_first;
        p.K = K_first;
        p.splits = splits_first;
        using namespace q8dl;
        using T = Tile<WM, WN, TM, TN, STAGES, BK>;
        constexpr int BM = T::BM, BN = T::BN, NSUB = T::NSUB, RPL = T::ROWS_PER_LOAD;
        constexpr int PIECES = BK / 16; // 16-byte pieces of a row of a stage
        // the piece a row's data sits at is XORed with bits of the row so that the 128-bit fragment reads are conflict free
        auto swizzle = [](int row) { return BK == 64 ? (row >> 2) & 3 : (row >> 1) & 7; };
        constexpr int A_LOADS = T::A_LOADS, W_LOADS = T::W_LOADS, TILE_LOADS = T::TILE_LOADS;
        constexpr int A_TILE_BYTES = T::A_TILE_BYTES, STAGE_BYTES = T::STAGE_BYTES;
        extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int wm = wave / WN, wn = wave % WN;
        const int l32 = lane & 31, h = lane >> 5;
        const int K = p.K;
        const int G = K >> 7;

        const int tiles_m = (p.M + BM - 1) / BM;
        const int tiles_n = (p.N + BN - 1) / BN;
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
        const int m0 = tm * BM, n0 = tn * BN;

        // this workgroup's K range, in units of 128 (all of K without SPLITK)
        const int g_begin = SPLITK ? (int)(((long long)split * G) / p.splits) : 0;
        const int g_end = SPLITK ? (int)(((long long)(split + 1) * G) / p.splits) : G;
        const int KT = (128 / BK) * (g_end - g_begin);
        const int k_begin = g_begin * 128;

        // ---- direct-load maps: chunk c fills LDS rows c*16 .. +15 (64 B each; 128 B: c*8 .. +7); lane l lands at
        // (row = c*16 + l/4, slot = l%4) and therefore fetches piece  slot ^ swizzle(row)  of that row
        const int8_t* a_src[A_LOADS];
        int a_chunk[A_LOADS];
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i)
        {
            a_chunk[i] = (wave * A_LOADS + i) % T::A_CHUNKS;
            int row = a_chunk[i] * RPL + lane / PIECES;
            int piece = (lane % PIECES) ^ swizzle(row);
            a_src[i] = p.A + (size_t)min(m0 + row, p.M - 1) * K + k_begin + piece * 16;
        }
        const int8_t* w_src[W_LOADS];
        int w_chunk[W_LOADS];
#pragma unroll
        for (int i = 0; i < W_LOADS; ++i)
        {
            w_chunk[i] = (wave * W_LOADS + i) % T::W_CHUNKS;
            int row = w_chunk[i] * RPL + lane / PIECES;
            int piece = (lane % PIECES) ^ swizzle(row);
            w_src[i] = p.W + (size_t)min(n0 + row, p.N - 1) * K + k_begin + piece * 16;
        }
        auto issue_tile_loads = [&](int kt, int stage) {
            uint8_t* base = smem + stage * STAGE_BYTES;
            const int k0 = kt * BK;
#pragma unroll
            for (int i = 0; i < A_LOADS; ++i)
                __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)(a_src[i] + k0),
                                                 (void __attribute__((address_space(3)))*)(base + a_chunk[i] * 1024), 16, 0,
                                                 0);
#pragma unroll
            for (int i = 0; i < W_LOADS; ++i)
                __builtin_amdgcn_global_load_lds(
                    (const void __attribute__((address_space(1)))*)(w_src[i] + k0),
                    (void __attribute__((address_space(3)))*)(base + A_TILE_BYTES + w_chunk[i] * 1024), 16, 0, 0);
        };

        // ---- per-lane fragment addresses in LDS ------------------------------------------------------
        int a_frag[TM], a_swz[TM], w_frag[TN], w_swz[TN];
#pragma unroll
        for (int i = 0; i < TM; ++i)
        {
            int r = wm * (TM * 32) + i * 32 + l32;
            a_frag[i] = r * BK;
            a_swz[i] = swizzle(r);
        }
#pragma unroll
        for (int j = 0; j < TN; ++j)
        {
            int r = wn * (TN * 32) + j * 32 + l32;
            w_frag[j] = A_TILE_BYTES + r * BK;
            w_swz[j] = swizzle(r);
        }

        intx16 acc[TM][TN];
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    acc[i][j][e] = 0;

        // A K step is NSUB sub-steps of 32 bytes; the fragments of a sub-step (TM + TN 128-bit reads) are
        // fetched from LDS while the MFMAs of the sub-step before it run, into the other of two register sets.
        // Row r of a fragment and row r + 32 share their swizzle: the reads of a set are one address per
        // operand plus constant offsets.
        intx4 af[2][TM], bf[2][TN];
        uint32_t a_addr[NSUB], w_addr[NSUB];
#pragma unroll
        for (int s = 0; s < NSUB; ++s)
        {
            const uint32_t piece = (uint32_t)(((2 * s + h) ^ swizzle(l32)) << 4);
            a_addr[s] = lds_address(smem) + (uint32_t)((wm * (TM * 32) + l32) * BK) + piece;
            w_addr[s] = lds_address(smem) + (uint32_t)((wn * (TN * 32) + l32) * BK) + piece;
        }
        constexpr int FRAG_READS = TM + TN;
        auto read_frags = [&](int stage, auto s_c, auto set_c) {
            constexpr int s = decltype(s_c)::value, set = decltype(set_c)::value;
            const uint32_t off = (uint32_t)(stage * STAGE_BYTES);
            const uint32_t aa = a_addr[s] + off, ww = w_addr[s] + off;
            unroll_for<0, TM>([&](auto i) { lds_read_b128_nowait<decltype(i)::value * 32 * BK>(af[set][i], aa); });
            unroll_for<0, TN>(
                [&](auto j) { lds_read_b128_nowait<A_TILE_BYTES + decltype(j)::value * 32 * BK>(bf[set][j], ww); });
        };
        // read x of a set: the TM activation fragments, then the TN weight fragments
        auto read_one_frag = [&](int stage, auto s_c, auto set_c, auto x_c) {
            constexpr int s = decltype(s_c)::value, set = decltype(set_c)::value, x = decltype(x_c)::value;
            const uint32_t off = (uint32_t)(stage * STAGE_BYTES);
            if constexpr (x < TM)
                lds_read_b128_nowait<x * 32 * BK>(af[set][x], a_addr[s] + off);
            else
                lds_read_b128_nowait<A_TILE_BYTES + (x - TM) * 32 * BK>(bf[set][x - TM], w_addr[s] + off);
        };
        // load x of a K step: the A_LOADS activation loads, then the W_LOADS weight loads
        auto issue_one_load = [&](int kt, int stage, auto x_c) {
            constexpr int x = decltype(x_c)::value;
            uint8_t* base = smem + stage * STAGE_BYTES;
            const int k0 = kt * BK;
            if constexpr (x < A_LOADS)
                __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)(a_src[x] + k0),
                                                 (void __attribute__((address_space(3)))*)(base + a_chunk[x] * 1024), 16, 0, 0);
            else
                __builtin_amdgcn_global_load_lds(
                    (const void __attribute__((address_space(1)))*)(w_src[x - A_LOADS] + k0),
                    (void __attribute__((address_space(3)))*)(base + A_TILE_BYTES + w_chunk[x - A_LOADS] * 1024), 16, 0, 0);
        };
        // the set is usable once at most `later` LDS reads issued after it are in flight
        auto wait_frags = [&](auto set_c, auto later_c) {
            constexpr int set = decltype(set_c)::value;
            lds_wait<decltype(later_c)::value>(af[set][0]);
            unroll_for<1, TM>([&](auto i) { lds_wait_also(af[set][i]); });
            unroll_for<0, TN>([&](auto j) { lds_wait_also(bf[set][j]); });
        };
        // MFMAs [FIRST, LAST) of a sub-step, numbered j * TM + i
        auto mfma_range = [&](auto set_c, auto first_c, auto last_c) {
            constexpr int set = decltype(set_c)::value;
            unroll_for<decltype(first_c)::value, decltype(last_c)::value>([&](auto x_c) {
                constexpr int j = decltype(x_c)::value / TM, i = decltype(x_c)::value % TM;
                if (RAW || SPLITK)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[set][i], bf[set][j], acc[i][j], 0, 0, 0);
                else
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[set][j], af[set][i], acc[i][j], 0, 0, 0);
            });
        };
        auto mfmas = [&](auto set_c) {
            constexpr int set = decltype(set_c)::value;
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int i = 0; i < TM; ++i)
                    {
                        // fp16 results are written by rows (D[n][m]: four consecutive columns per lane); int32
                        // results by columns (D[m][n]: 32 consecutive columns per store)
                        if (RAW || SPLITK)
                            acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[set][i], bf[set][j], acc[i][j], 0, 0, 0);
                        else
                            acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[set][j], af[set][i], acc[i][j], 0, 0, 0);
                    }
        };
        using I0 = std::integral_constant<int, 0>;
        using I1 = std::integral_constant<int, 1>;
        using NONE = std::integral_constant<int, 0>;
        using ONE_SET = std::integral_constant<int, FRAG_READS>;

        // ---- K loop: stage kt % STAGES; loads run STAGES-1 K steps ahead ------------------------------------
        // Vector-memory operations complete in order and every step issues TILE_LOADS of them.
        // AHEAD (four stages or more): the barrier of step kt also certifies stage kt+1 (at most the loads
        // issued during step kt-1 are outstanding), so the first fragments of step kt+1 are read during
        // step kt and no MFMA waits for LDS behind a barrier.  The stage refilled during step kt is the one
        // of step kt-1, whose last fragment reads every wavefront has waited for before its MFMAs of kt-1.
        constexpr bool AHEAD = STAGES >= 4;
        constexpr int WAIT_LOADS = AHEAD ? (STAGES - 3) * TILE_LOADS : (STAGES - 2) * TILE_LOADS;
#pragma unroll
        for (int s = 0; s < STAGES - 1; ++s)
            issue_tile_loads(min(s, KT - 1), s);
        int stage = 0;
        if (AHEAD)
        {
            __builtin_amdgcn_s_waitcnt(vmcnt_imm((STAGES - 2) * TILE_LOADS));
            __builtin_amdgcn_s_barrier();
            read_frags(0, I0{}, I0{});
        }
        constexpr int NM = TM * TN; // MFMAs per sub-step
        for (int kt = 0; kt < KT; ++kt)
        {
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(WAIT_LOADS));
            __builtin_amdgcn_s_barrier();
            if constexpr (AHEAD)
            {
                // The fragments of sub-step 0 were read during the step before: the first MFMA goes out right behind the
                // barrier, and everything else this step issues goes out one piece at a time between two MFMAs (it
                // executes while the matrix core works): the LDS reads of the next sub-step behind the first MFMAs of a
                // sub-step (behind those of the last one: the next step's sub-step 0), this step's loads behind the later
                // MFMAs of every sub-step but the last.
                constexpr int HALF = NM / 2;
                constexpr int LOAD_SLOTS = (NSUB - 1) * HALF; // MFMAs with loads behind them
                constexpr int RPM = (FRAG_READS + HALF - 1) / HALF, LPM = (TILE_LOADS + LOAD_SLOTS - 1) / LOAD_SLOTS;
                int st = stage + STAGES - 1;
                st = st >= STAGES ? st - STAGES : st;
                const int kt_load = min(kt + STAGES - 1, KT - 1);
                const int next_stage = stage + 1 == STAGES ? 0 : stage + 1;
                unroll_for<0, NSUB>([&](auto u_c) {
                    constexpr int U = decltype(u_c)::value;
                    using SET = std::integral_constant<int, U & 1>;
                    using OTHER = std::integral_constant<int, (U & 1) ^ 1>;
                    using NEXT_SUB = std::integral_constant<int, U + 1 < NSUB ? U + 1 : 0>;
                    wait_frags(SET{}, NONE{});
                    unroll_for<0, NM>([&](auto x_c) {
                        constexpr int x = decltype(x_c)::value;
                        __builtin_amdgcn_sched_barrier(0);
                        mfma_range(SET{}, x_c, std::integral_constant<int, x + 1>{});
                        __builtin_amdgcn_sched_barrier(0);
                        if constexpr (x < HALF) // (after the last step: a stage nobody uses any more)
                            unroll_for<x * RPM, (x + 1) * RPM < FRAG_READS ? (x + 1) * RPM : FRAG_READS>(
                                [&](auto r_c) { read_one_frag(U + 1 < NSUB ? stage : next_stage, NEXT_SUB{}, OTHER{}, r_c); });
                        else if constexpr (U + 1 < NSUB)
                        {
                            constexpr int SLOT = U * HALF + (x - HALF);
                            unroll_for<(SLOT * LPM < TILE_LOADS ? SLOT * LPM : TILE_LOADS), ((SLOT + 1) * LPM < TILE_LOADS ? (SLOT + 1) * LPM : TILE_LOADS)>(
                                [&](auto l_c) { issue_one_load(kt_load, st, l_c); });
                        }
                    });
                    __builtin_amdgcn_sched_barrier(0);
                });
                stage = next_stage;
            }
            else
            {
                // two or three stages: the fragments of a step are read behind its barrier (past the end: a valid tile is
                // reloaded into the free stage)
                int st = stage + STAGES - 1;
                st = st >= STAGES ? st - STAGES : st;
                issue_tile_loads(min(kt + STAGES - 1, KT - 1), st);
                read_frags(stage, I0{}, I0{});
                read_frags(stage, I1{}, I1{});
                unroll_for<0, NSUB>([&](auto u_c) {
                    constexpr int U = decltype(u_c)::value;
                    using SET = std::integral_constant<int, U & 1>;
                    // behind this sub-step's fragments: those of the next one
                    if constexpr (U + 1 < NSUB)
                        wait_frags(SET{}, ONE_SET{});
                    else
                        wait_frags(SET{}, NONE{});
                    __builtin_amdgcn_sched_barrier(0);
                    mfmas(SET{});
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (U + 2 < NSUB)
                        read_frags(stage, std::integral_constant<int, U + 2>{}, SET{});
                });
                stage = stage + 1 == STAGES ? 0 : stage + 1;
            }
        }
        if (AHEAD)
            wait_frags(I0{}, NONE{}); // the registers of the last, unused set are free only now
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(0)); // drain the tail loads before the LDS goes away

        // ---- epilogue -------------------------------------------------------------------------------------
        const int m_wave = m0 + wm * (TM * 32), n_wave = n0 + wn * (TN * 32);
        if (RAW || SPLITK)
        {
            // int32 results straight from the registers.  Here the activation fragment is the MFMA's first
            // operand: D[m][n], lane (n = l32, h), element e: row m = 8*(e/4) + 4*h + (e%4), so a store covers
            // 32 consecutive columns (128 bytes) of two rows.
            int32_t* out = SPLITK ? p.partial + (size_t)split * p.M * p.N : p.acc;
#pragma unroll
            for (int j = 0; j < TN; ++j)
            {
                const int n = n_wave + j * 32 + l32;
                if (n >= p.N)
                    continue;
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int e = 0; e < 16; ++e)
                    {
                        const int m = m_wave + i * 32 + 8 * (e >> 2) + 4 * h + (e & 3);
                        if (m < p.M)
                            out[(size_t)m * p.N + n] = acc[i][j][e];
                    }
            }
            return;
        }
        // fp16 results.  The weight fragment is the MFMA's first operand, so a 32x32 result is D[n][m]: lane
        // (m = l32, h) holds, in element e, column n = 8*(e/4) + 4*h + (e%4): four consecutive output columns
        // per group of four elements.  They are scaled in registers, turned through a private piece of LDS
        // (the ring is free after the barrier) and written as whole rows of the wavefront's sub-tile, 16
        // bytes per lane.
        constexpr int ROUND_TM = TM >= 2 ? 2 : 1;  // 32-row blocks per pass through LDS
        constexpr int PITCH = TN * 64 + 16;        // bytes per staged row (padding spreads the banks)
        constexpr int REGION = ROUND_TM * 32 * PITCH;
        static_assert(T::WAVES * REGION <= T::LDS_BYTES, "the staging regions reuse the ring");
        constexpr int LANES_PER_ROW = TN * 4, ROWS_PER_READ = 64 / LANES_PER_ROW;
        __builtin_amdgcn_s_barrier(); // every wavefront has read its last fragments
        uint8_t* region = smem + wave * REGION;
        const bool sch_vec = (reinterpret_cast<uintptr_t>(p.s_ch) & 15) == 0;
        const bool y_vec = ((p.N & 7) == 0) && ((reinterpret_cast<uintptr_t>(p.Y) & 15) == 0);
#pragma unroll
        for (int r = 0; r < TM / ROUND_TM; ++r)
        {
#pragma unroll
            for (int ii = 0; ii < ROUND_TM; ++ii)
            {
                const int i = r * ROUND_TM + ii;
                const float st = p.s_tok[min(m_wave + i * 32 + l32, p.M - 1)];
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int g = 0; g < 4; ++g)
                    {
                        const int n = n_wave + j * 32 + 8 * g + 4 * h;
                        float sch[4];
                        if (sch_vec && n + 3 < p.N)
                        {
                            const floatx4 v = *reinterpret_cast<const floatx4*>(p.s_ch + n);
                            sch[0] = v.x, sch[1] = v.y, sch[2] = v.z, sch[3] = v.w;
                        }
                        else
                        {
                            for (int k = 0; k < 4; ++k)
                                sch[k] = p.s_ch[min(n + k, p.N - 1)];
                        }
                        half4_t y;
#pragma unroll
                        for (int k = 0; k < 4; ++k)
                        {
                            const float t = (float)acc[i][j][4 * g + k] * st;
                            y[k] = f32_to_f16_two_step(t * sch[k]);
                        }
                        *reinterpret_cast<half4_t*>(region + (ii * 32 + l32) * PITCH + (j * 32 + 8 * g + 4 * h) * 2) = y;
                    }
            }
            // LDS operations of one wavefront execute in order: no barrier around the private region
#pragma unroll
            for (int it = 0; it < ROUND_TM * 32 / ROWS_PER_READ; ++it)
            {
                const int row = it * ROWS_PER_READ + lane / LANES_PER_ROW;
                const int piece = lane % LANES_PER_ROW;
                const uintx4 v = *reinterpret_cast<const uintx4*>(region + row * PITCH + piece * 16);
                const int m = m_wave + r * (ROUND_TM * 32) + row;
                const int n = n_wave + piece * 8;
                if (m >= p.M || n >= p.N)
                    continue;
                half_t* dst = p.Y + (size_t)m * p.N + n;
                if (y_vec)
                    *reinterpret_cast<uintx4*>(dst) = v;
                else
                {
                    const half8_t hv = __builtin_bit_cast(half8_t, v);
                    for (int k = 0; k < 8; ++k)
                        if (n + k < p.N)
                            dst[k] = hv[k];
                }
            }
        }
    }

    // acc[m, n] = sum_s partial[s][m][n] (exact), then the same epilogue; four columns per thread
    template <bool RAW>
    __global__ __launch_bounds__(256) void w8a8_splitk_reduce_kernel(Q8GemmParams p)
    {
        // grid: x over groups of four columns, y = row
        const int quads = (p.N + 3) >> 2;
        const int q = (int)blockIdx.x * 256 + (int)threadIdx.x;
        if (q >= quads)
            return;
        const int m = blockIdx.y;
        const int n = q * 4;
        const size_t plane = (size_t)p.M * p.N;
        const int32_t* src = p.partial + (size_t)m * p.N + n;
        const bool vec = (p.N & 3) == 0;
        int a[4] = {0, 0, 0, 0};
#pragma unroll 4
        for (int s = 0; s < p.splits; ++s)
        {
            const int32_t* ps = src + (size_t)s * plane;
            if (vec)
            {
                intx4 v = *reinterpret_cast<const intx4*>(ps);
                a[0] += v.x, a[1] += v.y, a[2] += v.z, a[3] += v.w;
            }
            else
            {
                for (int j = 0; j < 4; ++j)
                    if (n + j < p.N)
                        a[j] += ps[j];
            }
        }
        const float st = RAW ? 0.f : p.s_tok[m];
        for (int j = 0; j < 4 && n + j < p.N; ++j)
        {
            if (RAW)
                p.acc[(size_t)m * p.N + n + j] = a[j];
            else
            {
                float v = (float)a[j] * st;
                p.Y[(size_t)m * p.N + n + j] = f32_to_f16_two_step(v * p.s_ch[n + j]);
            }
        }
    }

    namespace
    {
        template <int WM, int WN, int TM, int TN, int STAGES, bool RAW, bool SPLITK, int MINW, int BK = 64>
        hipError_t launch_tile(hipStream_t stream, const Q8GemmParams& p)
        {
            using T = q8dl::Tile<WM, WN, TM, TN, STAGES, BK>;
            const int tiles_m = (p.M + T::BM - 1) / T::BM;
            const int tiles_n = (p.N + T::BN - 1) / T::BN;
            auto kernel = &w8a8_gemm_dl_kernel<WM, WN, TM, TN, STAGES, RAW, SPLITK, MINW, BK>;
            if (T::LDS_BYTES > 64 * 1024)
            {
                static LdsGrant granted;
                const hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), granted, T::LDS_BYTES);
                if (e != hipSuccess)
                    return e;
            }
            const int splits = SPLITK ? p.splits : 1;
            hipLaunchKernelGGL(kernel, dim3(tiles_m * tiles_n * splits), dim3(T::THREADS), T::LDS_BYTES, stream, p.A, p.W, p.M, p.N,
                               p.K, p.splits, p);
            return hipGetLastError();
        }

        template <bool RAW>
        hipError_t launch_plan(hipStream_t stream, const Q8GemmParams& p, const workspace::GemmPlan& plan)
        {
            hipError_t e;
            // K steps of 128 bytes (whole lines per load) wherever LDS holds three of them.  Measured against steps of
            // 64 with the same tiles, weights no cache holds: 64 x 256 tiles 5 - 18 % faster (M = 40 .. 64), 128 x 128
            // 10 - 17 % (M = 160 .. 512; one workgroup per CU with four stages against two with three), 256 x 128
            // 4 - 13 % (M = 640 .. 2048).  Not for the 256 x 256 tile, where only two such stages fit (M = 4096: 1.5 %
            // slower), nor for 128 x 128 tiles whose workgroups get less than 2560 of K (M = 128, N = K = 8192, four
            // ranges of 2048: 25.1 -> 27.4 us; two resident workgroups with short loops cover for each other).
            const bool long_k = p.K / (p.splits > 0 ? p.splits : 1) >= 2560;
            switch (plan.tile)
            {
            case workspace::GEMM_TILE_BIG: // 256 x 256, four stages of 64, one workgroup per CU
                if (!plan.reduce_pass)
                    return launch_tile<2, 4, 4, 2, 4, RAW, false, 2>(stream, p);
                e = launch_tile<2, 4, 4, 2, 4, RAW, true, 2>(stream, p);
                break;
            case workspace::GEMM_TILE_TALL: // 256 x 128, three stages of 128, one workgroup per CU
                if (!plan.reduce_pass)
                    return launch_tile<2, 4, 4, 1, 3, RAW, false, 2, 128>(stream, p);
                e = launch_tile<2, 4, 4, 1, 3, RAW, true, 2, 128>(stream, p);
                break;
            case workspace::GEMM_TILE_MID: // 128 x 128: four stages of 128, one workgroup per CU; or three of 64, two per CU
                if (long_k)
                {
                    if (!plan.reduce_pass)
                        return launch_tile<2, 4, 2, 1, 4, RAW, false, 2, 128>(stream, p);
                    e = launch_tile<2, 4, 2, 1, 4, RAW, true, 2, 128>(stream, p);
                    break;
                }
                if (!plan.reduce_pass)
                    return launch_tile<2, 4, 2, 1, 3, RAW, false, 4>(stream, p);
                e = launch_tile<2, 4, 2, 1, 3, RAW, true, 4>(stream, p);
                break;
            default: // 64 x 256, always through the partial sums: three stages of 128, one workgroup per CU
                e = launch_tile<1, 8, 2, 1, 3, RAW, true, 2, 128>(stream, p);
                break;
            }
            if (e != hipSuccess)
                return e;
            const int quads = (p.N + 3) >> 2;
            hipLaunchKernelGGL((w8a8_splitk_reduce_kernel<RAW>), dim3((unsigned)((quads + 255) / 256), (unsigned)p.M), dim3(256), 0,
                               stream, p);
            return hipGetLastError();
        }
    } // namespace

    hipError_t launch_w8a8_gemm(hipStream_t stream, const void* A, const void* s_tok, const void* W, const void* s_ch,
                                void* Y, void* acc, int M, int N, int K, void* partial_ws, const LaunchChoice& choice)
    {
        const int tile = workspace::w8a8_forced_tile(choice.tile_rows, choice.tile_cols);
        const workspace::GemmPlan plan = workspace::plan_w8a8_gemm(M, N, K, tile, choice.k_parts);
        if (plan.reduce_pass && !partial_ws)
            return hipErrorInvalidValue;
        Q8GemmParams p;
        p.A = (const int8_t*)A;
        p.W = (const int8_t*)W;
        p.s_tok = (const float*)s_tok;
        p.s_ch = (const float*)s_ch;
        p.Y = (half_t*)Y;
        p.acc = (int32_t*)acc;
        p.partial = (int32_t*)partial_ws;
        p.M = M;
        p.N = N;
        p.K = K;
        p.splits = plan.splits;
        return acc ? launch_plan<true>(stream, p, plan) : launch_plan<false>(stream, p, plan);
    }
} // namespace nnf
