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
//     permuted); with up to two groups per wavefront it is then kept in registers --
//     and from six rows on each wavefront loads its share straight from global memory into those
//     registers, in the MFMA operand layout (16 rows x 64 bytes per load), instead of the staging;
//   * nibbles are turned into fp16 with one v_and_or_b32 per pair: (q | 0x6400) = 1024 + q (0x6400 is
//     1024 with an ulp of 1), and a nibble four bits up gives (16 q | 0x5400) = 64 + q (0x5400 is 64
//     with an ulp of 1/16): both exact, and the activations are used as they are.  Instead of
//     subtracting the 1024 / 64 and the zero point from every weight, the constant part
//         corr[m, group] = (1024 + zp) * sum_even a + (64 + zp) * sum_odd a
//     is computed once per wavefront (one MFMA chain against a constant operand) and used as the
//     negative initial accumulator of each group.  Products are exact in fp32, the sum of a group
//     is of order 1e4 at fp32 precision, i.e. an absolute error of ~1e-3 on a group sum of order 50;
//   * the group scale multiplies the fp32 group sum (4 FMAs per group and lane);
//   * the partial tiles of the KS wavefronts meet in LDS (one LDS-only barrier per tile, so the
//     prefetched global loads stay in flight); results are parked in LDS and written after the last
//     tile's barrier, when no load is left to protect.
#include "nnf_device.h"
#include "nnf_launch.h"

#include "../nnf_workspace.h"

#include <algorithm>
#include <type_traits>

namespace nnf
{
    // LDS, in this order (A_REGS: the partial sums and the parked outputs reuse the space of the staged
    // activations, which are only needed until every wavefront has copied its share into registers):
    //   activations as 16-byte units  unit(m, c, kq, j) = m*(16 G + 1) + (c*4 + kq)*4 + j  holding
    //       the eight fp16  a[m][c*128 + kq*32 + j*8 + {0,4,1,5,2,6,3,7}]
    //       (a row of A is staged in memory order; the odd row stride keeps rows on different banks)
    //   ncorr    [G][16 m] fp32: constant part of every group sum, negated
    //   scales   sc[2][16 rows][G] fp16 (as in memory), each copy padded to 16 bytes
    //   red      [2][M][16 n][16] fp32 partial sums, the KS <= 16 wavefronts of one output side by side
    //            (slots of absent wavefronts stay zero)
    //   outb     [tiles of this workgroup][M][16] fp32
    // Group (chunk) index of wavefront w, pass h, slot c:  (h*KS + w)*CPS + c.
    //
    // KSPLIT: K is cut into ranges of K columns each (the kernel's K is the range length) handled by different
    // workgroups, for shapes whose M x K activations do not fit in LDS at once; workgroup b works on range
    // b % ksplits and writes fp32 partial sums [range][M][N], which the GEMM's reduction pass adds up.
    struct SkinnySplit
    {
        int ksplits;       // number of K ranges
        int lda;           // row stride of A (elements) = the full K
        int w_row_bytes;   // row stride of Wq (bytes)
        int s_row_groups;  // row stride of S (elements) = full K / 128
        int k_last;        // length of the last range (the kernel's K is the length of the others)
        float* partial;    // [ksplits][M][N]
    };

    // rows of activations from which a wavefront loads its own operand instead of staging all rows in LDS
    // (below it the sixteen-fold repetition of the few rows costs more than the staging)
    constexpr int SKINNY_DIRECT_MIN_ROWS = 6; // measured: equal at 4 rows, 3-10 % faster from 6 rows on

    // pack = M | zp << 8 | wavefronts per workgroup << 16 | direct << 24 (A_REGS: every wavefront loads its own
    // share of the activations straight into registers, no staging in LDS);  n_wg: workgroups per K range;  a workgroup's tiles:
    // tiles_q, one more for the first tiles_r workgroups (n_tiles = tiles_q * n_wg + tiles_r, divided on the host).
    // The first arguments are the ones the first loads need: they arrive preloaded in scalar registers.
    template <int CPS, bool A_REGS, int H, bool KSPLIT>
    __global__ __launch_bounds__(1024) void w4a16_skinny_kernel(const half_t* __restrict__ A,
                                                                const uint8_t* __restrict__ Wq,
                                                                const half_t* __restrict__ S,
                                                                half_t* __restrict__ Y,
                                                                int N, int K, int tiles_q, int tiles_r, int n_wg,
                                                                int pack, SkinnySplit sp)
    {
        static_assert(H == 1 || H == 2, "one or two passes over K");
        static_assert(!A_REGS || H == 1, "register-resident activations only with one pass");
        extern __shared__ uintx4 lds[];
        // volatile: the vector move must stay here, where every lane is active
        uint32_t MAGIC, MAGIC_HI, MASK_LO, MASK_HI;
        asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(MAGIC));
        asm volatile("v_mov_b32 %0, 0x54005400" : "=v"(MAGIC_HI));
        asm volatile("s_mov_b32 %0, 0x000F000F" : "=s"(MASK_LO));
        asm volatile("s_mov_b32 %0, 0x00F000F0" : "=s"(MASK_HI));
        // ---- up to the first loads: as few instructions as possible ----------------------------------------
        // Sixteen wavefronts share one scalar unit and four share a vector unit: every instruction ahead of the
        // weight loads is paid sixteen (four) times over before the workgroup's memory stream starts.  So: all
        // loads are  kernel-argument base + 32-bit offset  (the host checks that the offsets fit), a wavefront's
        // groups are consecutive (immediate offsets), and everything the loads do not need comes after them.
        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6); // in a scalar register, and what follows from it
        const int M = pack & 0xff, zp = (pack >> 8) & 0xff, KS = (pack >> 16) & 0xff;
        const bool direct = A_REGS && ((pack >> 24) & 1); // uniform over the grid
        const int n_threads = KS << 6;
        const int col = lane & 15; // n within the tile (B operand / D column), m for the A operand
        const int kq = lane >> 4;  // K quarter of the MFMA (A/B operands), row quad of D
        // this workgroup among those of its K range
        const int k_range = KSPLIT ? (int)blockIdx.x % sp.ksplits : 0;
        const int wg = KSPLIT ? (int)blockIdx.x / sp.ksplits : (int)blockIdx.x;
        const int lda = KSPLIT ? sp.lda : K;
        if (KSPLIT)
        {
            A += (size_t)k_range * K;
            Wq += (size_t)k_range * (K >> 1);
            S += (size_t)k_range * (K >> 7);
            if (k_range == sp.ksplits - 1)
                K = sp.k_last; // the last range may be shorter
        }
        const int G = K >> 7;
        const uint32_t row_bytes = KSPLIT ? (uint32_t)sp.w_row_bytes : (uint32_t)(K >> 1);
        const int s_row_groups = KSPLIT ? sp.s_row_groups : G;
        const int stride = n_wg;
        const int tile0 = wg; // the grid never exceeds the number of tiles (per K range)
        const int T = tiles_q + (wg < tiles_r ? 1 : 0);
        auto tile_at = [&](int k) { return tile0 + k * stride; };
        // A tile is 16 whole rows: the last tile of an N that is not a multiple of 16 is moved back to
        // rows N-16 .. N-1 (some rows are then computed twice, with identical results), so that no
        // address needs a per-lane clamp.
        auto row0_of = [&](int tile) { return __builtin_amdgcn_readfirstlane(min(tile * 16, N - 16)); };

        // Groups (chunks) of wavefront w in pass h: CPS consecutive ones from (h*KS + w)*CPS; where that runs past
        // the end of K the window is moved back to end at the last group, and the groups that then belong to
        // another wavefront are masked out at use (chunk_ok).
        int chunk_start[H], chunk_base[H];
        uint32_t w_voff[H];
#pragma unroll
        for (int h = 0; h < H; ++h)
        {
            chunk_start[h] = (h * KS + wave) * CPS;
            chunk_base[h] = min(chunk_start[h], G - CPS);
            w_voff[h] = (uint32_t)col * row_bytes + (uint32_t)kq * 16u + (uint32_t)chunk_base[h] * 64u;
        }
        // (real = false: every lane reads the first bytes of the matrix instead -- a load that costs next to
        // nothing, for a register set that will not be used, where a branch around the loads would cost more)
        auto load_w = [&](int tile, int h, uintx4* w, bool real = true) {
            const uint32_t off = real ? w_voff[h] + (uint32_t)row0_of(tile) * row_bytes : 0u;
#pragma unroll
            for (int c = 0; c < CPS; ++c)
                w[c] = *reinterpret_cast<const uintx4*>(Wq + (size_t)off + c * 64);
        };
        // scale block of a tile: 16 rows x G fp16, contiguous; thread t carries bytes [16t, 16t+16) of it
        // (threads beyond the block re-read its last 16 bytes)
        // (KSPLIT: the rows of the block are s_row_groups apart; a row's share is ceil(G / 8) 16-byte pieces, the
        // last of them moved back to end with the range, so that nothing is read past it)
        const int pieces = (G + 7) >> 3;
        const int sc_units = KSPLIT ? 16 * pieces : 2 * G; // 16-byte units of one scale copy
        const int sc_stride = KSPLIT ? pieces * 8 : G;     // fp16 per row of it
        uint32_t s_lane_off = (uint32_t)min(tid, sc_units - 1) * 16u;
        if (KSPLIT)
        {
            const int t = min(tid, sc_units - 1);
            s_lane_off = (uint32_t)(t / pieces) * (uint32_t)s_row_groups * 2u + (uint32_t)min((t % pieces) * 16, G * 2 - 16);
        }
        auto load_s = [&](int tile) -> uintx4 {
            const uint32_t off = s_lane_off + (uint32_t)row0_of(tile) * (uint32_t)s_row_groups * 2u;
            return *reinterpret_cast<const uintx4*>(reinterpret_cast<const uint8_t*>(S) + (size_t)off);
        };

        // ---- prologue loads ----------------------------------------------------------------------------
        // Row 0 of the activations (all of them for M = 1) and the scales of the first two tiles are
        // requested before the weights: they are small and shared by every workgroup (cache hits), loads
        // complete in order, and the barrier that publishes them in LDS should not have to wait for the
        // first weights, which come from HBM.
        constexpr int A_EARLY = H; // one pass: K <= 8192, a row of A is at most one 16-byte unit per thread
        const int row0_units = G * 16;
        // Every wavefront-wide load instruction occupies the CU's one address unit for the same time whether its
        // lanes fetch distinct data or not, so wavefronts without a share of the activations or of the scales
        // skip those loads (branches on wavefront-uniform conditions, ahead of the unconditional weight loads).
        uintx4 a_early[A_EARLY];
#pragma unroll
        for (int e = 0; e < A_EARLY; ++e)
            a_early[e] = uintx4{0u, 0u, 0u, 0u};
        // Through a pointer the compiler knows nothing about, and with a compiler-level memory barrier behind:
        // otherwise these loads are moved down into the block that uses them, behind the weights.
        typedef const uint8_t __attribute__((address_space(1))) * global_bytes_t;
        typedef const uintx4 __attribute__((address_space(1))) * global_units_t;
        global_bytes_t a_bytes = (global_bytes_t) reinterpret_cast<const uint8_t*>(A);
        asm volatile("" : "+s"(a_bytes));
        // direct: lane (m = col, kq) of a wavefront fetches the 64 bytes of row m that its MFMA operand holds of
        // each of the wavefront's groups (k = 32 kq .. 32 kq + 31 of the group); rows past M repeat row M-1
        // A_REGS: a wavefront's operand and its constants are kept in registers (16 + 4 VGPRs per group);
        // otherwise both are re-read from LDS for every tile
        uintx4 areg[A_REGS ? CPS : 1][4];
        floatx4 ncreg[A_REGS ? CPS : 1];
        if (A_REGS && direct)
        {
            const uint32_t a_off = (uint32_t)min(col, M - 1) * (uint32_t)lda * 2u + (uint32_t)chunk_base[0] * 256u + (uint32_t)kq * 64u;
#pragma unroll
            for (int c = 0; c < CPS; ++c)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    areg[A_REGS ? c : 0][j] = *(global_units_t)(a_bytes + (size_t)(a_off + c * 256 + j * 16));
            asm volatile("" ::: "memory");
        }
        if (!direct && wave * 64 < row0_units)
        {
#pragma unroll
            for (int e = 0; e < A_EARLY; ++e)
            {
                const uint32_t u = (uint32_t)min(tid + e * n_threads, row0_units - 1);
                a_early[e] = *(global_units_t)(a_bytes + (size_t)(u * 16u));
            }
            asm volatile("" ::: "memory");
        }
        // A load issued at the end of the prologue would be the newest one when the tile loop is entered,
        // and the loop's wait for the scale registers would then wait for every weight load in flight:
        // hence the second tile's scales here, and the second register set loaded without a branch.
        // Register set 0 / 1: H == 1: even / odd tiles;  H == 2: first / second pass of the current tile.
        uintx4 w0[CPS], w1[CPS], sreg = {0u, 0u, 0u, 0u}, sfirst = {0u, 0u, 0u, 0u};
        const int tile_second = tile_at(min(1, T - 1));
        if (wave * 64 < sc_units)
        {
            sfirst = load_s(tile0);
            sreg = load_s(tile_second);
        }
        load_w(tile0, 0, w0);
        if (H == 2)
            load_w(tile0, H - 1, w1);
        else
            load_w(tile_second, 0, w1, T > 1);
        __builtin_amdgcn_sched_barrier(0);

        // ---- everything else ---------------------------------------------------------------------------
        const int row_units = G * 16 + 1; // 16-byte units per staged row of A (one unit of padding)
        const int a_units = row_units * M;
        constexpr int KSP = 16; // partial-sum slots per output: a constant, so that the row stride below is an immediate
        const int red_copy = M * 16 * KSP;
        // 16-byte units of the first region: the staged activations, or (A_REGS) whichever is larger of them and
        // the partial sums + parked outputs of the tiles_q (+1) tiles of a workgroup
        const int tail_units = (2 * red_copy + (tiles_q + (tiles_r ? 1 : 0)) * M * 16 + 3) >> 2;
        const int first_units = A_REGS ? max(a_units, tail_units) : a_units;
        floatx4* nc_lds = reinterpret_cast<floatx4*>(lds + first_units); // [G][4 kq] x (4 m)
        uintx4* sc_lds = lds + first_units + G * 4;
        float* red = A_REGS ? reinterpret_cast<float*>(lds) : reinterpret_cast<float*>(sc_lds + 2 * sc_units); // [2][M][16][KSP]
        float* outb = red + 2 * red_copy;
        const int m_rd = min(col, M - 1); // rows >= M read a valid row; their D rows are never stored
        const bool s_loader = tid < sc_units;
        int chunk_of[H][CPS];
        int sc_of[H][CPS]; // where the scale of the group sits in a row of the LDS copy
        float s_mask[H][CPS];
#pragma unroll
        for (int h = 0; h < H; ++h)
#pragma unroll
            for (int c = 0; c < CPS; ++c)
            {
                chunk_of[h][c] = chunk_base[h] + c;
                s_mask[h][c] = chunk_of[h][c] >= chunk_start[h] ? 1.0f : 0.0f;
                sc_of[h][c] = chunk_of[h][c];
                if (KSPLIT && chunk_of[h][c] >= (pieces - 1) * 8) // in the piece that was moved back
                    sc_of[h][c] = (pieces - 1) * 8 + chunk_of[h][c] - (G - 8);
            }

        // ---- activations -> LDS ---------------------------------------------------------------------
        // Staged once per workgroup (one coalesced 16-byte load per thread and unit); every wavefront
        // loading its own operand straight from global memory would cost 8 load instructions per
        // wavefront, almost all of whose lanes are redundant.
        // The constant part of a group sum,
        //     corr[m, group] = (1024 + zp) * sum_even a + (64 + zp) * sum_odd a,
        // is accumulated on the way: the 16 units of a group sit in 16 consecutive lanes.
        const float ce = -(1024.0f + (float)zp);
        const float co = -(64.0f + (float)zp);
        auto stage_unit = [&](uintx4 a, int m, int u) {
            a = permute_a8(a);
            lds[m * row_units + u] = a;
            const half2_t x = as_half2(a.x), y = as_half2(a.y), z = as_half2(a.z), w = as_half2(a.w);
            float se = ((float)x.x + (float)x.y) + ((float)z.x + (float)z.y);
            float so = ((float)y.x + (float)y.y) + ((float)w.x + (float)w.y);
            float pc = row16_sum(ce * se + co * so);
            if ((u & 15) == 0)
                reinterpret_cast<float*>(nc_lds)[(u >> 4) * 16 + m] = pc;
        };
        if (!direct)
        {
#pragma unroll
            for (int e = 0; e < A_EARLY; ++e)
            {
                int u = tid + e * n_threads;
                if (u < row0_units)
                    stage_unit(a_early[e], 0, u);
            }
            // what the early loads did not cover of row 0 (very long rows only) ...
            for (int u = tid + A_EARLY * n_threads; u < row0_units; u += n_threads)
                stage_unit(*reinterpret_cast<const uintx4*>(A + u * 8), 0, u);
        }
        // ... and rows 1 .. M-1, as one index space over all threads with four loads in flight per thread: row by
        // row, each row would cost a full memory round trip of its own
        if (!direct)
        {
            const int rest = (M - 1) * row0_units;
            for (int v0 = tid; v0 < rest; v0 += 4 * n_threads)
            {
                uintx4 av[4];
                int am[4], au[4];
#pragma unroll
                for (int e = 0; e < 4; ++e)
                {
                    const int v = min(v0 + e * n_threads, rest - 1);
                    am[e] = 1 + v / row0_units;
                    au[e] = v - (am[e] - 1) * row0_units;
                    av[e] = *reinterpret_cast<const uintx4*>(A + (size_t)am[e] * lda + au[e] * 8);
                }
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (v0 + e * n_threads < rest)
                        stage_unit(av[e], am[e], au[e]);
            }
        }
        if (!A_REGS && KSP != KS)
            for (int i = tid; i < 2 * red_copy; i += n_threads)
                red[i] = 0.f;
        int a_unit[H][CPS];
#pragma unroll
        for (int h = 0; h < H; ++h)
#pragma unroll
            for (int c = 0; c < CPS; ++c)
                a_unit[h][c] = m_rd * row_units + chunk_of[h][c] * 16 + kq * 4;
        // scales of the first tile -> LDS copy 0
        if (s_loader)
            sc_lds[tid] = sfirst;
        lds_barrier();

        // A_REGS without direct loads: the operand and its constants are read from LDS once
        if (A_REGS && direct)
        {
            // the pair order of the nibble trick in registers; the constant part of a group sum is
            // a product with a constant vector: four MFMAs whose B operand is (ce, co, ce, co) for every column
            const half_t ceh = (half_t)ce, coh = (half_t)co; // -(1024 + zp) and -(64 + zp): exact in fp16
            const uint32_t ce2 = as_u32(half2_t{ceh, ceh}), co2 = as_u32(half2_t{coh, coh});
            const uintx4 cvec = {ce2, co2, ce2, co2};
#pragma unroll
            for (int c = 0; c < CPS; ++c)
            {
                floatx4 t = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int j = 0; j < 4; ++j)
                {
                    const uintx4 a = permute_a8(areg[A_REGS ? c : 0][j]);
                    areg[A_REGS ? c : 0][j] = a;
                    t = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a),
                                                               __builtin_bit_cast(half8_t, cvec), t, 0, 0, 0);
                }
                ncreg[A_REGS ? c : 0] = t;
            }
        }
        else if (A_REGS)
        {
#pragma unroll
            for (int c = 0; c < CPS; ++c)
            {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    areg[A_REGS ? c : 0][j] = lds[a_unit[0][c] + j];
                ncreg[A_REGS ? c : 0] = nc_lds[chunk_of[0][c] * 4 + kq];
            }
        }
        if (A_REGS)
        {
            // from here on the staging area holds the partial sums: wait until every wavefront has its copy
            lds_barrier();
            if (KSP != KS)
                for (int i = tid; i < 2 * red_copy; i += n_threads)
                    red[i] = 0.f;
        }
        auto a_op = [&](int h, int c, int j) -> uintx4 {
            if (A_REGS)
                return areg[A_REGS ? c : 0][j];
            return lds[a_unit[h][c] + j];
        };
        auto ncorr = [&](int h, int c) -> floatx4 {
            if (A_REGS)
                return ncreg[A_REGS ? c : 0];
            return nc_lds[chunk_of[h][c] * 4 + kq];
        };

        // (w & mask) | magic as a single v_and_or_b32: the instruction takes no 32-bit literal and only one
        // scalar operand, so the masks live in scalar registers and the magic number in a vector register
        // (MAGIC is set at the top of the kernel, with every lane active)

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
                floatx4 t = ncorr(h, c);
                const uint32_t ww[4] = {wt[c].x, wt[c].y, wt[c].z, wt[c].w};
#pragma unroll
                for (int j = 0; j < 4; ++j)
                {
                    uint32_t w = ww[j];
                    uint32_t w8 = w >> 8;
                    uintx4 b;
                    b.x = (w & MASK_LO) | MAGIC;  // 1024 + (q0, q4)
                    b.y = (w & MASK_HI) | MAGIC_HI; // 64 + (q1, q5)
                    b.z = (w8 & MASK_LO) | MAGIC; // 1024 + (q2, q6)
                    b.w = (w8 & MASK_HI) | MAGIC_HI; // 64 + (q3, q7)
                    t = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a_op(h, c, j)),
                                                               __builtin_bit_cast(half8_t, b), t, 0, 0, 0);
                }
                float s = (float)sc[col * sc_stride + sc_of[h][c]] * s_mask[h][c];
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
                          uintx4* w_free, auto last, int tile_cur) {
            {
                // The address is recomputed at every call (two instructions): kept across the unrolled
                // tail of the tile loop it would be spilled.
                int slot = (kq * 64 + col) * KSP + wave;
                asm volatile("" : "+v"(slot));
                float* rp = red + par * red_copy + slot;
                const float av[4] = {acc.x, acc.y, acc.z, acc.w};
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (kq * 4 + r < M)
                        rp[r * 16 * KSP] = av[r];
            }
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
            // Four lanes per output: each adds four of the KSP partial sums, then the quad is summed.
            // Except after the last tile the sums are parked in LDS: a global store inside the loop
            // would make later address arithmetic wait for it, and with it for every prefetched load
            // issued before it (one in-order counter covers both).
            // (a workgroup with fewer than M wavefronts takes several rounds; whole wavefronts stay together)
            for (int t = tid; t < M * 64; t += n_threads)
            {
                const int o = t >> 2, q = t & 3; // o = m*16 + n
                floatx4 p4 = {0.f, 0.f, 0.f, 0.f};
                p4 = *reinterpret_cast<const floatx4*>(red + par * red_copy + o * KSP + q * 4);
                float v = quad_sum((p4.x + p4.y) + (p4.z + p4.w));
                if (decltype(last)::value)
                {
                    const int n = row0_of(tile_cur) + (o & 15);
                    if (q == 0)
                    {
                        if (KSPLIT)
                            sp.partial[((size_t)k_range * M + (o >> 4)) * N + n] = v;
                        else
                            Y[(size_t)(o >> 4) * N + n] = (half_t)v;
                    }
                }
                else if (q == 0)
                {
                    outb[local_tile * M * 16 + o] = v;
                }
            }
            if (decltype(last)::value)
            {
                // the sums parked by earlier tiles (written before the barrier above)
                const int per_tile = M * 16;
                for (int i = tid; i < local_tile * per_tile; i += n_threads)
                {
                    int lt = i / per_tile;
                    int r = i - lt * per_tile;
                    int n = min((tile0 + lt * stride) * 16, N - 16) + (r & 15); // per lane: no scalar row0_of here
                    if (KSPLIT)
                        sp.partial[((size_t)k_range * M + (r >> 4)) * N + n] = outb[i];
                    else
                        Y[(size_t)(r >> 4) * N + n] = (half_t)outb[i];
                }
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
                finish(acc, 0, yes, yes, tile_at(k + 2), yes, tile_at(k + 2), 0, w0, no, 0);
                acc = compute(zero, w1, h0, 1);
                finish(acc, 1, yes, yes, tile_at(k + 3), yes, tile_at(k + 3), 0, w1, no, 0);
            }
            const int rest = T - k; // 1, 2 or 3
            if (rest == 3)
            {
                floatx4 acc = compute(zero, w0, h0, 0);
                finish(acc, 0, yes, yes, tile_at(k + 2), yes, tile_at(k + 2), 0, w0, no, 0);
                acc = compute(zero, w1, h0, 1);
                finish(acc, 1, yes, no, 0, no, 0, 0, w1, no, 0);
                acc = compute(zero, w0, h0, 0);
                finish(acc, 0, no, no, 0, no, 0, 0, w0, yes, tile_at(k + 2));
            }
            else if (rest == 2)
            {
                floatx4 acc = compute(zero, w0, h0, 0);
                finish(acc, 0, yes, no, 0, no, 0, 0, w0, no, 0);
                acc = compute(zero, w1, h0, 1);
                finish(acc, 1, no, no, 0, no, 0, 0, w1, yes, tile_at(k + 1));
            }
            else
            {
                floatx4 acc = compute(zero, w0, h0, 0);
                finish(acc, 0, no, no, 0, no, 0, 0, w0, yes, tile_at(k));
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
                finish(acc, k & 1, yes, yes, tile_at(k + 2), yes, tile_at(k + 1), H - 1, w1, no, 0);
            }
            if (T - k == 2)
            {
                floatx4 acc = compute(zero, w0, h0, k & 1);
                load_w(tile_at(k + 1), 0, w0);
                __builtin_amdgcn_sched_barrier(0);
                acc = compute(acc, w1, h1, k & 1);
                finish(acc, k & 1, yes, no, 0, yes, tile_at(k + 1), H - 1, w1, no, 0);
                ++k;
            }
            floatx4 acc = compute(zero, w0, h0, k & 1);
            acc = compute(acc, w1, h1, k & 1);
            finish(acc, k & 1, no, no, 0, no, 0, 0, w1, yes, tile_at(k));
        }
    }

    namespace
    {
        using workspace::SkinnyPlan;
        SkinnyPlan plan_skinny(int M, int K) { return workspace::plan_w4a16_skinny(M, K, 0); }

        // K: the length of a K range (all of K without KSPLIT)
        template <int CPS, bool A_REGS, int H, bool KSPLIT = false>
        hipError_t launch_cps(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M, int N,
                              int K, int zp, const SkinnyPlan& p, int num_cu, SkinnySplit sp = SkinnySplit())
        {
            const int n_tiles = (N + 15) / 16;
            const int ksplits = KSPLIT ? sp.ksplits : 1;
            // persistent workgroups: one per CU when it has >= 8 wavefronts, else two
            const int per_cu = p.ks >= 8 ? 1 : 2;
            // workgroups per K range
            int grid = std::min(n_tiles, std::max(1, num_cu * per_cu / ksplits));
            int tiles_per_wg = (n_tiles + grid - 1) / grid;
            size_t lds_total = p.lds((size_t)tiles_per_wg * M * 16 * 4);
            while (lds_total > MAX_LDS_BYTES && grid < n_tiles)
            {
                // a very large N: more, shorter workgroups so that the parked outputs fit
                grid = std::min(n_tiles, grid * 2);
                tiles_per_wg = (n_tiles + grid - 1) / grid;
                lds_total = p.lds((size_t)tiles_per_wg * M * 16 * 4);
            }
            if (lds_total > MAX_LDS_BYTES)
                return hipErrorInvalidValue;
            if (lds_total > 64 * 1024)
            {
                static LdsGrant granted;
                const hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(&w4a16_skinny_kernel<CPS, A_REGS, H, KSPLIT>),
                                                       granted, (int)MAX_LDS_BYTES);
                if (e != hipSuccess)
                    return e;
            }
            hipLaunchKernelGGL((w4a16_skinny_kernel<CPS, A_REGS, H, KSPLIT>), dim3(grid * ksplits), dim3(p.ks * 64), lds_total,
                               stream, (const half_t*)A, (const uint8_t*)Wq, (const half_t*)S, (half_t*)Y, N, K,
                               n_tiles / grid, n_tiles % grid, grid,
                               M | (zp << 8) | (p.ks << 16) | ((A_REGS && M >= SKINNY_DIRECT_MIN_ROWS) ? (1 << 24) : 0), sp);
            return hipGetLastError();
        }
    } // namespace

    bool w4a16_skinny_supported(int M, int N, int K)
    {
        return workspace::w4a16_skinny_fits(M, N, K, 0);
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

    int w4a16_skinny_ksplits(int M, int N, int K)
    {
        return workspace::w4a16_skinny_ksplits(M, N, K);
    }

    hipError_t launch_w4a16_skinny_split(hipStream_t stream, const void* A, const void* Wq, const void* S, float* partial,
                                         int M, int N, int K, int zp, int ksplits, int num_cu)
    {
        const int k_range = workspace::w4a16_skinny_split_range(M, N, K);
        if (k_range <= 0 || (K + k_range - 1) / k_range != ksplits)
            return hipErrorInvalidValue;
        SkinnyPlan p = workspace::plan_w4a16_skinny(M, k_range);
        SkinnySplit sp;
        sp.ksplits = ksplits;
        sp.lda = K;
        sp.w_row_bytes = K >> 1;
        sp.s_row_groups = K >> 7;
        sp.k_last = K - (ksplits - 1) * k_range;
        sp.partial = partial;
        switch (p.cps * 10 + p.h)
        {
        case 11: return launch_cps<1, true, 1, true>(stream, A, Wq, S, nullptr, M, N, k_range, zp, p, num_cu, sp);
        case 21: return launch_cps<2, true, 1, true>(stream, A, Wq, S, nullptr, M, N, k_range, zp, p, num_cu, sp);
        default: return hipErrorInvalidValue;
        }
    }
} // namespace nnf
