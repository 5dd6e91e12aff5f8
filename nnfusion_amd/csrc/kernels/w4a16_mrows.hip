// fp16 x int4 (g128) for 2 <= M <= 16 activation rows and K = 1024, 2048, ... 8192 (M <= 32 up to K = 4096): the
// memory pipeline of the
// row-streaming GEMV (w4a16_gemv_rows.hip) under the arithmetic of the M <= 16 MFMA kernel
// (w4a16_skinny.hip).
//
//   Y[M,N] = A[M,K] . ((Wq - zp) * S)^T
//
// Replaces the cublasHgemm call of cuda::Dot (src/nnfusion/core/kernels/cuda_gpu/kernels/dot.cpp:271-363) for a
// weight-quantized Dot node with a handful of activation rows.
//
//   * One workgroup of eight wavefronts per CU owns a contiguous run of 16-row weight tiles.  All eight work on
//     the same tile, in STEPS steps of 8 x GW groups of 128 along K; wavefront w owns GW groups of every step
//     (GW*64 bytes of a weight row), so that the workgroup's loads of a step cover the 16 rows without gaps.
//   * A wavefront's part of a step (16 rows x GW*64 bytes = GW KiB) goes global -> LDS without registers
//     (global_load_lds_dwordx4, 1 KiB per wavefront-wide load) into a private two-slot ring, together with its
//     16 x GW group scales (one 4-byte load per lane); the slot of the step after next is requested as soon as
//     the current one has been copied into registers.  Nothing but the wavefront's own loads feeds its MFMAs:
//     no barrier on the load path.  Two steps per tile (one tile in flight per wavefront) measured fastest.
//     The 16-byte pieces of a row are XOR-swizzled with the row number on the way (each lane chooses which
//     piece it fetches), so the 128-bit operand reads are conflict free.
//   * The activations never touch LDS: lane (m, kq) loads the 64 bytes of row m that its MFMA operand holds of
//     each of the wavefront's groups, once, and keeps them (16 VGPRs per group; hence K <= 8192), in the pair
//     order of the nibble trick; the constant part of a group sum is an MFMA against a
//     constant operand and becomes the (negative) initial accumulator of the group (see w4a16_skinny.hip).
//   * Per step: GW x 4 MFMAs (v_mfma_f32_16x16x32_f16, weights as the B operand) per wavefront, the group sum
//     times the group scale in fp32; per tile the eight partial 16 x 16 tiles meet in LDS (one LDS-only barrier,
//     two alternating buffers), 256 threads add them and park the sums in LDS; Y is written after the
//     last tile.  Every workgroup reads all of A (M x K x 2 bytes, from the L2): with 16 rows of K = 8192 that
//     is twice the bytes of its weights.
//   * LDS writes inside the tile loop are inline ds_write instructions: ahead of an LDS write that it can see,
//     the compiler waits for every LDS-bound load in flight.
#include "nnf_device.h"
#include "nnf_launch.h"

#include "../nnf_workspace.h"

namespace nnf
{
    namespace
    {
        constexpr int MR_WAVES = 8;
        typedef const void __attribute__((address_space(1))) * mr_global_ptr_t;
        typedef void __attribute__((address_space(3))) * mr_lds_ptr_t;
        // s_waitcnt with only the vector-memory counter set (gfx9 encoding: vmcnt = bits 3:0 and 15:14)
        constexpr int mr_vmcnt(int n) { return (n & 0xF) | ((n >> 4) << 14) | (0x7 << 4) | (0xF << 8); }
    } // namespace

    // ---- pieces shared by the two forms of the kernel ----------------------------------------------------------------
    // The activations of a wavefront as loaded -> the MFMA operand order of the nibble trick (pairs (a0,a4) (a1,a5)
    // (a2,a6) (a3,a7)), and per group the constant part of its sum (an MFMA against a
    // constant operand), negative, as the initial accumulator of the group.
    // areg[.][g][.] *= the RMSNorm weight of the same k (fp16 products, rounded once); gsrc: the lane's 64 bytes of
    // gamma for group g start at gsrc(g)
    template <int MB, int GA, class F>
    __device__ __forceinline__ void mrows_scale_a(uintx4 (&areg)[MB][GA][4], F&& gsrc)
    {
#pragma unroll
        for (int g = 0; g < GA; ++g)
        {
            const uintx4* gp = reinterpret_cast<const uintx4*>(gsrc(g));
#pragma unroll
            for (int j = 0; j < 4; ++j)
            {
                const uintx4 gm = gp[j];
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
                {
                    uintx4 a = areg[mb][g][j];
                    a.x = as_u32(as_half2(a.x) * as_half2(gm.x));
                    a.y = as_u32(as_half2(a.y) * as_half2(gm.y));
                    a.z = as_u32(as_half2(a.z) * as_half2(gm.z));
                    a.w = as_u32(as_half2(a.w) * as_half2(gm.w));
                    areg[mb][g][j] = a;
                }
            }
        }
    }

    // The workgroup's parked sums -> Y.  Plain: fp16 of the sum.  Fused (see GemvFusion in nnf_launch.h): the sums of
    // row m times rstd[m]; gate: tiles 2 i and 2 i + 1 of the workgroup are the gate and the up rows of its output tile
    // i; bias and residual.  t0: the workgroup's first output tile, T_out of them; N: output columns.
    // sum_sq ([8 wavefronts][MB x 16 rows], or null) and K: RMSNorm without a pass of its own (gamma, no rstd).
    template <bool FUSED, int MB>
    __device__ __forceinline__ void mrows_flush(const float* parked, half_t* __restrict__ Y, int t0, int T_out, int M, int N,
                                                int tid, const GemvFusionArgs& f, int gate, const float* sum_sq = nullptr, int K = 0)
    {
        for (int idx = tid; idx < T_out * M * 16; idx += 512)
        {
            const int n = idx & 15;
            const int im = idx >> 4;
            const int it = im / M, m = im - it * M;
            const int nn = min((t0 + it) * 16, N - 16) + n;
            // (the last tile of an N that is not a multiple of 16 was moved back over columns that the tile before it
            // owns: written once, so that a residual that is the output buffer itself is added once)
            if (nn < (t0 + it) * 16)
                continue;
            const size_t at = (size_t)m * N + nn;
            if (!FUSED)
                Y[at] = (half_t)parked[idx];
            else
            {
                float rs = f.rstd ? f.rstd[m] : 1.0f;
                if (sum_sq)
                {
                    float total = 0.f;
#pragma unroll
                    for (int w = 0; w < MR_WAVES; ++w)
                        total += sum_sq[w * (MB * 16) + m];
                    rs = 1.0f / __builtin_sqrtf(total / (float)K + f.rms_eps);
                }
                if (gate)
                    Y[at] = finish_silu_gate(parked[((2 * it) * M + m) * 16 + n] * rs, parked[((2 * it + 1) * M + m) * 16 + n] * rs);
                else
                    Y[at] = finish_bias_residual(parked[idx] * rs, f.bias, nn, f.residual, at);
            }
        }
    }

    template <int MB, int GA>
    __device__ __forceinline__ void mrows_prepare_a(uintx4 (&areg)[MB][GA][4], floatx4 (&ncorr)[MB][GA], int zp)
    {
        const half_t ceh = (half_t)(-(1024.0f + (float)zp)), coh = (half_t)(-(64.0f + (float)zp)); // exact
        const uint32_t ce2 = as_u32(half2_t{ceh, ceh}), co2 = as_u32(half2_t{coh, coh});
        const uintx4 cvec = {ce2, co2, ce2, co2};
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int g = 0; g < GA; ++g)
            {
                floatx4 t = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int j = 0; j < 4; ++j)
                {
                    const uintx4 a = permute_a8(areg[mb][g][j]);
                    areg[mb][g][j] = a;
                    t = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, cvec), t,
                                                               0, 0, 0);
                }
                ncorr[mb][g] = t;
            }
    }

    // One group of 128 along K: the lane's 16 bytes of weights (32 nibbles) against group ga of the activations,
    // the fp32 group sum times the group's scale onto acc.  MAGIC = 0x64006400 (1024 + q for a nibble in bits 0..3),
    // MAGIC_HI = 0x54005400 (64 + q for a nibble in bits 4..7), MASK_LO = 0x000F000F, MASK_HI = 0x00F000F0.
    template <int MB, int GA>
    __device__ __forceinline__ void mrows_group(floatx4 (&acc)[MB], const uintx4 (&areg)[MB][GA][4],
                                                const floatx4 (&ncorr)[MB][GA], int ga, uintx4 wv, float scale, uint32_t MAGIC,
                                                uint32_t MAGIC_HI, uint32_t MASK_LO, uint32_t MASK_HI)
    {
        floatx4 t[MB];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
            t[mb] = ncorr[mb][ga];
        const uint32_t ww[4] = {wv.x, wv.y, wv.z, wv.w};
#pragma unroll
        for (int j = 0; j < 4; ++j)
        {
            const uint32_t w = ww[j];
            const uint32_t w8 = w >> 8;
            uintx4 bq;
            bq.x = (w & MASK_LO) | MAGIC;  // 1024 + (q0, q4)
            bq.y = (w & MASK_HI) | MAGIC_HI; // 64 + (q1, q5)
            bq.z = (w8 & MASK_LO) | MAGIC; // 1024 + (q2, q6)
            bq.w = (w8 & MASK_HI) | MAGIC_HI; // 64 + (q3, q7)
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
                t[mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, areg[mb][ga][j]),
                                                               __builtin_bit_cast(half8_t, bq), t[mb], 0, 0, 0);
        }
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
        {
            acc[mb].x = __builtin_fmaf(t[mb].x, scale, acc[mb].x);
            acc[mb].y = __builtin_fmaf(t[mb].y, scale, acc[mb].y);
            acc[mb].z = __builtin_fmaf(t[mb].z, scale, acc[mb].z);
            acc[mb].w = __builtin_fmaf(t[mb].w, scale, acc[mb].w);
        }
    }

    // End of a tile: the partial 16 x 16 tiles of the eight wavefronts meet in LDS (red: [2][8][MB KiB], buffer
    // rbuf), MB x 256 outputs per tile are added by the 512 threads and parked: they add them and park the sums of tile `it` ([tile][M][16] fp32 at parked_addr).
    // D layout: lane (n = col, kq), element e: row m = 16 mb + 4 kq + e.
    template <int MB>
    __device__ __forceinline__ void mrows_reduce_park(const floatx4 (&acc)[MB], const uint8_t* red, uint32_t red_addr,
                                                      uint32_t parked_addr, int rbuf, int it, int M, int tid)
    {
        const int lane = tid & 63, col = lane & 15, kq = lane >> 4;
        // Hazard: the accumulators may come straight out of an MFMA, and a read of an MFMA's result needs wait states
        // after it (up to 19 for a 16-pass MFMA) that the compiler inserts only ahead of instructions it emits itself,
        // not ahead of inline assembly.  They are therefore part of the block that holds the stores: one block, which
        // reads every accumulator, so that no MFMA can be scheduled behind the wait states.
        static_assert(MB >= 1 && MB <= 4, "up to four blocks of 16 rows");
        const uint32_t at = red_addr + (uint32_t)(rbuf * MR_WAVES * MB * 1024);
#define NNF_PARK_WAIT "s_nop 15\n\ts_nop 3\n\t"
        if constexpr (MB == 1)
            asm volatile(NNF_PARK_WAIT "ds_write_b128 %0, %1" ::"v"(at), "v"(acc[0]) : "memory");
        else if constexpr (MB == 2)
            asm volatile(NNF_PARK_WAIT "ds_write_b128 %0, %1\n\tds_write_b128 %0, %2 offset:1024" ::"v"(at), "v"(acc[0]), "v"(acc[MB - 1])
                         : "memory");
        else if constexpr (MB == 3)
            asm volatile(NNF_PARK_WAIT "ds_write_b128 %0, %1\n\tds_write_b128 %0, %2 offset:1024\n\tds_write_b128 %0, %3 offset:2048" ::"v"(at),
                         "v"(acc[0]), "v"(acc[1]), "v"(acc[MB - 1])
                         : "memory");
        else
            asm volatile(NNF_PARK_WAIT "ds_write_b128 %0, %1\n\tds_write_b128 %0, %2 offset:1024\n\tds_write_b128 %0, %3 offset:2048\n\t"
                                       "ds_write_b128 %0, %4 offset:3072" ::"v"(at),
                         "v"(acc[0]), "v"(acc[1]), "v"(acc[2]), "v"(acc[MB - 1])
                         : "memory");
#undef NNF_PARK_WAIT
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        for (int o = tid; o < MB * 256; o += MR_WAVES * 64) // (o & 63 == lane)
        {
            const int mb = o >> 8, e = (o >> 6) & 3;
            const float* rp = reinterpret_cast<const float*>(red + rbuf * MR_WAVES * MB * 1024 + mb * 1024) + lane * 4 + e;
            float sum = 0.f;
#pragma unroll
            for (int w = 0; w < MR_WAVES; ++w)
                sum += rp[w * (MB * 256)];
            const int m = 16 * mb + 4 * kq + e;
            if (m < M)
            {
                const uint32_t at = parked_addr + (uint32_t)(((it * M + m) * 16 + col) * 4);
                asm volatile("ds_write_b32 %0, %1" ::"v"(at), "v"(sum) : "memory");
            }
        }
    }

    // K = GW * STEPS * 1024; MB = blocks of 16 activation rows (1 or 2).
    // LDS (bytes): weights [8 wavefronts][2 slots][GW KiB] | scales [8][2][256] | partial tiles [2][8][MB KiB] |
    //              parked sums [tiles of the workgroup][M][16] fp32
    // pack = M | zp << 8 | gate << 16;  a workgroup's output tiles: tiles_q, one more for the first tiles_r workgroups.
    // FUSED: the prologue / epilogue of `f`; gate != 0: N outputs from 2 N weight rows, the workgroup walks the gate and
    // the up tile of each of its output tiles in turn (twice the tiles).
    // STAGE: the activations through LDS as whole lines (row_block_fetch); otherwise straight into the registers
    template <int GW, int STEPS, int MB, bool FUSED, bool STAGE>
    __global__ __launch_bounds__(512) void w4a16_mrows_kernel(const half_t* __restrict__ A, const uint8_t* __restrict__ Wq,
                                                              const half_t* __restrict__ S, half_t* __restrict__ Y, int N,
                                                              int tiles_q, int tiles_r, int pack, GemvFusionArgs f)
    {
        static_assert(GW >= 1 && GW <= 8 && STEPS >= 1 && GW * STEPS <= 8, "K = GW * STEPS * 1024");
        static_assert(MB == 1 || (MB == 2 && GW * STEPS <= 4), "two blocks of rows: 32 VGPRs per group");
        constexpr int K = GW * STEPS * 1024, G = K / 128;
        constexpr int GAMMA_LOADS = (GW * STEPS + 3) / 4; // of the RMSNorm weight into LDS: 1 KiB, four groups, each
        constexpr int GA = GW * STEPS;         // groups of a wavefront
        constexpr int ROW_BYTES = K / 2;       // a weight row
        constexpr int SLICE = GW * 64;         // a wavefront's bytes of a weight row per step
        constexpr int SPAN = 8 * SLICE;        // bytes of a weight row that the workgroup covers per step
        constexpr int TILE_BYTES = 16 * SLICE; // = GW KiB: GW wavefront-wide loads
        constexpr int LT = GW + 1;             // loads per step and wavefront (weights + scales)
        constexpr int SC_LANES = (GW + 1) / 2; // 4-byte scale loads per row (odd GW: one half-word of a neighbour comes along)
        extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
        uint32_t MAGIC, MAGIC_HI, MASK_LO, MASK_HI;
        asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(MAGIC));
        asm volatile("v_mov_b32 %0, 0x54005400" : "=v"(MAGIC_HI));
        asm volatile("s_mov_b32 %0, 0x000F000F" : "=s"(MASK_LO));
        asm volatile("s_mov_b32 %0, 0x00F000F0" : "=s"(MASK_HI));

        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int col = lane & 15; // n within the tile (B operand / D column), m for the A operand
        const int kq = lane >> 4;  // K quarter of the MFMA operands, row quad of D
        // (gate rides in `pack`, among the arguments that arrive in scalar registers with the wavefront: as an argument of
        // its own behind `f` it was loaded from memory and waited for ahead of the first weight load)
        const int M = pack & 0xff, zp = (pack >> 8) & 0xff, gate = (pack >> 16) & 1;
        const int b = blockIdx.x;
        const int t0 = b * tiles_q + min(b, tiles_r);
        const int T_out = tiles_q + (b < tiles_r ? 1 : 0);
        const int T = (FUSED && gate) ? 2 * T_out : T_out; // weight tiles this workgroup walks
        // weight rows of the workgroup's tile i (the last tile of an N that is not a multiple of 16 is moved back to
        // rows N-16 .. N-1)
        auto row0_of = [&](int i) {
            if (FUSED && gate)
                return __builtin_amdgcn_readfirstlane(((i & 1) ? N : 0) + min((t0 + (i >> 1)) * 16, N - 16));
            return __builtin_amdgcn_readfirstlane(min((t0 + i) * 16, N - 16));
        };

        uint8_t* ring = smem + wave * (2 * TILE_BYTES);
        uint8_t* sc_ring = smem + MR_WAVES * 2 * TILE_BYTES + wave * 512;
        uint8_t* red = smem + MR_WAVES * 2 * TILE_BYTES + MR_WAVES * 512; // [2][8][1024]
        float* sum_sq = reinterpret_cast<float*>(red + 2 * MR_WAVES * MB * 1024); // [8][MB x 16]
        float* parked = sum_sq + MR_WAVES * MB * 16;

        // ---- what each lane fetches -------------------------------------------------------------------------
        // Load c of a tile fills bytes [c KiB, (c+1) KiB) of the slot; lane i lands at byte c*1024 + 16 i =
        // (row r, position q) of the [16][SLICE] image and fetches piece q ^ swz(r) of that row's slice.
        // swz: the rows whose slices start in the same 64-byte quarter of the 256-byte bank period get different
        // values: all 16 rows when SLICE is a multiple of 256, 8 when of 128, else 4.  The XOR stays inside an
        // aligned block of 16 / 8 / 4 pieces, which the slice is a multiple of.
        auto swz = [](int r) { return GW % 4 == 0 ? (r & 15) : GW % 2 == 0 ? (r >> 1) & 7 : (r >> 2) & 3; };
        uint32_t w_off[GW];
#pragma unroll
        for (int c = 0; c < GW; ++c)
        {
            const int pos = c * 1024 + 16 * lane;
            const int r = pos / SLICE, q = (pos % SLICE) >> 4;
            w_off[c] = (uint32_t)r * ROW_BYTES + (uint32_t)wave * SLICE + (uint32_t)((q ^ swz(r)) << 4);
        }
        // scales: lane l fetches 4 bytes (two groups) of row l / SC_LANES, from the 4-byte boundary at or below the
        // wavefront's first group (odd GW, odd wavefront: one group below it; sc_skip)
        const int s_row = min(lane / SC_LANES, 15);
        const uint32_t s_off = (uint32_t)s_row * (G * 2) +
                               (((uint32_t)wave * (GW * 2)) & ~3u) + (uint32_t)(lane % SC_LANES) * 4u;
        const int sc_skip = (wave * GW) & 1;

        // step st (0 .. STEPS-1) of tile `tile` into slot `slot`
        auto issue = [&](int tile, int st, int slot) {
            const uint32_t row0 = (uint32_t)row0_of(tile);
            const uint8_t* wsrc = Wq + (size_t)row0 * ROW_BYTES + st * SPAN;
#pragma unroll
            for (int c = 0; c < GW; ++c)
                __builtin_amdgcn_global_load_lds((mr_global_ptr_t)(wsrc + w_off[c]),
                                                 (mr_lds_ptr_t)(ring + slot * TILE_BYTES + c * 1024), 16, 0, 0);
            __builtin_amdgcn_global_load_lds((mr_global_ptr_t)(reinterpret_cast<const uint8_t*>(S) + (size_t)row0 * (G * 2) + st * (8 * GW * 2) + s_off),
                                             (mr_lds_ptr_t)(sc_ring + slot * 256), 4, 0, 0);
        };

        // ---- the first two tiles, then the activations: straight into the MFMA operand registers -----------------
        // (the activations are requested last: vector-memory operations complete in order and the compiler waits
        // for them where they are used, which then also covers the two tiles -- requested first, those tiles'
        // loads are not held back by anything)
        issue(0, 0, 0);
        issue(min(1 / STEPS, T - 1), 1 % STEPS, 1);
        // (through LDS as whole lines, see row_block_fetch: two blocks per wavefront, over what holds the partial tiles
        // and the parked sums later -- hence the barrier behind the last block)
        // (a few rows: a load touches few lines as it is -- the lanes of the rows that do not exist ask for the last row
        // again -- and the detour costs 0.3 - 0.5 us: straight into the registers)
        uintx4 areg[MB][GA][4];
        if constexpr (!STAGE)
        {
            const uint8_t* a_bytes = reinterpret_cast<const uint8_t*>(A);
            const uint32_t a_off = (uint32_t)min(col, M - 1) * (uint32_t)(K * 2) + (uint32_t)wave * (GW * 256) + (uint32_t)kq * 64u;
#pragma unroll
            for (int g = 0; g < GA; ++g)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    areg[0][g][j] = *reinterpret_cast<const uintx4*>(a_bytes + (size_t)(a_off + (g / GW) * (SPAN * 4) + (g % GW) * 256 + j * 16));
        }
        else
        {
            uint8_t* stage = red + wave * (2 * ROW_BLOCK_BYTES);
            constexpr int NP = MB * GA;
            auto fetch = [&](int p) {
                const int mb = p / GA, g = p % GA;
                row_block_fetch(reinterpret_cast<const uint8_t*>(A), (size_t)K * 2, mb * 16, M - 1,
                                (size_t)((g / GW) * (SPAN * 4) + wave * (GW * 256) + (g % GW) * 256), stage + (p & 1) * ROW_BLOCK_BYTES, lane);
            };
            fetch(0);
#pragma unroll
            for (int p = 0; p < NP; ++p)
            {
                if (p + 1 < NP)
                {
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // block p-1 has been read out of the half that is filled next
                    fetch(p + 1);
                    __builtin_amdgcn_s_waitcnt(vmcnt_only(4));
                }
                else if (FUSED && f.gamma)
                {
                    // The RMSNorm weight of the wavefront's k positions (GA x 256 bytes) follows the last block into the
                    // free half, one load per four groups: as sixteen 16-byte loads per lane straight into registers --
                    // the sixteen lanes of a column asking for the same bytes -- it took the load pipeline a microsecond
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
                    for (int i = 0; i < GAMMA_LOADS; ++i)
                    {
                        const int g = min(4 * i + (lane >> 4), GA - 1);
                        const uint8_t* src = reinterpret_cast<const uint8_t*>(f.gamma) + wave * (GW * 256) + (g / GW) * (SPAN * 4) +
                                             (g % GW) * 256 + (lane & 15) * 16;
                        __builtin_amdgcn_global_load_lds((mr_global_ptr_t)src, (mr_lds_ptr_t)(stage + (NP & 1) * ROW_BLOCK_BYTES + i * 1024),
                                                         16, 0, 0);
                    }
                    __builtin_amdgcn_s_waitcnt(vmcnt_only(GAMMA_LOADS));
                }
                else
                    __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    areg[p / GA][p % GA][j] = row_block_piece(stage + (p & 1) * ROW_BLOCK_BYTES, col, kq * 4 + j);
            }
        }
        // RMSNorm without a pass of its own: the wavefront's share of sum a^2 of every row, from the registers
        const bool own_rstd = FUSED && f.gamma && !f.rstd;
        float ss[MB];
        if (own_rstd)
        {
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
            {
                ss[mb] = 0.f;
#pragma unroll
                for (int g = 0; g < GA; ++g)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                    {
                        // (v_dot2_f32_f16: one instruction per pair; with conversions and multiplies of its own the sum took
                        // more than a microsecond of a SIMD's vector unit at 16 rows x 4096)
                        const uint32_t rr[4] = {areg[mb][g][j].x, areg[mb][g][j].y, areg[mb][g][j].z, areg[mb][g][j].w};
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            ss[mb] = dot2(as_half2(rr[i]), as_half2(rr[i]), ss[mb]);
                    }
                ss[mb] += __shfl_xor(ss[mb], 16, 64);
                ss[mb] += __shfl_xor(ss[mb], 32, 64);
            }
        }
        if constexpr (STAGE)
        {
            if (FUSED && f.gamma)
            {
                const uint8_t* gamma_block = red + wave * (2 * ROW_BLOCK_BYTES) + ((MB * GA) & 1) * ROW_BLOCK_BYTES;
                __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
                mrows_scale_a<MB, GA>(areg, [&](int g) { return gamma_block + g * 256 + kq * 64; });
            }
            // (the blocks lay over what holds the partial tiles, the sums of squares and the parked sums from here on)
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __syncthreads();
        }
        else if (FUSED && f.gamma)
            mrows_scale_a<MB, GA>(areg, [&](int g) {
                return reinterpret_cast<const uint8_t*>(f.gamma) + wave * (GW * 256) + kq * 64 + (g / GW) * (SPAN * 4) + (g % GW) * 256;
            });
        if (own_rstd && kq == 0)
        {
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
                sum_sq[wave * (MB * 16) + mb * 16 + col] = ss[mb];
        }
        floatx4 ncorr[MB][GA];
        mrows_prepare_a<MB, GA>(areg, ncorr, zp);

        // ---- tile loop ---------------------------------------------------------------------------------------
        // operand reads of a slot: lane (n = col, kq), group g: piece g*4 + kq of row n
        const uint32_t rd_base = (uint32_t)col * SLICE;
        const int rd_swz = swz(col);
        const uint32_t red_addr = lds_address(red) + (uint32_t)(wave * (MB * 1024) + lane * 16);
        const uint32_t parked_addr = lds_address(parked);
        int slot = 0; // step s of the workgroup sits in slot s & 1
        for (int it = 0; it < T; ++it)
        {
            floatx4 acc[MB];
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
                acc[mb] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int st = 0; st < STEPS; ++st)
            {
                // this step has landed when at most the next step's loads are outstanding
                __builtin_amdgcn_s_waitcnt(mr_vmcnt(LT));
                uintx4 wv[GW];
                float sv[GW];
                {
                    const uint8_t* sl = ring + slot * TILE_BYTES + rd_base;
                    const half_t* sc = reinterpret_cast<const half_t*>(sc_ring + slot * 256);
#pragma unroll
                    for (int g = 0; g < GW; ++g)
                    {
                        wv[g] = *reinterpret_cast<const uintx4*>(sl + (((g * 4 + kq) ^ rd_swz) << 4));
                        sv[g] = (float)sc[col * (SC_LANES * 2) + sc_skip + g];
                    }
                }
                // the slot has been read before it is refilled with the step after next (past the end: a valid
                // tile again, so that the wait count above holds for every step)
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                issue(min(it + (st + 2) / STEPS, T - 1), (st + 2) % STEPS, slot);
                slot ^= 1;
#pragma unroll
                for (int g = 0; g < GW; ++g)
                    mrows_group<MB, GA>(acc, areg, ncorr, st * GW + g, wv[g], sv[g], MAGIC, MAGIC_HI, MASK_LO, MASK_HI);
            }
            mrows_reduce_park<MB>(acc, red, red_addr, parked_addr, it & 1, it, M, tid);
        }
        __builtin_amdgcn_s_waitcnt(mr_vmcnt(0)); // the reloads past the end, before the LDS goes away
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        // ---- flush: parked sums -> Y -----------------------------------------------------------------------------
        mrows_flush<FUSED, MB>(parked, Y, t0, T_out, M, N, tid, f, gate, own_rstd ? sum_sq : nullptr, K);
    }

    // ---- other block parameters ------------------------------------------------------------------------------------
    // The same kernel for groups of 2^GSHIFT = 32 / 64 / 128 weights and (ZPT) a zero point per (row, group) from
    // `zps`, u8 [N, K / group / 2], even group in the low nibble; 2 <= M <= 16 MB, K = GW * 2048 (two steps per tile).
    // A lane's 16-byte piece of a weight row (32 weights) lies in one group whatever its size, but the four lanes that meet
    // in one MFMA column hold pieces of up to four groups: a scale cannot be applied to the MFMA's sum.  The weights
    // are therefore dequantised before the MFMA, as the tile GEMM does:  fp16((q - z) * s),  q - z exact (nibble trick
    // plus -(1024 + z) or -(64 + z), which is the same trick applied to z with the sign bit set), one rounding in the
    // product; the accumulators take the MFMA results as they are.
    // Per step a wavefront fetches, next to its weights, the SPR = GW * 128 / group scales of each of the 16 rows (4-byte
    // loads, NSL of them) and, ZPT, their zero points (one byte per lane, NZL loads; a byte load lands in a lane's four
    // bytes of LDS).
    // LDS (bytes): weights [8 wavefronts][2 slots][GW KiB] | scales and zero points [8][2][(NSL + NZL) x 256] |
    //              partial tiles [2][8][MB KiB] | parked sums [tiles of the workgroup][M][16] fp32
    // pack = M | zp << 8.
    template <int GW, int GSHIFT, bool ZPT, int MB>
    __global__ __launch_bounds__(512) void w4a16_mrows_q_kernel(const half_t* __restrict__ A, const uint8_t* __restrict__ Wq,
                                                                const half_t* __restrict__ S, half_t* __restrict__ Y,
                                                                const uint8_t* __restrict__ zps, int N, int tiles_q,
                                                                int tiles_r, int pack)
    {
        static_assert(GW == 1 || GW == 2 || GW == 4, "K = 2048, 4096, 8192");
        static_assert(GSHIFT >= 5 && GSHIFT <= 7 && ((GW << (7 - GSHIFT)) & 1) == 0, "whole words of scales, whole bytes of zero points");
        static_assert(MB == 1 || (MB == 2 && GW <= 2), "two blocks of rows: 32 VGPRs per group");
        constexpr int STEPS = 2;
        constexpr int K = GW * STEPS * 1024, G = K >> GSHIFT;
        constexpr int GA = GW * STEPS;         // groups of 128 of a wavefront
        constexpr int ROW_BYTES = K / 2;       // a weight row
        constexpr int SLICE = GW * 64;         // a wavefront's bytes of a weight row per step
        constexpr int SPAN = 8 * SLICE;        // bytes of a weight row that the workgroup covers per step
        constexpr int TILE_BYTES = 16 * SLICE; // = GW KiB: GW wavefront-wide loads
        constexpr int SPR = GW << (7 - GSHIFT); // scales per row, step and wavefront
        constexpr int WPR = SPR / 2;            // ... as 4-byte words = bytes of zero points
        constexpr int NSL = (16 * WPR + 63) / 64;
        constexpr int NZL = ZPT ? NSL : 0;
        constexpr int AUX = (NSL + NZL) * 256;
        constexpr int LT = GW + NSL + NZL;      // loads per step and wavefront
        extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
        uint32_t MAGIC, MAGIC_HI, MASK_LO, MASK_HI;
        asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(MAGIC));
        asm volatile("v_mov_b32 %0, 0x54005400" : "=v"(MAGIC_HI));
        asm volatile("s_mov_b32 %0, 0x000F000F" : "=s"(MASK_LO));
        asm volatile("s_mov_b32 %0, 0x00F000F0" : "=s"(MASK_HI));

        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int col = lane & 15; // n within the tile (B operand / D column), m for the A operand
        const int kq = lane >> 4;  // K quarter of the MFMA operands, row quad of D
        const int M = pack & 0xff, zp = (pack >> 8) & 0xff;
        const int b = blockIdx.x;
        const int t0 = b * tiles_q + min(b, tiles_r);
        const int T = tiles_q + (b < tiles_r ? 1 : 0);
        auto row0_of = [&](int i) { return __builtin_amdgcn_readfirstlane(min((t0 + i) * 16, N - 16)); };

        uint8_t* ring = smem + wave * (2 * TILE_BYTES);
        uint8_t* aux = smem + MR_WAVES * 2 * TILE_BYTES + wave * (2 * AUX);
        uint8_t* red = smem + MR_WAVES * 2 * TILE_BYTES + MR_WAVES * 2 * AUX; // [2][8][1024]
        float* parked = reinterpret_cast<float*>(red + 2 * MR_WAVES * MB * 1024);

        // weights: as in w4a16_mrows_kernel
        auto swz = [](int r) { return GW % 4 == 0 ? (r & 15) : GW % 2 == 0 ? (r >> 1) & 7 : (r >> 2) & 3; };
        uint32_t w_off[GW];
#pragma unroll
        for (int c = 0; c < GW; ++c)
        {
            const int pos = c * 1024 + 16 * lane;
            const int r = pos / SLICE, q = (pos % SLICE) >> 4;
            w_off[c] = (uint32_t)r * ROW_BYTES + (uint32_t)wave * SLICE + (uint32_t)((q ^ swz(r)) << 4);
        }
        // scales: lane l of load i fetches word (64 i + l) % WPR of row (64 i + l) / WPR (lanes past the 16 rows: the
        // last row again); zero points: the same with bytes
        uint32_t s_off[NSL], z_off[NSL];
#pragma unroll
        for (int i = 0; i < NSL; ++i)
        {
            const int at = i * 64 + lane;
            const int r = min(at / WPR, 15), wd = at % WPR;
            s_off[i] = (uint32_t)r * (G * 2) + (uint32_t)wave * (SPR * 2) + (uint32_t)wd * 4u;
            z_off[i] = (uint32_t)r * (G / 2) + (uint32_t)wave * WPR + (uint32_t)wd;
        }

        // step st (0 .. 1) of tile `tile` into slot `slot`
        auto issue = [&](int tile, int st, int slot) {
            const uint32_t row0 = (uint32_t)row0_of(tile);
            const uint8_t* wsrc = Wq + (size_t)row0 * ROW_BYTES + st * SPAN;
#pragma unroll
            for (int c = 0; c < GW; ++c)
                __builtin_amdgcn_global_load_lds((mr_global_ptr_t)(wsrc + w_off[c]),
                                                 (mr_lds_ptr_t)(ring + slot * TILE_BYTES + c * 1024), 16, 0, 0);
            const uint8_t* ssrc = reinterpret_cast<const uint8_t*>(S) + (size_t)row0 * (G * 2) + st * (8 * SPR * 2);
#pragma unroll
            for (int i = 0; i < NSL; ++i)
                __builtin_amdgcn_global_load_lds((mr_global_ptr_t)(ssrc + s_off[i]), (mr_lds_ptr_t)(aux + slot * AUX + i * 256), 4, 0, 0);
            if constexpr (ZPT)
            {
                const uint8_t* zsrc = zps + (size_t)row0 * (G / 2) + st * (8 * WPR);
#pragma unroll
                for (int i = 0; i < NSL; ++i)
                    __builtin_amdgcn_global_load_lds((mr_global_ptr_t)(zsrc + z_off[i]),
                                                     (mr_lds_ptr_t)(aux + slot * AUX + (NSL + i) * 256), 1, 0, 0);
            }
        };

        issue(0, 0, 0);
        issue(0, 1, 1);
        // activations: into the MFMA operand registers (through LDS as whole lines from a few rows on, see
        // workspace::mrows_stages_activations), then in the pair order of the nibble trick
        uintx4 areg[MB][GA][4];
        if (MB == 1 && !workspace::mrows_stages_activations(M, K))
        {
            const uint8_t* a_bytes = reinterpret_cast<const uint8_t*>(A);
            const uint32_t a_off = (uint32_t)min(col, M - 1) * (uint32_t)(K * 2) + (uint32_t)wave * (GW * 256) + (uint32_t)kq * 64u;
#pragma unroll
            for (int g = 0; g < GA; ++g)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    areg[0][g][j] = *reinterpret_cast<const uintx4*>(a_bytes + (size_t)(a_off + (g / GW) * (SPAN * 4) + (g % GW) * 256 + j * 16));
        }
        else
        {
            uint8_t* stage = red + wave * (2 * ROW_BLOCK_BYTES);
            constexpr int NP = MB * GA;
            auto fetch = [&](int p) {
                const int mb = p / GA, g = p % GA;
                row_block_fetch(reinterpret_cast<const uint8_t*>(A), (size_t)K * 2, mb * 16, M - 1,
                                (size_t)((g / GW) * (SPAN * 4) + wave * (GW * 256) + (g % GW) * 256), stage + (p & 1) * ROW_BLOCK_BYTES, lane);
            };
            fetch(0);
#pragma unroll
            for (int p = 0; p < NP; ++p)
            {
                if (p + 1 < NP)
                {
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // block p-1 has been read out of the half that is filled next
                    fetch(p + 1);
                    __builtin_amdgcn_s_waitcnt(vmcnt_only(4));
                }
                else
                    __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    areg[p / GA][p % GA][j] = row_block_piece(stage + (p & 1) * ROW_BLOCK_BYTES, col, kq * 4 + j);
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __syncthreads();
        }
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int g = 0; g < GA; ++g)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    areg[mb][g][j] = permute_a8(areg[mb][g][j]);

        // ---- tile loop ---------------------------------------------------------------------------------------
        const uint32_t rd_base = (uint32_t)col * SLICE;
        const int rd_swz = swz(col);
        const uint32_t red_addr = lds_address(red) + (uint32_t)(wave * (MB * 1024) + lane * 16);
        const uint32_t parked_addr = lds_address(parked);
        // the lane's piece of group g of a step lies in scale (g * 128 + kq * 32) >> GSHIFT of the row's SPR
        uint32_t sc_rd[GW], z_rd[GW], z_sh[GW];
#pragma unroll
        for (int g = 0; g < GW; ++g)
        {
            const int i = (g * 128 + kq * 32) >> GSHIFT;
            sc_rd[g] = (uint32_t)(col * SPR + i) * 2u;
            z_rd[g] = (uint32_t)(NSL * 256 + (col * WPR + (i >> 1)) * 4);
            z_sh[g] = (uint32_t)(i & 1) * 4u;
        }
        const uint32_t zp16 = (uint32_t)zp | ((uint32_t)zp << 16);
        int slot = 0;
        for (int it = 0; it < T; ++it)
        {
            floatx4 acc[MB];
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
                acc[mb] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int st = 0; st < STEPS; ++st)
            {
                __builtin_amdgcn_s_waitcnt(mr_vmcnt(LT));
                uintx4 wv[GW];
                uint32_t s2[GW], z16[GW];
                {
                    const uint8_t* sl = ring + slot * TILE_BYTES + rd_base;
                    const uint8_t* ax = aux + slot * AUX;
#pragma unroll
                    for (int g = 0; g < GW; ++g)
                    {
                        wv[g] = *reinterpret_cast<const uintx4*>(sl + (((g * 4 + kq) ^ rd_swz) << 4));
                        const uint32_t sh = *reinterpret_cast<const uint16_t*>(ax + sc_rd[g]);
                        s2[g] = sh | (sh << 16);
                        if constexpr (ZPT)
                        {
                            const uint32_t z = ((uint32_t)ax[z_rd[g]] >> z_sh[g]) & 15u;
                            z16[g] = z | (z << 16);
                        }
                        else
                            z16[g] = zp16;
                    }
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                issue(min(it + (st + 2) / STEPS, T - 1), (st + 2) % STEPS, slot);
                slot ^= 1;
#pragma unroll
                for (int g = 0; g < GW; ++g)
                {
                    const half2_t sc = as_half2(s2[g]);
                    const half2_t lo_add = as_half2(z16[g] | 0xE400E400u);        // -(1024 + z)
                    const half2_t hi_add = as_half2((z16[g] << 4) | 0xD400D400u); // -(64 + z)
                    const uint32_t ww[4] = {wv[g].x, wv[g].y, wv[g].z, wv[g].w};
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                    {
                        const uint32_t w = ww[j];
                        const uint32_t w8 = w >> 8;
                        uintx4 bq;
                        bq.x = as_u32((as_half2((w & MASK_LO) | MAGIC) + lo_add) * sc);     // (q0, q4)
                        bq.y = as_u32((as_half2((w & MASK_HI) | MAGIC_HI) + hi_add) * sc);  // (q1, q5)
                        bq.z = as_u32((as_half2((w8 & MASK_LO) | MAGIC) + lo_add) * sc);    // (q2, q6)
                        bq.w = as_u32((as_half2((w8 & MASK_HI) | MAGIC_HI) + hi_add) * sc); // (q3, q7)
#pragma unroll
                        for (int mb = 0; mb < MB; ++mb)
                            acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, areg[mb][st * GW + g][j]),
                                                                             __builtin_bit_cast(half8_t, bq), acc[mb], 0, 0, 0);
                    }
                }
            }
            mrows_reduce_park<MB>(acc, red, red_addr, parked_addr, it & 1, it, M, tid);
        }
        __builtin_amdgcn_s_waitcnt(mr_vmcnt(0)); // the reloads past the end, before the LDS goes away
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        mrows_flush<false, MB>(parked, Y, t0, T, M, N, tid, GemvFusionArgs{nullptr, nullptr, nullptr, nullptr, 0.f}, 0);
    }

    // ---- 8-bit weights -------------------------------------------------------------------------------------------------
    // w4a16_mrows_q_kernel for 8-bit weights (u8 [N, K]; zero points, ZPT, u8 [N, K / group]), 2 <= M <= 16 MB (two
    // blocks of rows up to K = 4096).  The geometry
    // in bytes is the same (a wavefront takes GW x 64 bytes of each of a tile's 16 weight rows per step, the eight
    // wavefronts side by side along the row), so K = GW x 512 x STEPS; a lane's 16 bytes are 16 weights and meet 32 bytes
    // of activations (two MFMAs per piece instead of four), kept in memory order: a byte b becomes 1024 + b with one
    // v_perm_b32 per pair (0x64 above it), -(1024 + z) is the same pattern applied to z with the sign bit set, then the
    // scale: fp16((q - z) * s) with one rounding.
    // Per step a wavefront fetches the SPR = GW x 64 / group scales of each of the 16 rows (4-byte loads) and, ZPT, their
    // zero points (one byte per lane).  LDS and `pack` as in w4a16_mrows_q_kernel.
    template <int GW, int STEPS, int GSHIFT, bool ZPT, int MB>
    __global__ __launch_bounds__(512) void w8a16_mrows_q_kernel(const half_t* __restrict__ A, const uint8_t* __restrict__ Wq,
                                                                const half_t* __restrict__ S, half_t* __restrict__ Y,
                                                                const uint8_t* __restrict__ zps, int N, int tiles_q,
                                                                int tiles_r, int pack)
    {
        static_assert((GW == 2 || GW == 4) && (STEPS == 2 || STEPS == 4), "K = 2048, 4096, 8192");
        static_assert(GSHIFT >= 5 && GSHIFT <= 7 && (((GW * 64) >> GSHIFT) & 1) == 0 && ((GW * 64) >> GSHIFT) >= 2, "whole words of scales");
        static_assert(MB == 1 || (MB == 2 && GW * STEPS <= 8), "two blocks of rows: 16 VGPRs per piece");
        constexpr int ROW_BYTES = GW * 512 * STEPS; // a weight row
        constexpr int K = ROW_BYTES, G = K >> GSHIFT;
        constexpr int GA = GW * STEPS;          // 64-byte pieces of a weight row per wavefront
        constexpr int SLICE = GW * 64;          // a wavefront's bytes of a weight row per step
        constexpr int SPAN = 8 * SLICE;         // bytes of a weight row that the workgroup covers per step
        constexpr int TILE_BYTES = 16 * SLICE;  // = GW KiB: GW wavefront-wide loads
        constexpr int SPR = (GW * 64) >> GSHIFT; // scales (and zero points) per row, step and wavefront
        constexpr int WPR = SPR / 2;             // ... as 4-byte words
        constexpr int NSL = (16 * WPR + 63) / 64;
        constexpr int NZL = ZPT ? (16 * SPR + 63) / 64 : 0;
        constexpr int AUX = (NSL + NZL) * 256;
        constexpr int LT = GW + NSL + NZL; // loads per step and wavefront
        extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int col = lane & 15; // n within the tile (B operand / D column), m for the A operand
        const int kq = lane >> 4;  // K quarter of the MFMA operands, row quad of D
        const int M = pack & 0xff, zp = (pack >> 8) & 0xff;
        const int b = blockIdx.x;
        const int t0 = b * tiles_q + min(b, tiles_r);
        const int T = tiles_q + (b < tiles_r ? 1 : 0);
        auto row0_of = [&](int i) { return __builtin_amdgcn_readfirstlane(min((t0 + i) * 16, N - 16)); };

        uint8_t* ring = smem + wave * (2 * TILE_BYTES);
        uint8_t* aux = smem + MR_WAVES * 2 * TILE_BYTES + wave * (2 * AUX);
        uint8_t* red = smem + MR_WAVES * 2 * TILE_BYTES + MR_WAVES * 2 * AUX; // [2][8][1024]
        float* parked = reinterpret_cast<float*>(red + 2 * MR_WAVES * MB * 1024);

        // weights: as in w4a16_mrows_kernel
        auto swz = [](int r) { return GW % 4 == 0 ? (r & 15) : (r >> 1) & 7; };
        uint32_t w_off[GW];
#pragma unroll
        for (int c = 0; c < GW; ++c)
        {
            const int pos = c * 1024 + 16 * lane;
            const int r = pos / SLICE, q = (pos % SLICE) >> 4;
            w_off[c] = (uint32_t)r * ROW_BYTES + (uint32_t)wave * SLICE + (uint32_t)((q ^ swz(r)) << 4);
        }
        // scales: lane l of load i fetches word (64 i + l) % WPR of row (64 i + l) / WPR (lanes past the 16 rows: the
        // last row again); zero points: the same with the SPR bytes of a row
        uint32_t s_off[NSL], z_off[NZL > 0 ? NZL : 1];
#pragma unroll
        for (int i = 0; i < NSL; ++i)
        {
            const int at = i * 64 + lane;
            const int r = min(at / WPR, 15), wd = at % WPR;
            s_off[i] = (uint32_t)r * (G * 2) + (uint32_t)wave * (SPR * 2) + (uint32_t)wd * 4u;
        }
#pragma unroll
        for (int i = 0; i < NZL; ++i)
        {
            const int at = i * 64 + lane;
            const int r = min(at / SPR, 15), bz = at % SPR;
            z_off[i] = (uint32_t)r * G + (uint32_t)wave * SPR + (uint32_t)bz;
        }

        // step st of tile `tile` into slot `slot`
        auto issue = [&](int tile, int st, int slot) {
            const uint32_t row0 = (uint32_t)row0_of(tile);
            const uint8_t* wsrc = Wq + (size_t)row0 * ROW_BYTES + st * SPAN;
#pragma unroll
            for (int c = 0; c < GW; ++c)
                __builtin_amdgcn_global_load_lds((mr_global_ptr_t)(wsrc + w_off[c]),
                                                 (mr_lds_ptr_t)(ring + slot * TILE_BYTES + c * 1024), 16, 0, 0);
            const uint8_t* ssrc = reinterpret_cast<const uint8_t*>(S) + (size_t)row0 * (G * 2) + st * (8 * SPR * 2);
#pragma unroll
            for (int i = 0; i < NSL; ++i)
                __builtin_amdgcn_global_load_lds((mr_global_ptr_t)(ssrc + s_off[i]), (mr_lds_ptr_t)(aux + slot * AUX + i * 256), 4, 0, 0);
            if constexpr (ZPT)
            {
                const uint8_t* zsrc = zps + (size_t)row0 * G + st * (8 * SPR);
#pragma unroll
                for (int i = 0; i < NZL; ++i)
                    __builtin_amdgcn_global_load_lds((mr_global_ptr_t)(zsrc + z_off[i]),
                                                     (mr_lds_ptr_t)(aux + slot * AUX + (NSL + i) * 256), 1, 0, 0);
            }
        };

        issue(0, 0, 0);
        issue(0, 1, 1);
        // activations: into the MFMA operand registers (through LDS as whole lines from a few rows on, see
        // workspace::mrows_stages_activations); a block of 16 rows x 256 bytes holds two neighbouring pieces
        uintx4 areg[MB][GA][2];
        if (MB == 1 && !workspace::mrows_stages_activations(M, K))
        {
            const uint8_t* a_bytes = reinterpret_cast<const uint8_t*>(A);
            const uint32_t a_off = (uint32_t)min(col, M - 1) * (uint32_t)(K * 2) + (uint32_t)wave * (GW * 128) + (uint32_t)kq * 32u;
#pragma unroll
            for (int g = 0; g < GA; ++g)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    areg[0][g][j] = *reinterpret_cast<const uintx4*>(a_bytes + (size_t)(a_off + (g / GW) * (SPAN * 2) + (g % GW) * 128 + j * 16));
        }
        else
        {
            uint8_t* stage = red + wave * (2 * ROW_BLOCK_BYTES);
            constexpr int NP = MB * (GA / 2);
            auto fetch = [&](int p) {
                const int mb = p / (GA / 2), g = 2 * (p % (GA / 2));
                row_block_fetch(reinterpret_cast<const uint8_t*>(A), (size_t)K * 2, mb * 16, M - 1,
                                (size_t)((g / GW) * (SPAN * 2) + wave * (GW * 128) + (g % GW) * 128), stage + (p & 1) * ROW_BLOCK_BYTES, lane);
            };
            fetch(0);
#pragma unroll
            for (int p = 0; p < NP; ++p)
            {
                if (p + 1 < NP)
                {
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // block p-1 has been read out of the half that is filled next
                    fetch(p + 1);
                    __builtin_amdgcn_s_waitcnt(vmcnt_only(4));
                }
                else
                    __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
#pragma unroll
                for (int h = 0; h < 2; ++h)
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        areg[p / (GA / 2)][2 * (p % (GA / 2)) + h][j] = row_block_piece(stage + (p & 1) * ROW_BLOCK_BYTES, col, h * 8 + kq * 2 + j);
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __syncthreads();
        }

        // ---- tile loop ---------------------------------------------------------------------------------------
        const uint32_t rd_base = (uint32_t)col * SLICE;
        const int rd_swz = swz(col);
        const uint32_t red_addr = lds_address(red) + (uint32_t)(wave * (MB * 1024) + lane * 16);
        const uint32_t parked_addr = lds_address(parked);
        // the lane's piece g of a step lies in scale (g * 64 + kq * 16) >> GSHIFT of the row's SPR
        uint32_t sc_rd[GW], z_rd[GW];
#pragma unroll
        for (int g = 0; g < GW; ++g)
        {
            const int i = (g * 64 + kq * 16) >> GSHIFT;
            sc_rd[g] = (uint32_t)(col * SPR + i) * 2u;
            z_rd[g] = (uint32_t)(NSL * 256 + (col * SPR + i) * 4);
        }
        const uint32_t zp16 = (uint32_t)zp | ((uint32_t)zp << 16);
        int slot = 0;
        for (int it = 0; it < T; ++it)
        {
            floatx4 acc[MB];
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
                acc[mb] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int st = 0; st < STEPS; ++st)
            {
                __builtin_amdgcn_s_waitcnt(mr_vmcnt(LT));
                uintx4 wv[GW];
                uint32_t s2[GW], z16[GW];
                {
                    const uint8_t* sl = ring + slot * TILE_BYTES + rd_base;
                    const uint8_t* ax = aux + slot * AUX;
#pragma unroll
                    for (int g = 0; g < GW; ++g)
                    {
                        wv[g] = *reinterpret_cast<const uintx4*>(sl + (((g * 4 + kq) ^ rd_swz) << 4));
                        const uint32_t sh = *reinterpret_cast<const uint16_t*>(ax + sc_rd[g]);
                        s2[g] = sh | (sh << 16);
                        if constexpr (ZPT)
                        {
                            const uint32_t z = (uint32_t)ax[z_rd[g]];
                            z16[g] = z | (z << 16);
                        }
                        else
                            z16[g] = zp16;
                    }
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                issue(min(it + (st + 2) / STEPS, T - 1), (st + 2) % STEPS, slot);
                slot ^= 1;
#pragma unroll
                for (int g = 0; g < GW; ++g)
                {
                    const half2_t sc = as_half2(s2[g]);
                    const half2_t add = as_half2(z16[g] | 0xE400E400u); // -(1024 + z)
                    const uint32_t ww[4] = {wv[g].x, wv[g].y, wv[g].z, wv[g].w};
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                    {
                        // v_perm_b32(S0, S1, sel): selectors 0-3 pick bytes of S1, 4-7 of S0
                        const uint32_t w0 = ww[2 * j], w1 = ww[2 * j + 1];
                        uintx4 bq;
                        bq.x = as_u32((as_half2(__builtin_amdgcn_perm(0x64646464u, w0, 0x04010400u)) + add) * sc);
                        bq.y = as_u32((as_half2(__builtin_amdgcn_perm(0x64646464u, w0, 0x04030402u)) + add) * sc);
                        bq.z = as_u32((as_half2(__builtin_amdgcn_perm(0x64646464u, w1, 0x04010400u)) + add) * sc);
                        bq.w = as_u32((as_half2(__builtin_amdgcn_perm(0x64646464u, w1, 0x04030402u)) + add) * sc);
#pragma unroll
                        for (int mb = 0; mb < MB; ++mb)
                            acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, areg[mb][st * GW + g][j]),
                                                                             __builtin_bit_cast(half8_t, bq), acc[mb], 0, 0, 0);
                    }
                }
            }
            mrows_reduce_park<MB>(acc, red, red_addr, parked_addr, it & 1, it, M, tid);
        }
        __builtin_amdgcn_s_waitcnt(mr_vmcnt(0)); // the reloads past the end, before the LDS goes away
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        mrows_flush<false, MB>(parked, Y, t0, T, M, N, tid, GemvFusionArgs{nullptr, nullptr, nullptr, nullptr, 0.f}, 0);
    }

    // w4a16_mrows_q_kernel with K as a run-time value (any multiple of 256; 2 <= M <= 16), as w4a16_mrows_any_kernel below
    // does it for groups of 128 with a scalar zero point: two steps of 8 * GW blocks of 128 weights; a wavefront whose
    // blocks of a step would reach past the end of its range of K fetches the last GW blocks of the range instead and
    // multiplies what another wavefront already covers by scales of zero.  blockIdx.y numbers ranges of range_blocks
    // blocks of K (the last one may be shorter, at least GW blocks); with `partial` the workgroups of a range write its
    // fp32 sums to partial[range][M][N] for the reduction pass.
    // A block of 128 weights has SPC = 128 / group scales; with groups of 128 a wavefront's first block may be an odd one:
    // its scales are fetched from the 4-byte word, its zero points from the byte, at or below it (`skip` = 1), and
    // one word / byte more per row comes along.
    template <int GW, int GSHIFT, bool ZPT>
    __global__ __launch_bounds__(512) void w4a16_mrows_q_any_kernel(const half_t* __restrict__ A, const uint8_t* __restrict__ Wq,
                                                                    const half_t* __restrict__ S, half_t* __restrict__ Y,
                                                                    const uint8_t* __restrict__ zps, float* __restrict__ partial,
                                                                    int N, int K, int range_blocks, int tiles_q, int tiles_r,
                                                                    int pack)
    {
        static_assert(GW >= 2 && GW <= 4 && GSHIFT >= 5 && GSHIFT <= 7, "blocks per wavefront and step; groups of 32 / 64 / 128");
        constexpr int STEPS = 2, MB = 1;
        constexpr int GA = GW * STEPS;
        constexpr int SLICE = GW * 64;
        constexpr int TILE_BYTES = 16 * SLICE;
        constexpr int SPC = 1 << (7 - GSHIFT);                     // scales per block of 128 weights
        constexpr int WPR = SPC == 1 ? GW / 2 + 1 : GW * SPC / 2;  // 4-byte words of scales (= bytes of zero points) per row
        constexpr int NSL = (16 * WPR + 63) / 64;
        constexpr int NZL = ZPT ? NSL : 0;
        constexpr int AUX = (NSL + NZL) * 256;
        constexpr int LT = GW + NSL + NZL;
        extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
        uint32_t MAGIC, MAGIC_HI, MASK_LO, MASK_HI;
        asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(MAGIC));
        asm volatile("v_mov_b32 %0, 0x54005400" : "=v"(MAGIC_HI));
        asm volatile("s_mov_b32 %0, 0x000F000F" : "=s"(MASK_LO));
        asm volatile("s_mov_b32 %0, 0x00F000F0" : "=s"(MASK_HI));

        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int col = lane & 15;
        const int kq = lane >> 4;
        const int M = pack & 0xff, zp = (pack >> 8) & 0xff;
        const int B = K >> 7, ROW_BYTES = K >> 1; // blocks of 128 weights in a row
        const int SROW = (K >> GSHIFT) * 2;       // bytes of a row of scales
        const int ZROW = K >> (GSHIFT + 1);       // bytes of a row of zero points
        const int b = blockIdx.x;
        const int t0 = b * tiles_q + min(b, tiles_r);
        const int T = tiles_q + (b < tiles_r ? 1 : 0);
        auto row0_of = [&](int i) { return __builtin_amdgcn_readfirstlane(min((t0 + i) * 16, N - 16)); };
        const int b_lo = (int)blockIdx.y * range_blocks, b_hi = min(B, b_lo + range_blocks); // this workgroup's part of K
        auto own_block = [&](int st) { return b_lo + st * (8 * GW) + wave * GW; };
        auto fetch_block = [&](int st) { return min(own_block(st), b_hi - GW); };

        uint8_t* ring = smem + wave * (2 * TILE_BYTES);
        uint8_t* aux = smem + MR_WAVES * 2 * TILE_BYTES + wave * (2 * AUX);
        uint8_t* red = smem + MR_WAVES * 2 * TILE_BYTES + MR_WAVES * 2 * AUX; // [2][8][1024]
        float* parked = reinterpret_cast<float*>(red + 2 * MR_WAVES * MB * 1024);

        auto swz = [](int r) { return GW % 4 == 0 ? (r & 15) : GW % 2 == 0 ? (r >> 1) & 7 : (r >> 2) & 3; };
        uint32_t w_off[GW];
#pragma unroll
        for (int c = 0; c < GW; ++c)
        {
            const int pos = c * 1024 + 16 * lane;
            const int r = pos / SLICE, q = (pos % SLICE) >> 4;
            w_off[c] = (uint32_t)r * (uint32_t)ROW_BYTES + (uint32_t)((q ^ swz(r)) << 4);
        }
        // scales / zero points: lane l of load i fetches word / byte (64 i + l) % WPR of row (64 i + l) / WPR, counted from
        // the word / byte that holds the first fetched block's (never past the end of the row: the last one again instead)
        int aux_row[NSL], aux_word[NSL];
#pragma unroll
        for (int i = 0; i < NSL; ++i)
        {
            const int at = i * 64 + lane;
            aux_row[i] = min(at / WPR, 15);
            aux_word[i] = at % WPR;
        }

        auto issue = [&](int tile, int st, int slot) {
            const uint32_t row0 = (uint32_t)row0_of(tile);
            const int bs = fetch_block(st);
            const uint8_t* wsrc = Wq + (size_t)row0 * ROW_BYTES + bs * 64;
#pragma unroll
            for (int c = 0; c < GW; ++c)
                __builtin_amdgcn_global_load_lds((mr_global_ptr_t)(wsrc + w_off[c]),
                                                 (mr_lds_ptr_t)(ring + slot * TILE_BYTES + c * 1024), 16, 0, 0);
            const int s_first = (bs * SPC * 2) & ~3;            // byte of the first word within the row's scales
            const int s_last = ((SROW - s_first) >> 2) - 1;     // last word of this window that is still inside the row
            const uint8_t* ssrc = reinterpret_cast<const uint8_t*>(S) + (size_t)row0 * SROW + s_first;
#pragma unroll
            for (int i = 0; i < NSL; ++i)
                __builtin_amdgcn_global_load_lds((mr_global_ptr_t)(ssrc + (uint32_t)(aux_row[i] * SROW + 4 * min(aux_word[i], s_last))),
                                                 (mr_lds_ptr_t)(aux + slot * AUX + i * 256), 4, 0, 0);
            if constexpr (ZPT)
            {
                const int z_first = (bs * SPC) >> 1;
                const int z_last = ZROW - z_first - 1;
                const uint8_t* zsrc = zps + (size_t)row0 * ZROW + z_first;
#pragma unroll
                for (int i = 0; i < NSL; ++i)
                    __builtin_amdgcn_global_load_lds((mr_global_ptr_t)(zsrc + (uint32_t)(aux_row[i] * ZROW + min(aux_word[i], z_last))),
                                                     (mr_lds_ptr_t)(aux + slot * AUX + (NSL + i) * 256), 1, 0, 0);
            }
        };
        issue(0, 0, 0);
        issue(0, 1, 1);

        const uint32_t rd_base = (uint32_t)col * SLICE;
        const int rd_swz = swz(col);
        const uint32_t red_addr = lds_address(red) + (uint32_t)(wave * (MB * 1024) + lane * 16);
        const uint32_t parked_addr = lds_address(parked);
        // activations: into the MFMA operand registers (through LDS as whole lines from a few rows on, see
        // workspace::mrows_stages_activations), then in the pair order of the nibble trick
        uintx4 areg[GA][4];
        {
            if (!workspace::mrows_stages_activations(M, K))
            {
                const uint8_t* a_row = reinterpret_cast<const uint8_t*>(A) + (size_t)min(col, M - 1) * (size_t)(K * 2) + kq * 64;
#pragma unroll
                for (int st = 0; st < STEPS; ++st)
                {
                    const uint8_t* a_src = a_row + (size_t)fetch_block(st) * 256;
#pragma unroll
                    for (int g = 0; g < GW; ++g)
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            areg[st * GW + g][j] = *reinterpret_cast<const uintx4*>(a_src + g * 256 + j * 16);
                }
            }
            else
            {
                uint8_t* stage = red + wave * (2 * ROW_BLOCK_BYTES);
                auto fetch = [&](int p) {
                    row_block_fetch(reinterpret_cast<const uint8_t*>(A), (size_t)K * 2, 0, M - 1, (size_t)(fetch_block(p / GW) + p % GW) * 256,
                                    stage + (p & 1) * ROW_BLOCK_BYTES, lane);
                };
                fetch(0);
#pragma unroll
                for (int p = 0; p < GA; ++p)
                {
                    if (p + 1 < GA)
                    {
                        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // block p-1 has been read out of the half that is filled next
                        fetch(p + 1);
                        __builtin_amdgcn_s_waitcnt(vmcnt_only(4));
                    }
                    else
                        __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        areg[p][j] = row_block_piece(stage + (p & 1) * ROW_BLOCK_BYTES, col, kq * 4 + j);
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                __syncthreads();
            }
#pragma unroll
            for (int g = 0; g < GA; ++g)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    areg[g][j] = permute_a8(areg[g][j]);
        }
        const uint32_t zp16 = (uint32_t)zp | ((uint32_t)zp << 16);
        const int sub = (kq * 32) >> GSHIFT; // the lane's scale within a block
        int slot = 0;
        for (int it = 0; it < T; ++it)
        {
            floatx4 acc[MB] = {floatx4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int st = 0; st < STEPS; ++st)
            {
                // the blocks of this step that no other wavefront covers: from `fresh` on
                const int bs = fetch_block(st);
                const int fresh = own_block(st) - bs;
                const int skip = SPC == 1 ? (bs & 1) : 0;
                __builtin_amdgcn_s_waitcnt(mr_vmcnt(LT));
                uintx4 wv[GW];
                uint32_t s2[GW], z16[GW];
                {
                    const uint8_t* sl = ring + slot * TILE_BYTES + rd_base;
                    const uint8_t* ax = aux + slot * AUX;
#pragma unroll
                    for (int g = 0; g < GW; ++g)
                    {
                        wv[g] = *reinterpret_cast<const uintx4*>(sl + (((g * 4 + kq) ^ rd_swz) << 4));
                        const int idx = skip + g * SPC + sub; // among the scales this row fetched
                        const uint32_t sh = *reinterpret_cast<const uint16_t*>(ax + (col * (WPR * 2) + idx) * 2);
                        s2[g] = g >= fresh ? (sh | (sh << 16)) : 0u;
                        if constexpr (ZPT)
                        {
                            const uint32_t z = ((uint32_t)ax[NSL * 256 + (col * WPR + (idx >> 1)) * 4] >> ((idx & 1) * 4)) & 15u;
                            z16[g] = z | (z << 16);
                        }
                        else
                            z16[g] = zp16;
                    }
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                issue(min(it + (st + 2) / STEPS, T - 1), (st + 2) % STEPS, slot);
                slot ^= 1;
#pragma unroll
                for (int g = 0; g < GW; ++g)
                {
                    const half2_t sc = as_half2(s2[g]);
                    const half2_t lo_add = as_half2(z16[g] | 0xE400E400u);        // -(1024 + z)
                    const half2_t hi_add = as_half2((z16[g] << 4) | 0xD400D400u); // -(64 + z)
                    const uint32_t ww[4] = {wv[g].x, wv[g].y, wv[g].z, wv[g].w};
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                    {
                        const uint32_t w = ww[j];
                        const uint32_t w8 = w >> 8;
                        uintx4 bq;
                        bq.x = as_u32((as_half2((w & MASK_LO) | MAGIC) + lo_add) * sc);
                        bq.y = as_u32((as_half2((w & MASK_HI) | MAGIC_HI) + hi_add) * sc);
                        bq.z = as_u32((as_half2((w8 & MASK_LO) | MAGIC) + lo_add) * sc);
                        bq.w = as_u32((as_half2((w8 & MASK_HI) | MAGIC_HI) + hi_add) * sc);
                        acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, areg[st * GW + g][j]),
                                                                        __builtin_bit_cast(half8_t, bq), acc[0], 0, 0, 0);
                    }
                }
            }
            mrows_reduce_park<MB>(acc, red, red_addr, parked_addr, it & 1, it, M, tid);
        }
        __builtin_amdgcn_s_waitcnt(mr_vmcnt(0)); // the reloads past the end, before the LDS goes away
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        if (partial)
        {
            for (int idx = tid; idx < T * M * 16; idx += 512)
            {
                const int n = idx & 15;
                const int im = idx >> 4;
                const int it = im / M, m = im - it * M;
                partial[(size_t)blockIdx.y * M * N + (size_t)m * N + min((t0 + it) * 16, N - 16) + n] = parked[idx];
            }
        }
        else
            mrows_flush<false, MB>(parked, Y, t0, T, M, N, tid, GemvFusionArgs{nullptr, nullptr, nullptr, nullptr, 0.f}, 0);
    }

    // The same kernel with K as a run-time value: any multiple of 256 up to 8 * GW * STEPS groups (2 <= M <= 16).
    // A wavefront whose GW groups of a step would reach past the end of K fetches the last GW groups of the row
    // instead (the loads of every wavefront and step stay the same in number, which the hand-written wait counts
    // need) and multiplies what another wavefront already covers by a scale of zero.
    // (Longer K in several passes over the tiles, each with its own part of the activations in registers, was
    // measured: every pass pays the start of the kernel again, and the split-K kernel is faster.)
    // K above 8192: blockIdx.y numbers ranges of range_groups groups of K (the last one may be shorter, at least GW
    // groups); the workgroups of a range write its fp32 sums to partial[range][M][N] for the reduction pass.
    // MB = 2 (17 .. 32 rows): at most four groups per wavefront; MB = 4 (33 .. 64 rows): at most two.  LDS as above.
    // pack = M | zp << 8.
    // FUSED: as in w4a16_mrows_kernel; over ranges of K only the RMSNorm weight applies here (the sums of a range go to
    // `partial` as they are: rstd and the rest of the epilogue belong to the reduction pass).
    template <int GW, int STEPS, int MB, bool FUSED, bool STAGE>
    __global__ __launch_bounds__(512) void w4a16_mrows_any_kernel(const half_t* __restrict__ A, const uint8_t* __restrict__ Wq,
                                                                  const half_t* __restrict__ S, half_t* __restrict__ Y,
                                                                  float* __restrict__ partial, int N, int K, int tiles,
                                                                  int pack, GemvFusionArgs f, uint32_t* sync)
    {
        static_assert(GW >= 1 && GW <= 7 && STEPS >= 1 && GW * STEPS <= 8, "groups per wavefront");
        static_assert(MB == 1 || (MB == 2 && GW * STEPS <= 4) || (MB == 4 && GW * STEPS <= 2), "16 VGPRs per group and block of rows");
        constexpr int GA = GW * STEPS;         // groups of a wavefront
        constexpr int SLICE = GW * 64;         // a wavefront's bytes of a weight row per step
        constexpr int TILE_BYTES = 16 * SLICE; // = GW KiB: GW wavefront-wide loads
        constexpr int LT = GW + 1;             // loads per step and wavefront (weights + scales)
        constexpr int SC_LANES = GW / 2 + 1;   // 4-byte scale loads per row: GW groups from any 2-byte offset
        extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
        uint32_t MAGIC, MAGIC_HI, MASK_LO, MASK_HI;
        asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(MAGIC));
        asm volatile("v_mov_b32 %0, 0x54005400" : "=v"(MAGIC_HI));
        asm volatile("s_mov_b32 %0, 0x000F000F" : "=s"(MASK_LO));
        asm volatile("s_mov_b32 %0, 0x00F000F0" : "=s"(MASK_HI));

        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int col = lane & 15;
        const int kq = lane >> 4;
        // (fourteen dwords of arguments arrive in scalar registers with the wavefront: everything the first weight load
        // needs is among them -- tiles = tiles_q | tiles_r << 16, pack = M | zp << 8 | gate << 16 | range_groups << 17;
        // with more, the kernel began by waiting for a load of its own arguments)
        const int M = pack & 0xff, zp = (pack >> 8) & 0xff, gate = (pack >> 16) & 1, range_groups = (int)((unsigned)pack >> 17);
        const int tiles_q = tiles & 0xffff, tiles_r = (int)((unsigned)tiles >> 16);
        const int G = K >> 7, ROW_BYTES = K >> 1;
        const int b = blockIdx.x;
        const int t0 = b * tiles_q + min(b, tiles_r);
        const int T_out = tiles_q + (b < tiles_r ? 1 : 0);
        const int T = (FUSED && gate) ? 2 * T_out : T_out; // weight tiles this workgroup walks
        // weight rows of the workgroup's tile i (the last tile of an N that is not a multiple of 16 is moved back to
        // rows N-16 .. N-1)
        auto row0_of = [&](int i) {
            if (FUSED && gate)
                return __builtin_amdgcn_readfirstlane(((i & 1) ? N : 0) + min((t0 + (i >> 1)) * 16, N - 16));
            return __builtin_amdgcn_readfirstlane(min((t0 + i) * 16, N - 16));
        };
        const int g_lo = (int)blockIdx.y * range_groups, g_hi = min(G, g_lo + range_groups); // this workgroup's part of K
        // first group that wavefront `wave` owns in step st, and the first group it fetches
        auto own_group = [&](int st) { return g_lo + st * (8 * GW) + wave * GW; };
        auto fetch_group = [&](int st) { return min(own_group(st), g_hi - GW); };

        uint8_t* ring = smem + wave * (2 * TILE_BYTES);
        uint8_t* sc_ring = smem + MR_WAVES * 2 * TILE_BYTES + wave * 512;
        uint8_t* red = smem + MR_WAVES * 2 * TILE_BYTES + MR_WAVES * 512; // [2][8][1024]
        float* sum_sq = reinterpret_cast<float*>(red + 2 * MR_WAVES * MB * 1024); // [8][MB x 16]
        float* parked = sum_sq + MR_WAVES * MB * 16;

        auto swz = [](int r) { return GW % 4 == 0 ? (r & 15) : GW % 2 == 0 ? (r >> 1) & 7 : (r >> 2) & 3; };
        uint32_t w_off[GW];
#pragma unroll
        for (int c = 0; c < GW; ++c)
        {
            const int pos = c * 1024 + 16 * lane;
            const int r = pos / SLICE, q = (pos % SLICE) >> 4;
            w_off[c] = (uint32_t)r * (uint32_t)ROW_BYTES + (uint32_t)((q ^ swz(r)) << 4);
        }
        // scales: lane l fetches 4 bytes of row l / SC_LANES, counted from the 4-byte boundary at or below the first
        // fetched group (never past the end of the row: the last word is fetched twice instead)
        const uint32_t s_lane_row = (uint32_t)min(lane / SC_LANES, 15) * (uint32_t)(G * 2);
        const int s_lane_word = lane % SC_LANES;

        auto issue = [&](int tile, int st, int slot) {
            const uint32_t row0 = (uint32_t)row0_of(tile);
            const int gs = fetch_group(st);
            const uint8_t* wsrc = Wq + (size_t)row0 * ROW_BYTES + gs * 64;
#pragma unroll
            for (int c = 0; c < GW; ++c)
                __builtin_amdgcn_global_load_lds((mr_global_ptr_t)(wsrc + w_off[c]),
                                                 (mr_lds_ptr_t)(ring + slot * TILE_BYTES + c * 1024), 16, 0, 0);
            const int first = (gs * 2) & ~3;                  // byte offset of the first word within the row's scales
            const int last_word = ((G * 2 - first) >> 2) - 1; // of this window that is still inside the row
            const uint32_t s_off = s_lane_row + (uint32_t)(first + 4 * min(s_lane_word, last_word));
            __builtin_amdgcn_global_load_lds((mr_global_ptr_t)(reinterpret_cast<const uint8_t*>(S) + (size_t)row0 * (G * 2) + s_off),
                                             (mr_lds_ptr_t)(sc_ring + slot * 256), 4, 0, 0);
        };
        issue(0, 0, 0);
        issue(min(1 / STEPS, T - 1), 1 % STEPS, 1);

        const uint32_t rd_base = (uint32_t)col * SLICE;
        const int rd_swz = swz(col);
        const uint32_t red_addr = lds_address(red) + (uint32_t)(wave * (MB * 1024) + lane * 16);
        const uint32_t parked_addr = lds_address(parked);
        int slot = 0;
        {
            // ---- the activations: into the MFMA operand registers, through LDS as whole lines (see row_block_fetch: two
            // blocks per wavefront, over what holds the partial tiles and the parked sums later -- hence the barrier)
            // (a few rows: straight into the registers, as in the kernel above)
            uintx4 areg[MB][GA][4];
            floatx4 ncorr[MB][GA];
            if constexpr (!STAGE)
            {
                const uint8_t* a_row = reinterpret_cast<const uint8_t*>(A) + (size_t)min(col, M - 1) * (size_t)(K * 2) + kq * 64;
#pragma unroll
                for (int ga = 0; ga < GA; ++ga)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        areg[0][ga][j] = *reinterpret_cast<const uintx4*>(a_row + (size_t)(fetch_group(ga / GW) + ga % GW) * 256 + j * 16);
            }
            else
            {
                uint8_t* stage = red + wave * (2 * ROW_BLOCK_BYTES);
                constexpr int NP = MB * GA;
                auto fetch = [&](int p) {
                    const int mb = p / GA, ga = p % GA;
                    row_block_fetch(reinterpret_cast<const uint8_t*>(A), (size_t)K * 2, mb * 16, M - 1,
                                    (size_t)(fetch_group(ga / GW) + ga % GW) * 256, stage + (p & 1) * ROW_BLOCK_BYTES, lane);
                };
                fetch(0);
#pragma unroll
                for (int p = 0; p < NP; ++p)
                {
                    if (p + 1 < NP)
                    {
                        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // block p-1 has been read out of the half that is filled next
                        fetch(p + 1);
                        __builtin_amdgcn_s_waitcnt(vmcnt_only(4));
                    }
                    else
                        __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        areg[p / GA][p % GA][j] = row_block_piece(stage + (p & 1) * ROW_BLOCK_BYTES, col, kq * 4 + j);
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                __syncthreads();
            }
            if (FUSED && f.gamma)
                mrows_scale_a<MB, GA>(areg, [&](int g) {
                    return reinterpret_cast<const uint8_t*>(f.gamma) + kq * 64 + (size_t)fetch_group(g / GW) * 256 + (g % GW) * 256;
                });
            mrows_prepare_a<MB, GA>(areg, ncorr, zp);
            for (int it = 0; it < T; ++it)
            {
                floatx4 acc[MB];
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
                    acc[mb] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int st = 0; st < STEPS; ++st)
                {
                    // the groups of this step that no other wavefront covers: from `fresh` on
                    const int gs = fetch_group(st);
                    const int fresh = own_group(st) - gs;
                    const int sc_skip = gs & 1;
                    // this step has landed when at most the next step's loads are outstanding
                    __builtin_amdgcn_s_waitcnt(mr_vmcnt(LT));
                    uintx4 wv[GW];
                    float sv[GW];
                    {
                        const uint8_t* sl = ring + slot * TILE_BYTES + rd_base;
                        const half_t* sc = reinterpret_cast<const half_t*>(sc_ring + slot * 256);
#pragma unroll
                        for (int g = 0; g < GW; ++g)
                        {
                            wv[g] = *reinterpret_cast<const uintx4*>(sl + (((g * 4 + kq) ^ rd_swz) << 4));
                            const float sg = (float)sc[col * (SC_LANES * 2) + sc_skip + g];
                            sv[g] = g >= fresh ? sg : 0.f;
                        }
                    }
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    issue(min(it + (st + 2) / STEPS, T - 1), (st + 2) % STEPS, slot);
                    slot ^= 1;
#pragma unroll
                    for (int g = 0; g < GW; ++g)
                        mrows_group<MB, GA>(acc, areg, ncorr, st * GW + g, wv[g], sv[g], MAGIC, MAGIC_HI, MASK_LO, MASK_HI);
                }
                mrows_reduce_park<MB>(acc, red, red_addr, parked_addr, it & 1, it, M, tid);
            }
        }
        __builtin_amdgcn_s_waitcnt(mr_vmcnt(0)); // the reloads past the end, before the LDS goes away
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        if (partial && !sync)
        {
            for (int idx = tid; idx < T * M * 16; idx += 512)
            {
                const int n = idx & 15;
                const int im = idx >> 4;
                const int it = im / M, m = im - it * M;
                partial[(size_t)blockIdx.y * M * N + (size_t)m * N + min((t0 + it) * 16, N - 16) + n] = parked[idx];
            }
        }
        else if (partial)
        {
            // ---- ranges of K added up inside the launch: the workgroups that walked these tiles (one per range: same
            // blockIdx.x) count themselves in at sync[blockIdx.x] once their sums are visible to every CU (stores at device
            // scope, completed); the last to arrive adds the ranges in order -- so the result does not depend on who that
            // is -- runs the epilogue of the reduction pass (rstd, bias, residual: same roundings) and leaves the word zero
            // for the next launch.  Nobody waits.
            for (int idx = tid; idx < T * M * 16; idx += 512)
            {
                const int n = idx & 15;
                const int im = idx >> 4;
                const int it = im / M, m = im - it * M;
                __hip_atomic_store(partial + (size_t)blockIdx.y * M * N + (size_t)m * N + min((t0 + it) * 16, N - 16) + n, parked[idx],
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            __builtin_amdgcn_s_waitcnt(mr_vmcnt(0));
            // (a word of the partial tiles' LDS, free since the barrier above: the kernel's dynamic LDS may be all there is)
            volatile uint32_t* arrived_before = reinterpret_cast<volatile uint32_t*>(red);
            __syncthreads();
            if (tid == 0)
                *arrived_before = atomicAdd(sync + blockIdx.x, 1u);
            __syncthreads();
            if (*arrived_before == gridDim.y - 1)
            {
                const int ranges = (int)gridDim.y;
                for (int idx = tid; idx < T * M * 16; idx += 512)
                {
                    const int n = idx & 15;
                    const int im = idx >> 4;
                    const int it = im / M, m = im - it * M;
                    const int nn = min((t0 + it) * 16, N - 16) + n;
                    if (nn < (t0 + it) * 16) // (a last tile moved back: these columns belong to the tile before it)
                        continue;
                    const size_t at = (size_t)m * N + nn;
                    // (rstd, bias and residual are requested ahead of the ranges' sums and without a branch around the loads --
                    // an absent one reads a word of the sums instead, unused: asked for where they are added, or under a
                    // branch, each was a round trip of its own at the very end of the kernel)
                    half_t bias_n = (half_t)0.f, residual_at = (half_t)0.f;
                    float rstd_m = 1.0f;
                    if constexpr (FUSED)
                    {
                        const half_t* spare = reinterpret_cast<const half_t*>(partial);
                        bias_n = *(f.bias ? f.bias + nn : spare);
                        residual_at = *(f.residual ? f.residual + at : spare);
                        rstd_m = *(f.rstd ? f.rstd + m : reinterpret_cast<const float*>(partial));
                    }
                    // (four ranges in flight, added in order)
                    float sum = 0.f;
                    for (int r0 = 0; r0 < ranges; r0 += 4)
                    {
                        float part[4];
#pragma unroll
                        for (int d = 0; d < 4; ++d)
                            part[d] = __hip_atomic_load(partial + (size_t)min(r0 + d, ranges - 1) * M * N + at, __ATOMIC_RELAXED,
                                                        __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                        for (int d = 0; d < 4; ++d)
                            if (r0 + d < ranges)
                                sum += part[d];
                    }
                    if (FUSED)
                    {
                        // y = fp16(sum) (+ bias) (+ residual), each step rounded to fp16 (finish_bias_residual)
                        half_t y = (half_t)f32_product(sum, f.rstd ? rstd_m : 1.0f);
                        if (f.bias)
                            y = (half_t)((float)y + (float)bias_n);
                        if (f.residual)
                            y = (half_t)((float)y + (float)residual_at);
                        Y[at] = y;
                    }
                    else
                        Y[at] = (half_t)sum;
                }
                if (tid == 0)
                    atomicExch(sync + blockIdx.x, 0u);
            }
        }
        else
            mrows_flush<FUSED, MB>(parked, Y, t0, T_out, M, N, tid, f, gate);
    }

    namespace
    {
        GemvFusionArgs fusion_args(const GemvFusion& fusion)
        {
            return GemvFusionArgs{(const half_t*)fusion.gamma, fusion.rstd, (const half_t*)fusion.bias, (const half_t*)fusion.residual,
                                  fusion.rms_eps};
        }

        // N: output columns (fusion.gate: from 2 N weight rows)
        template <int GW, int STEPS, int MB, bool FUSED, bool STAGE = true>
        hipError_t launch_mrows_mb(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M, int N, int zp,
                                   int num_cu, const GemvFusion& fusion)
        {
            const int n_tiles = (N + 15) / 16;
            const int grid = n_tiles < num_cu ? n_tiles : num_cu;
            const int tiles_q = n_tiles / grid, tiles_r = n_tiles % grid;
            const size_t lds =
                workspace::w4a16_mrows_lds_bytes(GW * STEPS * 1024, M, (fusion.gate ? 2 : 1) * (tiles_q + (tiles_r ? 1 : 0)));
            if (lds > MAX_LDS_BYTES)
                return hipErrorInvalidValue;
            auto kernel = &w4a16_mrows_kernel<GW, STEPS, MB, FUSED, STAGE>;
            if (lds > 64 * 1024)
            {
                static LdsGrant granted;
                const hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), granted, (int)MAX_LDS_BYTES);
                if (e != hipSuccess)
                    return e;
            }
            hipLaunchKernelGGL(kernel, dim3(grid), dim3(MR_WAVES * 64), lds, stream, (const half_t*)A, (const uint8_t*)Wq,
                               (const half_t*)S, (half_t*)Y, N, tiles_q, tiles_r, M | (zp << 8) | (fusion.gate ? 1 << 16 : 0),
                               fusion_args(fusion));
            return hipGetLastError();
        }

        template <int GW, int STEPS>
        hipError_t launch_mrows(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M, int N, int zp,
                                int num_cu, const GemvFusion& fusion)
        {
            const bool fused = fusion.any();
            if (M <= 16 && !workspace::mrows_stages_activations(M, GW * STEPS * 1024))
                return fused ? launch_mrows_mb<GW, STEPS, 1, true, false>(stream, A, Wq, S, Y, M, N, zp, num_cu, fusion)
                             : launch_mrows_mb<GW, STEPS, 1, false, false>(stream, A, Wq, S, Y, M, N, zp, num_cu, fusion);
            if (M <= 16)
                return fused ? launch_mrows_mb<GW, STEPS, 1, true>(stream, A, Wq, S, Y, M, N, zp, num_cu, fusion)
                             : launch_mrows_mb<GW, STEPS, 1, false>(stream, A, Wq, S, Y, M, N, zp, num_cu, fusion);
            if constexpr (GW * STEPS <= 4)
                return fused ? launch_mrows_mb<GW, STEPS, 2, true>(stream, A, Wq, S, Y, M, N, zp, num_cu, fusion)
                             : launch_mrows_mb<GW, STEPS, 2, false>(stream, A, Wq, S, Y, M, N, zp, num_cu, fusion);
            return hipErrorInvalidValue;
        }
    } // namespace

    namespace
    {
        // ranges == 1: the whole of K, fp16 results to Y; otherwise ranges of range_groups groups, fp32 sums to partial
        template <int GW, int STEPS, int MB, bool FUSED, bool STAGE = true>
        hipError_t launch_mrows_any_mb(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M, int N, int K,
                                       int zp, int num_cu, float* partial, int ranges, int range_groups, const GemvFusion& fusion,
                                       uint32_t* sync)
        {
            const int n_tiles = (N + 15) / 16;
            const int per_range = num_cu / ranges > 0 ? num_cu / ranges : 1;
            const int grid = n_tiles < per_range ? n_tiles : per_range;
            const int tiles_q = n_tiles / grid, tiles_r = n_tiles % grid;
            const size_t lds = workspace::w4a16_mrows_lds_bytes_gw(GW, M, (fusion.gate ? 2 : 1) * (tiles_q + (tiles_r ? 1 : 0)));
            // over ranges of K the epilogue belongs to whoever adds the ranges up: the reduction pass, or (sync) the launch itself
            if (lds > MAX_LDS_BYTES || (ranges > 1 && (fusion.gate || (!sync && (fusion.bias || fusion.residual || fusion.rstd)))))
                return hipErrorInvalidValue;
            auto kernel = &w4a16_mrows_any_kernel<GW, STEPS, MB, FUSED, STAGE>;
            if (lds > 64 * 1024)
            {
                static LdsGrant granted;
                const hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), granted, (int)MAX_LDS_BYTES);
                if (e != hipSuccess)
                    return e;
            }
            if (tiles_q > 0xffff || tiles_r > 0xffff || range_groups > 0x7fff)
                return hipErrorInvalidValue;
            hipLaunchKernelGGL(kernel, dim3(grid, ranges), dim3(MR_WAVES * 64), lds, stream, (const half_t*)A, (const uint8_t*)Wq,
                               (const half_t*)S, (half_t*)Y, ranges > 1 ? partial : nullptr, N, K, tiles_q | (tiles_r << 16),
                               M | (zp << 8) | (fusion.gate ? 1 << 16 : 0) | (range_groups << 17), fusion_args(fusion),
                               ranges > 1 ? sync : nullptr);
            return hipGetLastError();
        }

        template <int GW, int STEPS, bool FUSED>
        hipError_t launch_mrows_any_f(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M, int N, int K,
                                      int zp, int num_cu, float* partial, int ranges, int range_groups, const GemvFusion& fusion,
                                      uint32_t* sync)
        {
            if (M <= 16 && !workspace::mrows_stages_activations(M, K))
                return launch_mrows_any_mb<GW, STEPS, 1, FUSED, false>(stream, A, Wq, S, Y, M, N, K, zp, num_cu, partial, ranges,
                                                                       range_groups, fusion, sync);
            if (M <= 16)
                return launch_mrows_any_mb<GW, STEPS, 1, FUSED>(stream, A, Wq, S, Y, M, N, K, zp, num_cu, partial, ranges, range_groups,
                                                                fusion, sync);
            if constexpr (GW * STEPS <= 4)
                if (M <= 32)
                    return launch_mrows_any_mb<GW, STEPS, 2, FUSED>(stream, A, Wq, S, Y, M, N, K, zp, num_cu, partial, ranges,
                                                                    range_groups, fusion, sync);
            if constexpr (GW * STEPS <= 2)
                if (M <= 64)
                    return launch_mrows_any_mb<GW, STEPS, 4, FUSED>(stream, A, Wq, S, Y, M, N, K, zp, num_cu, partial, ranges,
                                                                    range_groups, fusion, sync);
            return hipErrorInvalidValue;
        }

        template <int GW, int STEPS>
        hipError_t launch_mrows_any(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M, int N, int K,
                                    int zp, int num_cu, const GemvFusion& fusion, float* partial = nullptr, int ranges = 1,
                                    int range_groups = 64, uint32_t* sync = nullptr)
        {
            return fusion.any() ? launch_mrows_any_f<GW, STEPS, true>(stream, A, Wq, S, Y, M, N, K, zp, num_cu, partial, ranges,
                                                                      range_groups, fusion, sync)
                                : launch_mrows_any_f<GW, STEPS, false>(stream, A, Wq, S, Y, M, N, K, zp, num_cu, partial, ranges,
                                                                       range_groups, fusion, sync);
        }
    } // namespace

    bool w4a16_mrows_supported(int M, int N, int K, int num_cu, bool gate)
    {
        return workspace::w4a16_mrows_fits(M, N, K, num_cu, gate);
    }
    bool w4a16_mrows_preferred(int M, int N, int K, int num_cu, bool gate)
    {
        return workspace::w4a16_mrows_preferred(M, N, K, num_cu, gate);
    }

    hipError_t launch_w4a16_mrows(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M, int N,
                                  int K, int zp, int num_cu, const GemvFusion& fusion)
    {
        if (!w4a16_mrows_supported(M, N, K, num_cu, fusion.gate) || (fusion.gate && (fusion.bias || fusion.residual)))
            return hipErrorInvalidValue;
        if (!workspace::w4a16_mrows_fixed_k(M, K))
        {
            switch (workspace::w4a16_mrows_step_groups(M, K))
            {
            case 2: return launch_mrows_any<2, 2>(stream, A, Wq, S, Y, M, N, K, zp, num_cu, fusion);
            case 3: return launch_mrows_any<3, 2>(stream, A, Wq, S, Y, M, N, K, zp, num_cu, fusion);
            default: return launch_mrows_any<4, 2>(stream, A, Wq, S, Y, M, N, K, zp, num_cu, fusion);
            }
        }
        // K / 1024 = groups per wavefront and tile, walked in STEPS steps of GW groups.  Two steps per tile where
        // K / 1024 is even: with the two ring slots that is one tile in flight per wavefront (32 KiB per CU at
        // K = 4096, 64 KiB at 8192).  Measured against one step (two tiles in flight) and four steps (half a tile):
        // 5-25 % faster than either at K = 4096, 6144 and 8192.
        switch (K >> 10)
        {
        case 1: return launch_mrows<1, 1>(stream, A, Wq, S, Y, M, N, zp, num_cu, fusion);
        case 2: return launch_mrows<1, 2>(stream, A, Wq, S, Y, M, N, zp, num_cu, fusion);
        case 3: return launch_mrows<3, 1>(stream, A, Wq, S, Y, M, N, zp, num_cu, fusion);
        case 4: return launch_mrows<2, 2>(stream, A, Wq, S, Y, M, N, zp, num_cu, fusion);
        case 6: return launch_mrows<3, 2>(stream, A, Wq, S, Y, M, N, zp, num_cu, fusion);
        default: return launch_mrows<4, 2>(stream, A, Wq, S, Y, M, N, zp, num_cu, fusion);
        }
    }

    namespace
    {
        template <int GW, int GSHIFT, bool ZPT, int MB>
        hipError_t launch_mrows_q_mb(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M, int N, int zp,
                                     const void* zps, int num_cu)
        {
            if constexpr (((GW << (7 - GSHIFT)) & 1) != 0 || (MB == 2 && GW > 2))
                return hipErrorInvalidValue;
            else
            {
                const int n_tiles = (N + 15) / 16;
                const int grid = n_tiles < num_cu ? n_tiles : num_cu;
                const int tiles_q = n_tiles / grid, tiles_r = n_tiles % grid;
                const size_t lds = workspace::w4a16_mrows_q_lds_bytes(GW * 2048, M, tiles_q + (tiles_r ? 1 : 0), GSHIFT, ZPT);
                if (lds > MAX_LDS_BYTES)
                    return hipErrorInvalidValue;
                auto kernel = &w4a16_mrows_q_kernel<GW, GSHIFT, ZPT, MB>;
                if (lds > 64 * 1024)
                {
                    static LdsGrant granted;
                    const hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), granted, (int)MAX_LDS_BYTES);
                    if (e != hipSuccess)
                        return e;
                }
                hipLaunchKernelGGL(kernel, dim3(grid), dim3(MR_WAVES * 64), lds, stream, (const half_t*)A, (const uint8_t*)Wq,
                                   (const half_t*)S, (half_t*)Y, (const uint8_t*)zps, N, tiles_q, tiles_r, M | (zp << 8));
                return hipGetLastError();
            }
        }
        template <int GW, int GSHIFT, bool ZPT>
        hipError_t launch_mrows_q(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M, int N, int zp,
                                  const void* zps, int num_cu)
        {
            return M <= 16 ? launch_mrows_q_mb<GW, GSHIFT, ZPT, 1>(stream, A, Wq, S, Y, M, N, zp, zps, num_cu)
                           : launch_mrows_q_mb<GW, GSHIFT, ZPT, 2>(stream, A, Wq, S, Y, M, N, zp, zps, num_cu);
        }
        template <int GW>
        hipError_t launch_mrows_q_gw(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M, int N,
                                     int group_shift, int zp, const void* zps, int num_cu)
        {
            switch (group_shift * 2 + (zps ? 1 : 0))
            {
            case 10: return launch_mrows_q<GW, 5, false>(stream, A, Wq, S, Y, M, N, zp, zps, num_cu);
            case 11: return launch_mrows_q<GW, 5, true>(stream, A, Wq, S, Y, M, N, zp, zps, num_cu);
            case 12: return launch_mrows_q<GW, 6, false>(stream, A, Wq, S, Y, M, N, zp, zps, num_cu);
            case 13: return launch_mrows_q<GW, 6, true>(stream, A, Wq, S, Y, M, N, zp, zps, num_cu);
            case 15: return launch_mrows_q<GW, 7, true>(stream, A, Wq, S, Y, M, N, zp, zps, num_cu);
            default: return hipErrorInvalidValue; // groups of 128 with a scalar zero point: w4a16_mrows_kernel
            }
        }
    } // namespace

    bool w4a16_mrows_q_supported(int M, int N, int K, int group_shift, bool zero_points, int num_cu)
    {
        return !(group_shift == 7 && !zero_points) && workspace::w4a16_mrows_q_fits(M, N, K, group_shift, zero_points, num_cu);
    }

    hipError_t launch_w4a16_mrows_q(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M, int N,
                                    int K, int group_shift, int zp, const void* zero_points, int num_cu)
    {
        if (!w4a16_mrows_q_supported(M, N, K, group_shift, zero_points != nullptr, num_cu))
            return hipErrorInvalidValue;
        switch (K >> 11)
        {
        case 1: return launch_mrows_q_gw<1>(stream, A, Wq, S, Y, M, N, group_shift, zp, zero_points, num_cu);
        case 2: return launch_mrows_q_gw<2>(stream, A, Wq, S, Y, M, N, group_shift, zp, zero_points, num_cu);
        default: return launch_mrows_q_gw<4>(stream, A, Wq, S, Y, M, N, group_shift, zp, zero_points, num_cu);
        }
    }

    namespace
    {
        template <int GW, int STEPS, int GSHIFT, bool ZPT, int MB>
        hipError_t launch_mrows_q8_mb(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M, int N, int zp,
                                      const void* zps, int num_cu)
        {
            if constexpr (((GW * 64) >> GSHIFT) < 2 || (MB == 2 && GW * STEPS > 8))
                return hipErrorInvalidValue;
            else
            {
                const int n_tiles = (N + 15) / 16;
                const int grid = n_tiles < num_cu ? n_tiles : num_cu;
                const int tiles_q = n_tiles / grid, tiles_r = n_tiles % grid;
                const size_t lds = workspace::w8a16_mrows_q_lds_bytes(GW * 512 * STEPS, M, tiles_q + (tiles_r ? 1 : 0), GSHIFT, ZPT);
                if (lds > MAX_LDS_BYTES)
                    return hipErrorInvalidValue;
                auto kernel = &w8a16_mrows_q_kernel<GW, STEPS, GSHIFT, ZPT, MB>;
                if (lds > 64 * 1024)
                {
                    static LdsGrant granted;
                    const hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), granted, (int)MAX_LDS_BYTES);
                    if (e != hipSuccess)
                        return e;
                }
                hipLaunchKernelGGL(kernel, dim3(grid), dim3(MR_WAVES * 64), lds, stream, (const half_t*)A, (const uint8_t*)Wq,
                                   (const half_t*)S, (half_t*)Y, (const uint8_t*)zps, N, tiles_q, tiles_r, M | (zp << 8));
                return hipGetLastError();
            }
        }
        template <int GW, int STEPS, int GSHIFT, bool ZPT>
        hipError_t launch_mrows_q8(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M, int N, int zp,
                                   const void* zps, int num_cu)
        {
            return M <= 16 ? launch_mrows_q8_mb<GW, STEPS, GSHIFT, ZPT, 1>(stream, A, Wq, S, Y, M, N, zp, zps, num_cu)
                           : launch_mrows_q8_mb<GW, STEPS, GSHIFT, ZPT, 2>(stream, A, Wq, S, Y, M, N, zp, zps, num_cu);
        }
        template <int GW, int STEPS>
        hipError_t launch_mrows_q8_gw(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M, int N,
                                      int group_shift, int zp, const void* zps, int num_cu)
        {
            switch (group_shift * 2 + (zps ? 1 : 0))
            {
            case 10: return launch_mrows_q8<GW, STEPS, 5, false>(stream, A, Wq, S, Y, M, N, zp, zps, num_cu);
            case 11: return launch_mrows_q8<GW, STEPS, 5, true>(stream, A, Wq, S, Y, M, N, zp, zps, num_cu);
            case 12: return launch_mrows_q8<GW, STEPS, 6, false>(stream, A, Wq, S, Y, M, N, zp, zps, num_cu);
            case 13: return launch_mrows_q8<GW, STEPS, 6, true>(stream, A, Wq, S, Y, M, N, zp, zps, num_cu);
            case 14: return launch_mrows_q8<GW, STEPS, 7, false>(stream, A, Wq, S, Y, M, N, zp, zps, num_cu);
            case 15: return launch_mrows_q8<GW, STEPS, 7, true>(stream, A, Wq, S, Y, M, N, zp, zps, num_cu);
            default: return hipErrorInvalidValue;
            }
        }
    } // namespace

    bool w8a16_mrows_q_supported(int M, int N, int K, int group_shift, bool zero_points, int num_cu)
    {
        return workspace::w8a16_mrows_q_fits(M, N, K, group_shift, zero_points, num_cu);
    }

    hipError_t launch_w8a16_mrows_q(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M, int N,
                                    int K, int group_shift, int zp, const void* zero_points, int num_cu)
    {
        if (!w8a16_mrows_q_supported(M, N, K, group_shift, zero_points != nullptr, num_cu))
            return hipErrorInvalidValue;
        switch (K)
        {
        case 2048: return launch_mrows_q8_gw<2, 2>(stream, A, Wq, S, Y, M, N, group_shift, zp, zero_points, num_cu);
        case 4096: return launch_mrows_q8_gw<4, 2>(stream, A, Wq, S, Y, M, N, group_shift, zp, zero_points, num_cu);
        default: return launch_mrows_q8_gw<4, 4>(stream, A, Wq, S, Y, M, N, group_shift, zp, zero_points, num_cu);
        }
    }

    namespace
    {
        template <int GW, int GSHIFT, bool ZPT>
        hipError_t launch_mrows_q_any(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M, int N, int K,
                                      int zp, const void* zps, float* partial, int ranges, int range_blocks, int num_cu)
        {
            const int n_tiles = (N + 15) / 16;
            const int per_range = num_cu / ranges > 0 ? num_cu / ranges : 1;
            const int grid = n_tiles < per_range ? n_tiles : per_range;
            const int tiles_q = n_tiles / grid, tiles_r = n_tiles % grid;
            const size_t lds = workspace::w4a16_mrows_q_any_lds_bytes(GW, M, tiles_q + (tiles_r ? 1 : 0), GSHIFT, ZPT);
            if (lds > MAX_LDS_BYTES)
                return hipErrorInvalidValue;
            auto kernel = &w4a16_mrows_q_any_kernel<GW, GSHIFT, ZPT>;
            if (lds > 64 * 1024)
            {
                static LdsGrant granted;
                const hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), granted, (int)MAX_LDS_BYTES);
                if (e != hipSuccess)
                    return e;
            }
            hipLaunchKernelGGL(kernel, dim3(grid, ranges), dim3(MR_WAVES * 64), lds, stream, (const half_t*)A, (const uint8_t*)Wq,
                               (const half_t*)S, (half_t*)Y, (const uint8_t*)zps, ranges > 1 ? partial : nullptr, N, K, range_blocks,
                               tiles_q, tiles_r, M | (zp << 8));
            return hipGetLastError();
        }
        template <int GW>
        hipError_t launch_mrows_q_any_gw(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M, int N,
                                         int K, int group_shift, int zp, const void* zps, float* partial, int ranges,
                                         int range_blocks, int num_cu)
        {
            switch (group_shift * 2 + (zps ? 1 : 0))
            {
#define NNF_Q_ANY(GS, Z)                                                                                                          \
    return launch_mrows_q_any<GW, GS, Z>(stream, A, Wq, S, Y, M, N, K, zp, zps, partial, ranges, range_blocks, num_cu)
            case 10: NNF_Q_ANY(5, false);
            case 11: NNF_Q_ANY(5, true);
            case 12: NNF_Q_ANY(6, false);
            case 13: NNF_Q_ANY(6, true);
            case 15: NNF_Q_ANY(7, true);
#undef NNF_Q_ANY
            default: return hipErrorInvalidValue; // groups of 128 with a scalar zero point: w4a16_mrows_any_kernel
            }
        }
    } // namespace

    // ranges of K of the run-time-K form: 0 does not apply, 1 straight to Y, more: fp32 sums to partial[ranges][M][N] (the
    // caller runs the reduction pass)
    int w4a16_mrows_q_any_ranges(int M, int N, int K, int group_shift, bool zero_points, int num_cu)
    {
        if (group_shift == 7 && !zero_points)
            return 0;
        return workspace::w4a16_mrows_q_any_plan(M, N, K, group_shift, zero_points, num_cu).ranges;
    }

    hipError_t launch_w4a16_mrows_q_any(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, float* partial,
                                        int M, int N, int K, int group_shift, int zp, const void* zero_points, int num_cu)
    {
        const workspace::MrowsQAny pl = workspace::w4a16_mrows_q_any_plan(M, N, K, group_shift, zero_points != nullptr, num_cu);
        if (pl.ranges < 1 || (pl.ranges > 1 && !partial) || (group_shift == 7 && !zero_points))
            return hipErrorInvalidValue;
        switch (pl.gw)
        {
        case 2: return launch_mrows_q_any_gw<2>(stream, A, Wq, S, Y, M, N, K, group_shift, zp, zero_points, partial, pl.ranges, pl.range_blocks, num_cu);
        case 3: return launch_mrows_q_any_gw<3>(stream, A, Wq, S, Y, M, N, K, group_shift, zp, zero_points, partial, pl.ranges, pl.range_blocks, num_cu);
        default: return launch_mrows_q_any_gw<4>(stream, A, Wq, S, Y, M, N, K, group_shift, zp, zero_points, partial, pl.ranges, pl.range_blocks, num_cu);
        }
    }

    // K above 8192 (a multiple of 256, 2 <= M <= 16): the run-time-K kernel over ranges of K, fp32 sums to
    // partial[ranges][M][N] (the caller runs the reduction pass).  Returns the number of ranges; 0: does not apply.
    int w4a16_mrows_ksplits(int M, int N, int K, int num_cu) { return workspace::w4a16_mrows_split(M, N, K, num_cu).ranges; }

    size_t w4a16_mrows_split_sync_bytes(int num_cu) { return workspace::mrows_split_sync_bytes(num_cu); }

    hipError_t launch_w4a16_mrows_split(hipStream_t stream, const void* A, const void* Wq, const void* S, float* partial, int M,
                                        int N, int K, int zp, int num_cu, const void* gamma, void* Y, const GemvFusion* epilogue,
                                        uint32_t* sync)
    {
        // Of the fused parts only the RMSNorm weight belongs to the sums of a range.  With synchronisation words (one per
        // workgroup of a range, zero before and after) the launch adds the ranges up itself and runs `epilogue` (rstd,
        // bias, residual) on the way to Y; without them the sums stay in `partial` for the reduction pass.
        GemvFusion fusion;
        if (sync)
        {
            if (!Y || !epilogue || epilogue->gate)
                return hipErrorInvalidValue;
            fusion = *epilogue;
        }
        fusion.gamma = gamma;
        const workspace::MrowsSplit sp = workspace::w4a16_mrows_split(M, N, K, num_cu);
        if (sp.ranges < 2 || !partial)
            return hipErrorInvalidValue;
        switch (sp.gw)
        {
        case 1: return launch_mrows_any<1, 2>(stream, A, Wq, S, Y, M, N, K, zp, num_cu, fusion, partial, sp.ranges, sp.range_groups, sync);
        case 2: return launch_mrows_any<2, 2>(stream, A, Wq, S, Y, M, N, K, zp, num_cu, fusion, partial, sp.ranges, sp.range_groups, sync);
        case 3: return launch_mrows_any<3, 2>(stream, A, Wq, S, Y, M, N, K, zp, num_cu, fusion, partial, sp.ranges, sp.range_groups, sync);
        default: return launch_mrows_any<4, 2>(stream, A, Wq, S, Y, M, N, K, zp, num_cu, fusion, partial, sp.ranges, sp.range_groups, sync);
        }
    }
} // namespace nnf
