// W8A8 (int8 x int8 -> int32, exact) for 2 <= M <= 32 activation rows and K a multiple of 256 from 2048 to 16384
// (M <= 16; to 12288 for 17 .. 32 rows): the
// row-streaming kernel of w4a16_mrows.hip on the int8 matrix cores.
//
//   acc[M,N] = A[M,K] . W[N,K]^T  (int32, bit exact);  Y = fp16((float)acc * s_tok[m] * s_ch[n])
//
// Replaces the cublas GEMM behind cuda::Dot (src/nnfusion/core/kernels/cuda_gpu/kernels/dot.cpp:271-363) for an
// int8-quantized Dot node with a few activation rows.
//
//   * One workgroup of eight wavefronts per CU owns a contiguous run of 16-row weight tiles.  All eight work on
//     the same tile, in steps of 2 KiB of K: wavefront w owns bytes [256 w, 256 (w+1)) of every step, so that the
//     workgroup's loads of a step cover 2 KiB of each of the 16 rows without gaps.
//   * A step of a wavefront (16 rows x 256 bytes = 4 KiB) goes global -> LDS without registers
//     (global_load_lds_dwordx4, four wavefront-wide loads) into a private ring of NS slots; a slot is requested
//     again as soon as it has been copied into registers (16 VGPRs).  Nothing but the wavefront's own loads
//     feeds its MFMAs: no barrier on the load path.  The 16-byte pieces of a row are XOR-swizzled with the row
//     number on the way (each lane chooses which piece it fetches): conflict-free 128-bit operand reads.
//   * The activations never touch LDS: lane (m, kq) loads the 16 bytes of row m that its MFMA operand holds of
//     every 64-byte chunk of the wavefront's slice, once, and keeps them (K/512 x 4 VGPRs per block of 16 rows).
//   * Per step 4 (M <= 16) or 8 v_mfma_i32_16x16x64_i8, weights as the B operand.  Per tile the eight partial
//     16 x 16 (x 2) tiles meet in LDS (one LDS-only barrier, two alternating buffers), integer adds (the result
//     does not depend on the order); the sums are parked in LDS and scaled / written after the last tile.
//   * K need not fill the last step: a wavefront whose 256 bytes would lie past the end of K fetches the last
//     256 bytes of the row instead (every wavefront issues the same number of loads, which the hand-written wait
//     counts need) and multiplies them with activations of zero.
//   * LDS writes inside the loop are inline ds_write instructions: ahead of an LDS write that it can see, the
//     compiler waits for every LDS-bound load in flight.
#include "nnf_device.h"
#include "nnf_launch.h"

#include "../nnf_workspace.h"

namespace nnf
{
    namespace
    {
        constexpr int Q8MR_WAVES = 8;
        constexpr int Q8MR_STEP_BYTES = 256;                   // of a weight row, per wavefront and step
        constexpr int Q8MR_SLOT_BYTES = 16 * Q8MR_STEP_BYTES;  // 4 KiB: four wavefront-wide loads
        typedef const void __attribute__((address_space(1))) * q8mr_global_ptr_t;
        typedef void __attribute__((address_space(3))) * q8mr_lds_ptr_t;
        // s_waitcnt with only the vector-memory counter set (gfx9 encoding: vmcnt = bits 3:0 and 15:14)
        constexpr int q8mr_vmcnt(int n) { return (n & 0xF) | ((n >> 4) << 14) | (0x7 << 4) | (0xF << 8); }
    } // namespace

    // LDS (bytes): weights [8 wavefronts][NS slots][4 KiB] | partial tiles [2][8][MB KiB] |
    //              parked sums [tiles of the workgroup][M][16] int32
    // STEPS = ceil(K / 2048) (steps per tile and wavefront), MB = blocks of 16 activation rows (1 or 2), NS = ring slots.
    // A workgroup's tiles: tiles_q, one more for the first tiles_r workgroups.
    template <int STEPS, int MB, int NS, bool RAW_ACC>
    // (the arguments the first loads need come first: fourteen dwords arrive in scalar registers with the wavefront, the
    // rest -- what the epilogue needs -- is loaded from memory while the weights are on their way)
    __global__ __launch_bounds__(512) void w8a8_mrows_kernel(const int8_t* __restrict__ A, const int8_t* __restrict__ W, int M,
                                                             int N, int K, int tiles_q, int tiles_r, int ld,
                                                             const float* __restrict__ s_tok, const float* __restrict__ s_ch,
                                                             half_t* __restrict__ Y, int32_t* __restrict__ ACC,
                                                             int32_t* __restrict__ part, uint32_t* __restrict__ sync)
    {
        // K: the length of this workgroup's range of K, which starts at byte blockIdx.y * K of a row of ld bytes (one range:
        // ld = K, part = null).  Ranges: the sums of range r go to part + r * M * N, and the last workgroup of a
        // blockIdx.x to get there (sync: a zeroed word per blockIdx.x) adds them up and writes Y or ACC
        const int k0 = (int)blockIdx.y * K;
        static_assert(STEPS >= 1 && STEPS * MB <= 12 && STEPS <= 8 && (MB == 1 || MB == 2) && NS >= 2 && NS <= 4, "shape of the kernel");
        constexpr int CH = STEPS * 4;    // a wavefront's 64-byte chunks of a row (one MFMA each)
        constexpr int LPS = 4;           // loads per step and wavefront
        extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int col = lane & 15; // n within the tile (B operand / D column), m for the A operand
        const int kq = lane >> 4;  // K quarter of the MFMA operands, row quad of D
        const int b = blockIdx.x;
        const int t0 = b * tiles_q + min(b, tiles_r);
        const int T = tiles_q + (b < tiles_r ? 1 : 0);
        // the last tile of an N that is not a multiple of 16 is moved back to rows N-16 .. N-1
        auto row0_of = [&](int tile) { return __builtin_amdgcn_readfirstlane(min(tile * 16, N - 16)); };

        uint8_t* ring = smem + wave * (NS * Q8MR_SLOT_BYTES);
        uint8_t* red = smem + Q8MR_WAVES * NS * Q8MR_SLOT_BYTES; // [2][8][MB][1024]
        int32_t* parked = reinterpret_cast<int32_t*>(red + 2 * Q8MR_WAVES * MB * 1024);

        // ---- what each lane fetches -------------------------------------------------------------------------
        // Load c of a step fills bytes [c KiB, (c+1) KiB) of the slot; lane i lands at byte c*1024 + 16 i =
        // (row r = 4c + i/16, position q = i%16) of the [16][256] image and fetches piece q ^ r of that row's step.
        uint32_t w_off[LPS];
#pragma unroll
        for (int c = 0; c < LPS; ++c)
        {
            const int r = c * 4 + kq, q = col;
            w_off[c] = (uint32_t)r * (uint32_t)ld + (uint32_t)((q ^ r) << 4);
        }
        // where this wavefront's 256 bytes of step st start within a row; past the end of K: the row's last 256 bytes
        auto own_byte = [&](int st) { return st * (Q8MR_WAVES * Q8MR_STEP_BYTES) + wave * Q8MR_STEP_BYTES; };
        auto fetch_byte = [&](int st) { return min(own_byte(st), K - Q8MR_STEP_BYTES); };
        // step st (0 .. STEPS-1) of tile `tile` into slot `slot`
        auto issue = [&](int tile, int st, int slot) {
            const int8_t* wsrc = W + (size_t)row0_of(tile) * ld + k0 + fetch_byte(st);
#pragma unroll
            for (int c = 0; c < LPS; ++c)
                __builtin_amdgcn_global_load_lds((q8mr_global_ptr_t)(wsrc + w_off[c]),
                                                 (q8mr_lds_ptr_t)(ring + slot * Q8MR_SLOT_BYTES + c * 1024), 16, 0, 0);
        };

        // ---- the first NS steps, then the activations: straight into the MFMA operand registers -----------------
        // (the activations are requested last: vector-memory operations complete in order and the compiler waits
        // for them where they are used, which then also covers the first steps -- requested first, those are not
        // held back by anything)
#pragma unroll
        for (int s = 0; s < NS; ++s)
            issue(t0 + min(s / STEPS, T - 1), s % STEPS, s);
        // Two blocks of rows: through LDS as whole lines (see row_block_fetch: a block is a step's 256 bytes of 16 rows; two
        // blocks per wavefront, over what holds the partial tiles and the parked sums later -- hence the barrier behind
        // the last): N = 4096, K = 8192 at 32 rows 14.5 -> 12.3 us.  One block of rows: straight into the registers, 64
        // bytes of each row per load (half the lines of a load of 16-bit activations: the detour costs more than it saves,
        // N = K = 8192 at 8 rows 16.7 -> 18.7 us).
        uintx4 areg[MB][CH];
        if constexpr (MB == 1)
        {
            const uint8_t* a_row = reinterpret_cast<const uint8_t*>(A) + (size_t)min(col, M - 1) * (size_t)ld + k0 + kq * 16;
#pragma unroll
            for (int c = 0; c < CH; ++c)
            {
                const uintx4 v = *reinterpret_cast<const uintx4*>(a_row + fetch_byte(c >> 2) + (c & 3) * 64);
                const bool inside = own_byte(c >> 2) < K; // otherwise another wavefront covers these bytes
                areg[0][c] = inside ? v : uintx4{0u, 0u, 0u, 0u};
            }
        }
        else
        {
            uint8_t* stage = red + wave * (2 * ROW_BLOCK_BYTES);
            constexpr int NP = MB * STEPS;
            auto fetch = [&](int p) {
                const int mb = p / STEPS, st = p % STEPS;
                row_block_fetch(reinterpret_cast<const uint8_t*>(A), (size_t)ld, mb * 16, M - 1, (size_t)(k0 + fetch_byte(st)),
                                stage + (p & 1) * ROW_BLOCK_BYTES, lane);
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
                const bool inside = own_byte(p % STEPS) < K; // otherwise another wavefront covers these bytes
#pragma unroll
                for (int j = 0; j < 4; ++j)
                {
                    const uintx4 v = row_block_piece(stage + (p & 1) * ROW_BLOCK_BYTES, col, j * 4 + kq);
                    areg[p / STEPS][(p % STEPS) * 4 + j] = inside ? v : uintx4{0u, 0u, 0u, 0u};
                }
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __syncthreads();
        }

        // ---- tile loop ---------------------------------------------------------------------------------------
        // operand reads of a slot: lane (n = col, kq), chunk c of the step: piece c*4 + kq of row n
        const uint32_t rd_base = (uint32_t)col * Q8MR_STEP_BYTES;
        const uint32_t red_addr = lds_address(red) + (uint32_t)(wave * (MB * 1024) + lane * 16);
        const uint32_t parked_addr = lds_address(parked);
        // step s of the workgroup sits in slot s % NS; NS and STEPS are small: walk the slot number by hand
        int slot = 0;
        for (int it = 0; it < T; ++it)
        {
            intx4 acc[MB];
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
                acc[mb] = intx4{0, 0, 0, 0};
#pragma unroll
            for (int st = 0; st < STEPS; ++st)
            {
                // this step has landed when at most the NS-1 steps requested after it are outstanding
                __builtin_amdgcn_s_waitcnt(q8mr_vmcnt((NS - 1) * LPS));
                uintx4 wv[4];
                {
                    const uint8_t* sl = ring + slot * Q8MR_SLOT_BYTES + rd_base;
#pragma unroll
                    for (int c = 0; c < 4; ++c)
                        wv[c] = *reinterpret_cast<const uintx4*>(sl + (((c * 4 + kq) ^ col) << 4));
                }
                // the slot has been read before it is refilled: step s + NS (past the end: a valid tile again, so
                // that the wait count above holds for every step)
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                issue(t0 + min(it + (st + NS) / STEPS, T - 1), (st + NS) % STEPS, slot);
                slot = slot + 1 == NS ? 0 : slot + 1;
#pragma unroll
                for (int c = 0; c < 4; ++c)
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb)
                        acc[mb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(intx4, areg[mb][st * 4 + c]),
                                                                        __builtin_bit_cast(intx4, wv[c]), acc[mb], 0, 0, 0);
            }
            // partial tiles -> LDS (D layout: lane (n = col, kq), element e: row m = 16 mb + 4 kq + e)
            const int rbuf = it & 1;
            // The accumulators come straight from the matrix cores, and the writes below are inline instructions:
            // the compiler does not count the wait states between an MFMA and an LDS instruction that reads its
            // result for them (up to 18 for this MFMA).  These no-ops, tied to the registers, stand in.
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
                asm volatile("s_nop 15\n\ts_nop 7" : "+v"(acc[mb]));
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
            {
                const uint32_t at = red_addr + (uint32_t)(rbuf * Q8MR_WAVES * MB * 1024 + mb * 1024);
                asm volatile("ds_write_b128 %0, %1" ::"v"(at), "v"(acc[mb]) : "memory");
            }
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
            // MB x 256 threads: thread (mb, e, lane') adds the eight partial sums of output
            // (m = 16 mb + 4 (lane' >> 4) + e, n = lane' & 15)
            if (tid < MB * 256)
            {
                const int mb = tid >> 8, e = (tid >> 6) & 3;
                const int32_t* rp = reinterpret_cast<const int32_t*>(red + rbuf * Q8MR_WAVES * MB * 1024 + mb * 1024) + lane * 4 + e;
                int32_t sum = 0;
#pragma unroll
                for (int w = 0; w < Q8MR_WAVES; ++w)
                    sum += rp[w * (MB * 256)];
                const int m = 16 * mb + 4 * kq + e;
                if (m < M)
                {
                    const uint32_t at = parked_addr + (uint32_t)(((it * M + m) * 16 + col) * 4);
                    asm volatile("ds_write_b32 %0, %1" ::"v"(at), "v"(sum) : "memory");
                }
            }
        }
        __builtin_amdgcn_s_waitcnt(q8mr_vmcnt(0)); // the reloads past the end, before the LDS goes away
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        // ---- flush: parked sums -> Y (scaled) or ACC ---------------------------------------------------------------
        if (part)
        {
            int32_t* mine = part + (size_t)blockIdx.y * M * N;
            for (int idx = tid; idx < T * M * 16; idx += 512)
            {
                const int n = idx & 15;
                const int im = idx >> 4;
                const int it = im / M, m = im - it * M;
                const size_t at = (size_t)m * N + min((t0 + it) * 16, N - 16) + n;
                __hip_atomic_store(mine + at, parked[idx], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            // The sums are visible to every CU (device scope, completed) before this workgroup counts itself in; the last
            // of the ranges' workgroups to arrive adds the ranges (int32: exact in any order), finishes and leaves the word
            // zero for the next launch.  Nobody waits.
            __builtin_amdgcn_s_waitcnt(q8mr_vmcnt(0));
            volatile uint32_t* arrived_before = reinterpret_cast<volatile uint32_t*>(red);
            __syncthreads();
            if (tid == 0)
                *arrived_before = atomicAdd(sync + blockIdx.x, 1u);
            __syncthreads();
            if (*arrived_before != gridDim.y - 1)
                return;
            const int ranges = (int)gridDim.y;
            for (int idx = tid; idx < T * M * 16; idx += 512)
            {
                const int n = idx & 15;
                const int im = idx >> 4;
                const int it = im / M, m = im - it * M;
                const int gn = min((t0 + it) * 16, N - 16) + n;
                if (gn < (t0 + it) * 16) // (a last tile moved back: these columns belong to the tile before it)
                    continue;
                const size_t at = (size_t)m * N + gn;
                // (the two scales requested ahead of the ranges' sums: behind them, they were one more round trip)
                float st = 1.0f, sc = 1.0f;
                if constexpr (!RAW_ACC)
                {
                    st = s_tok[m];
                    sc = s_ch[gn];
                }
                int32_t sum = 0;
                for (int r0 = 0; r0 < ranges; r0 += 4)
                {
                    int32_t v[4];
#pragma unroll
                    for (int d = 0; d < 4; ++d)
                        v[d] = __hip_atomic_load(part + (size_t)min(r0 + d, ranges - 1) * M * N + at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                    for (int d = 0; d < 4; ++d)
                        sum += r0 + d < ranges ? v[d] : 0;
                }
                if (RAW_ACC)
                    ACC[at] = sum;
                else
                    Y[at] = f32_to_f16_two_step((float)sum * st * sc);
            }
            if (tid == 0)
                atomicExch(sync + blockIdx.x, 0u);
            return;
        }
        for (int idx = tid; idx < T * M * 16; idx += 512)
        {
            const int n = idx & 15;
            const int im = idx >> 4;
            const int it = im / M, m = im - it * M;
            const int gn = min((t0 + it) * 16, N - 16) + n;
            if (RAW_ACC)
            {
                ACC[(size_t)m * N + gn] = parked[idx];
            }
            else
            {
                const float t = (float)parked[idx] * s_tok[m];
                Y[(size_t)m * N + gn] = f32_to_f16_two_step(t * s_ch[gn]);
            }
        }
    }

    namespace
    {
        template <int STEPS, int MB, int NS, bool RAW>
        hipError_t launch_q8_mrows(hipStream_t stream, const void* A, const void* s_tok, const void* W, const void* s_ch, void* Y,
                                   void* acc, int M, int N, int K, int num_cu, int ranges = 1, int ld = 0, void* part = nullptr,
                                   uint32_t* sync = nullptr)
        {
            // (ranges > 1: K is the length of a range, ld the whole row, part the room for the [ranges][M][N] sums)
            const int n_tiles = (N + 15) / 16;
            const int per_range = num_cu / ranges > 0 ? num_cu / ranges : 1;
            const int grid = n_tiles < per_range ? n_tiles : per_range;
            const int tiles_q = n_tiles / grid, tiles_r = n_tiles % grid;
            const size_t lds = workspace::w8a8_mrows_lds_bytes(M, NS, tiles_q + (tiles_r ? 1 : 0));
            if (lds > MAX_LDS_BYTES)
                return hipErrorInvalidValue;
            auto kernel = &w8a8_mrows_kernel<STEPS, MB, NS, RAW>;
            if (lds > 64 * 1024)
            {
                static LdsGrant granted;
                const hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), granted, (int)MAX_LDS_BYTES);
                if (e != hipSuccess)
                    return e;
            }
            hipLaunchKernelGGL(kernel, dim3(grid, ranges), dim3(Q8MR_WAVES * 64), lds, stream, (const int8_t*)A, (const int8_t*)W,
                               M, N, K, tiles_q, tiles_r, ld ? ld : K, (const float*)s_tok, (const float*)s_ch, (half_t*)Y,
                               (int32_t*)acc, (int32_t*)part, sync);
            return hipGetLastError();
        }

        template <int STEPS, bool RAW>
        hipError_t launch_q8_mrows_m(hipStream_t stream, const void* A, const void* s_tok, const void* W, const void* s_ch,
                                     void* Y, void* acc, int M, int N, int K, int num_cu, int ranges = 1, int ld = 0,
                                     void* part = nullptr, uint32_t* sync = nullptr)
        {
            constexpr int NS = workspace::W8A8_MROWS_SLOTS;
            if (M <= 16)
                return launch_q8_mrows<STEPS, 1, NS, RAW>(stream, A, s_tok, W, s_ch, Y, acc, M, N, K, num_cu, ranges, ld, part, sync);
            if constexpr (STEPS <= 6) // 16 VGPRs of activations per step and block of rows
                return launch_q8_mrows<STEPS, 2, NS, RAW>(stream, A, s_tok, W, s_ch, Y, acc, M, N, K, num_cu, ranges, ld, part, sync);
            return hipErrorInvalidValue;
        }

        template <bool RAW>
        hipError_t launch_q8_mrows_any(hipStream_t stream, const void* A, const void* s_tok, const void* W, const void* s_ch,
                                       void* Y, void* acc, int M, int N, int K, int num_cu, int ranges = 1, int ld = 0,
                                       void* part = nullptr, uint32_t* sync = nullptr)
        {
            switch ((K + 2047) >> 11) // steps of 2 KiB of K
            {
            case 1: return launch_q8_mrows_m<1, RAW>(stream, A, s_tok, W, s_ch, Y, acc, M, N, K, num_cu, ranges, ld, part, sync);
            case 2: return launch_q8_mrows_m<2, RAW>(stream, A, s_tok, W, s_ch, Y, acc, M, N, K, num_cu, ranges, ld, part, sync);
            case 3: return launch_q8_mrows_m<3, RAW>(stream, A, s_tok, W, s_ch, Y, acc, M, N, K, num_cu, ranges, ld, part, sync);
            case 4: return launch_q8_mrows_m<4, RAW>(stream, A, s_tok, W, s_ch, Y, acc, M, N, K, num_cu, ranges, ld, part, sync);
            case 5: return launch_q8_mrows_m<5, RAW>(stream, A, s_tok, W, s_ch, Y, acc, M, N, K, num_cu, ranges, ld, part, sync);
            case 6: return launch_q8_mrows_m<6, RAW>(stream, A, s_tok, W, s_ch, Y, acc, M, N, K, num_cu, ranges, ld, part, sync);
            case 7: return launch_q8_mrows_m<7, RAW>(stream, A, s_tok, W, s_ch, Y, acc, M, N, K, num_cu, ranges, ld, part, sync);
            default: return launch_q8_mrows_m<8, RAW>(stream, A, s_tok, W, s_ch, Y, acc, M, N, K, num_cu, ranges, ld, part, sync);
            }
        }
    } // namespace

    bool w8a8_mrows_supported(int M, int N, int K, int num_cu) { return workspace::w8a8_mrows_fits(M, N, K, num_cu); }
    bool w8a8_mrows_preferred(int M, int N, int K, int num_cu) { return workspace::w8a8_mrows_preferred(M, N, K, num_cu); }

    // acc != nullptr: the raw int32 sums, otherwise Y = fp16(acc * s_tok[m] * s_ch[n])
    hipError_t launch_w8a8_mrows(hipStream_t stream, const void* A, const void* s_tok, const void* W, const void* s_ch, void* Y,
                                 void* acc, int M, int N, int K, int num_cu, void* partial_ws, size_t partial_bytes, uint32_t* sync,
                                 size_t sync_bytes)
    {
        if (!w8a8_mrows_supported(M, N, K, num_cu))
            return hipErrorInvalidValue;
        // over two ranges of K where that pays, given the room for their sums and the words to meet at
        const int ranges = workspace::w8a8_mrows_ranges(M, N, K, num_cu);
        if (ranges > 1 && partial_ws && partial_bytes >= workspace::w8a8_mrows_ranges_bytes(M, N, K, num_cu) && sync &&
            sync_bytes >= workspace::mrows_split_sync_bytes(num_cu))
            return acc ? launch_q8_mrows_any<true>(stream, A, s_tok, W, s_ch, Y, acc, M, N, K / ranges, num_cu, ranges, K, partial_ws, sync)
                       : launch_q8_mrows_any<false>(stream, A, s_tok, W, s_ch, Y, acc, M, N, K / ranges, num_cu, ranges, K, partial_ws, sync);
        return acc ? launch_q8_mrows_any<true>(stream, A, s_tok, W, s_ch, Y, acc, M, N, K, num_cu)
                   : launch_q8_mrows_any<false>(stream, A, s_tok, W, s_ch, Y, acc, M, N, K, num_cu);
    }
} // namespace nnf
