// The body of the fp16 x int4 GEMV for a single activation row (the kernels and their launchers: w4a16_gemv_rows.hip, where
// the design is described).  A header so that the measurement probes can compile the same code once more with time
// stamps (NNF_ROWS_TRACE names a `unsigned long long*` expression: eight stamps of the 100 MHz clock per workgroup,
// those of its first wavefront, written by its first thread; the product library is built without it).
#pragma once
#include "nnf_device.h"
#include "nnf_launch.h"

#include "../nnf_workspace.h"

#include <type_traits>

#ifdef NNF_ROWS_TRACE
// The stamps stay in (scalar) registers until the end of the kernel: a store in between would take part in the counted
// waits for the weights.
#define NNF_ROWS_STAMPS unsigned long long rows_stamp[8] = {0, 0, 0, 0, 0, 0, 0, 0}
#define NNF_ROWS_STAMP(i) rows_stamp[i] = __builtin_amdgcn_s_memrealtime()
#define NNF_ROWS_STAMP_FIRST(i)                                                                                         \
    do                                                                                                                  \
    {                                                                                                                   \
        if (rows_stamp[i] == 0)                                                                                         \
            rows_stamp[i] = __builtin_amdgcn_s_memrealtime();                                                           \
    } while (0)
#define NNF_ROWS_FLUSH()                                                                                                \
    do                                                                                                                  \
    {                                                                                                                   \
        rows_stamp[7] = __builtin_amdgcn_s_memrealtime();                                                               \
        if (threadIdx.x == 0)                                                                                           \
            for (int i_ = 0; i_ < 8; ++i_)                                                                              \
                (NNF_ROWS_TRACE)[(size_t)blockIdx.x * 8 + i_] = rows_stamp[i_];                                         \
    } while (0)
#else
#define NNF_ROWS_STAMPS (void)0
#define NNF_ROWS_STAMP(i) (void)0
#define NNF_ROWS_STAMP_FIRST(i) (void)0
#define NNF_ROWS_FLUSH() (void)0
#endif

namespace nnf
{
    namespace
    {
        // s_waitcnt with only the vector-memory counter set (gfx9 encoding: vmcnt = bits 3:0 and 15:14)
        constexpr int rows_vmcnt(int n) { return (n & 0xF) | ((n >> 4) << 14) | (0x7 << 4) | (0xF << 8); }

        // f(integral_constant<int, I>) for I = BEGIN .. END-1 (the wait counts below must be compile-time constants)
        template <int BEGIN, int END, class F>
        __device__ __forceinline__ void static_for(F&& f)
        {
            if constexpr (BEGIN < END)
            {
                f(std::integral_constant<int, BEGIN>{});
                static_for<BEGIN + 1, END>(f);
            }
        }

        typedef const void __attribute__((address_space(1))) * global_ptr_t;
        typedef void __attribute__((address_space(3))) * lds_ptr_t;
    } // namespace

    // LDS (bytes):  ring   [WAVES wavefronts][D rows][SEG] x 1 KiB
    //               act    K/8 16-byte units a[8u .. 8u+8), rounded up to whole KiB: first as in memory, then
    //                      as (a0,a4) (a1,a5) (a2,a6) (a3,a7); followed by four units of zeros (what a
    //                      lane past the end of K multiplies with)
    //               corr   one fp32 per unit: its part of the constant that the nibble trick adds to a row
    //               scales [rows of the workgroup][K/128] fp16 as in memory, rounded up to whole KiB
    //               out    [rows of the workgroup][KSW] fp32
    //               next   [KSW] row counters
    // SEG: wavefront-wide loads (1 KiB of a row each) per row and wavefront; D: rows in flight per wavefront;
    // WAVES: wavefronts per workgroup (one workgroup per CU).
    // pack = zp | log2(KSW) << 8, KSW = wavefronts sharing a row (each a segment of SEG KiB).
    // Workgroup b owns rows_q outputs (one more for b < rows_r), contiguous.
    // EPI: 0 plain; 1 the optional parts of `f` (RMSNorm: gamma onto the activations, rstd onto the sums; bias;
    // residual); 2 SiLU-gate (N outputs from 2 N weight rows: the workgroup walks the gate rows of its outputs, then
    // their up rows N further down; scales: two blocks in LDS) with the optional RMSNorm; 4 and 3: other block
    // parameters, pack = zp | log2(KSW) << 8 | log2(group) << 16 with groups of 32 / 64 / 128 (a lane's 32 weights of a
    // load lie in one group whatever its size: only the place of its scale changes) and, for 3, a zero point per
    // (row, group) in `zps`, u8 [N, (K / group + 1) / 2], even group in the low nibble.  With the weights of a row a
    // wavefront then fetches the bytes that hold the zero points of its K segment (one byte per lane, global -> LDS like
    // the weights: 256 bytes more per ring slot and 64 groups, waited for with the weights), and the constant part of a
    // lane's sum becomes  base - z (sum of the lane's activations),  base the constant for z = 0; both stay in registers.
    // BITS = 8 (with EPI 3 / 4 only): a row is K bytes, a lane's 16 bytes of a load are 16 weights (two units of
    // activations, kept in memory order), a byte b becomes 1024 + b with one v_perm_b32 per pair (0x64 above it: the
    // mantissa of 1024.0), and `zps` holds one byte per (row, group).
    template <int SEG, int D, int WAVES, int EPI, int BITS = 4>
    __device__ __forceinline__ void gemv_rows_body(const half_t* __restrict__ A, const uint8_t* __restrict__ Wq,
                                                   const half_t* __restrict__ S, half_t* __restrict__ Y, int N, int K,
                                                   int rows_q, int rows_r, int pack, const GemvFusionArgs& f,
                                                   const uint8_t* __restrict__ zps = nullptr)
    {
        constexpr bool GATE = EPI == 2;
        constexpr bool QZT = EPI == 3;            // zero points from `zps`
        constexpr bool QG = EPI == 3 || EPI == 4; // group size from `pack`
        constexpr bool W8 = BITS == 8;
        static_assert(BITS == 4 || (W8 && QG), "8-bit weights: the kernels for other block parameters only");
        constexpr int LOAD_K = W8 ? 1024 : 2048; // weights per wavefront-wide load
        constexpr int LANE_K = LOAD_K / 64;      // ... and lane
        constexpr int UPL = LANE_K / 8;          // units of activations a lane meets per load
        constexpr int ZL = QZT ? (SEG + 1) / 2 : 0; // loads of zero points per row and wavefront (64 bytes = 128 groups each;
                                                    // a segment of SEG KiB of weights has at most 64 SEG groups)
        constexpr int LPR = SEG + ZL;               // vector-memory loads per row and wavefront
        constexpr int SLOT_BYTES = SEG * 1024 + ZL * 256;
        const int gshift = QG ? (pack >> 16) : 7;
        extern __shared__ uintx4 lds[];
        uint32_t MAGIC, MAGIC_HI, MASK_LO, MASK_HI;
        asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(MAGIC));
        asm volatile("v_mov_b32 %0, 0x54005400" : "=v"(MAGIC_HI));
        asm volatile("s_mov_b32 %0, 0x000F000F" : "=s"(MASK_LO));
        asm volatile("s_mov_b32 %0, 0x00F000F0" : "=s"(MASK_HI));
        NNF_ROWS_STAMPS;
        NNF_ROWS_STAMP(0); // the workgroup runs
        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int zp = pack & 0xff, kshift = QG ? (pack >> 8) & 0xff : pack >> 8;
        const int ksw = 1 << kshift;
        const int kpart = wave & (ksw - 1);
        const int gpw = WAVES >> kshift; // wavefronts per K segment
        const int widx = wave >> kshift; // this one among them
        const int out0 = (int)blockIdx.x * rows_q + min((int)blockIdx.x, rows_r);
        const int n_out = rows_q + ((int)blockIdx.x < rows_r ? 1 : 0); // >= 1: the grid never exceeds N
        const int n_rows = GATE ? 2 * n_out : n_out;                   // weight rows this workgroup walks
        const uint32_t row_bytes = W8 ? (uint32_t)K : (uint32_t)K >> 1;
        const int G = K >> gshift;
        const int a_units = K >> 3;
        const int a_pad = (a_units + 63) & ~63; // whole wavefront-wide loads of activations
        const int sc_bytes = n_out * G * 2;     // this workgroup's block of S (GATE: one such block for the gate rows,
                                                // one for the up rows)
        const int sc_block = (((rows_q + 1) * G * 2) + 1023) & ~1023; // LDS bytes of a block
        // weight row r of the workgroup (relative) -> row of Wq / S
        auto phys_row = [&](int r) { return (GATE && r >= n_out) ? N + out0 + (r - n_out) : out0 + r; };

        uint8_t* lds_bytes = reinterpret_cast<uint8_t*>(lds);
        uint8_t* ring = lds_bytes + wave * (D * SLOT_BYTES);
        uintx4* act = lds + (WAVES * D * SLOT_BYTES) / 16;
        float* corr = reinterpret_cast<float*>(act + a_pad + 4);
        float* asum_u = corr + a_pad + 4; // QZT: one fp32 per unit, the sum of its eight activations
        uint8_t* scales = reinterpret_cast<uint8_t*>(corr + (QZT ? 2 : 1) * (a_pad + 4));
        float* outb = reinterpret_cast<float*>(scales + (GATE ? 2 : 1) * sc_block);
        int* next_row = reinterpret_cast<int*>(outb + (((GATE ? 2 : 1) * (rows_q + 1)) << kshift));
        float* sum_sq = reinterpret_cast<float*>(next_row + 8); // per wavefront: its share of sum a^2 (RMSNorm inside the kernel)
        const bool own_rstd = EPI != 0 && f.gamma && !f.rstd;

        // ---- activations and scales: requested first (few loads, cache hits), once per workgroup ------------
        // (global -> LDS like the weights: a load into registers followed by an LDS write would be made to wait
        // for every LDS-bound load in flight, i.e. for the first weights)
        const bool a_loader = wave * 64 < a_units; // this wavefront fetches a share of the activations
        for (int u0 = wave * 64; u0 < a_units; u0 += WAVES * 64)
        {
            const uint32_t u = (uint32_t)min(u0 + lane, a_units - 1);
            __builtin_amdgcn_global_load_lds((global_ptr_t)(reinterpret_cast<const uint8_t*>(A) + (size_t)(u * 16u)),
                                             (lds_ptr_t)(reinterpret_cast<uint8_t*>(act) + u0 * 16), 16, 0, 0);
        }
#pragma unroll
        for (int half = 0; half < (GATE ? 2 : 1); ++half)
        {
            // whole KiB of the block with 16 bytes per lane, the rest (a multiple of 4 bytes) with 4 bytes per
            // lane, lanes past the end re-reading its last word: nothing is read beyond the block
            const uint8_t* blk = reinterpret_cast<const uint8_t*>(S) + (size_t)(out0 + half * N) * G * 2;
            uint8_t* dst = scales + half * sc_block;
            const int full = sc_bytes >> 10;
            for (int i = wave; i < full; i += WAVES)
                __builtin_amdgcn_global_load_lds((global_ptr_t)(blk + i * 1024 + lane * 16), (lds_ptr_t)(dst + i * 1024), 16, 0,
                                                 0);
            const int tail_loads = ((sc_bytes & 1023) + 255) >> 8;
            for (int t = wave; t < tail_loads; t += WAVES)
            {
                const int off = full * 1024 + t * 256;
                __builtin_amdgcn_global_load_lds((global_ptr_t)(blk + min(off + lane * 4, sc_bytes - 4)),
                                                 (lds_ptr_t)(dst + off), 4, 0, 0);
            }
        }
        // RMSNorm weight of the units this lane prepares below: into registers, ahead of the weights (vector-memory
        // operations complete in order: the wait for the activations covers them)
        constexpr int GQ = EPI != 0 ? 2048 / (WAVES * 64) : 1; // units per lane at the largest K
        uintx4 gq[GQ];
        if (EPI != 0 && f.gamma)
        {
#pragma unroll
            for (int e = 0; e < GQ; ++e)
            {
                const int u = min(wave * 64 + e * (WAVES * 64) + lane, a_units - 1);
                gq[e] = reinterpret_cast<const uintx4*>(f.gamma)[u];
            }
        }

        // ---- this wavefront's K segment; its first D rows are fixed: widx, widx + gpw, ... ---------------------
        const uint32_t seg_byte0 = (uint32_t)kpart * (SEG * 1024);
        uint32_t w_off[SEG]; // byte offset within a row
        bool valid[SEG];
#pragma unroll
        for (int j = 0; j < SEG; ++j)
        {
            const uint32_t b = seg_byte0 + j * 1024 + lane * 16;
            valid[j] = b < row_bytes;
            w_off[j] = min(b, row_bytes - 16u);
        }
        // zero points: the first byte of this wavefront's K segment in a row of `zps` (a segment starts at an even
        // group), the byte each lane fetches (past the end of the row: its last byte), and where a lane finds the zero
        // point of its load j afterwards: byte (one per lane and four bytes of LDS) and nibble
        const int zp_stride = W8 ? G : (G + 1) >> 1;
        const int g_seg0 = (kpart * SEG * LOAD_K) >> gshift;
        uint32_t z_off[ZL > 0 ? ZL : 1], z_rd[SEG], z_sh[SEG];
        if constexpr (QZT)
        {
#pragma unroll
            for (int i = 0; i < ZL; ++i)
                z_off[i] = (uint32_t)min((W8 ? g_seg0 : g_seg0 >> 1) + i * 64 + lane, zp_stride - 1);
#pragma unroll
            for (int j = 0; j < SEG; ++j)
            {
                const int g = min(g_seg0 + ((j * LOAD_K + lane * LANE_K) >> gshift), G - 1);
                z_rd[j] = W8 ? (uint32_t)(g - g_seg0) * 4u : (uint32_t)((g >> 1) - (g_seg0 >> 1)) * 4u;
                z_sh[j] = W8 ? 0u : (uint32_t)(g & 1) * 4u;
            }
        }
        // weights of row r (relative to the workgroup's first; rows past the end re-read the last row) -> ring slot
        auto issue = [&](int r, int slot) {
            const int row = phys_row(min(r, n_rows - 1));
            const uint8_t* src = Wq + (size_t)row * row_bytes;
#pragma unroll
            for (int j = 0; j < SEG; ++j)
                __builtin_amdgcn_global_load_lds((global_ptr_t)(src + w_off[j]),
                                                 (lds_ptr_t)(ring + slot * SLOT_BYTES + j * 1024), 16, 0, 0);
            if constexpr (QZT)
            {
                const uint8_t* zsrc = zps + (size_t)row * zp_stride;
#pragma unroll
                for (int i = 0; i < ZL; ++i)
                    __builtin_amdgcn_global_load_lds((global_ptr_t)(zsrc + z_off[i]),
                                                     (lds_ptr_t)(ring + slot * SLOT_BYTES + SEG * 1024 + i * 256), 1, 0, 0);
            }
        };
        // (two rows now; the rest of the ring after the activations are in registers: with everything asked for at
        // once the last wavefronts stall at issue -- a CU takes about 64 wavefront-wide loads -- and hold up the barrier)
        constexpr int D0 = D < 2 ? D : 2;
#pragma unroll
        for (int d = 0; d < D0; ++d)
            issue(widx + d * gpw, d);
        __builtin_amdgcn_sched_barrier(0);
        if (tid < ksw)
            next_row[tid] = gpw * D; // the counters start behind the fixed rows
        if (tid < 4)
        {
            act[a_pad + tid] = uintx4{0u, 0u, 0u, 0u};
            corr[a_pad + tid] = 0.f;
            if (QZT)
                asum_u[a_pad + tid] = 0.f;
        }
        // where the lane finds the scale of its load j in a row of scales (a lane past the end of K: the last one)
        uint32_t s_rd[SEG];
#pragma unroll
        for (int j = 0; j < SEG; ++j)
            s_rd[j] = QG ? (uint32_t)min((kpart * SEG * LOAD_K + j * LOAD_K + lane * LANE_K) >> gshift, G - 1) * 2u
                         : (uint32_t)min(kpart * SEG * 16 + j * 16 + (lane >> 2), G - 1) * 2u;

        // ---- activations: prepared once per workgroup, then LDS -> registers ------------------------------
        // A lane of a fetching wavefront gets back exactly the unit it asked for (no barrier needed for that):
        // it stores the unit as (a0,a4) (a1,a5) (a2,a6) (a3,a7) and, next to it, the unit's part of the
        // constant  (1024 + zp) sum a_even + (64 + zp) sum a_odd  that the nibble trick adds to every row.
        // Only the weights asked for above may still be in flight afterwards: the scales have landed too.
        __builtin_amdgcn_s_waitcnt(rows_vmcnt(D0 * LPR));
        NNF_ROWS_STAMP(1); // activations and scales have arrived
        if (a_loader)
        {
            const float ce = -(1024.0f + (QZT ? 0.f : (float)zp));
            const float co = W8 ? ce : -(64.0f + (QZT ? 0.f : (float)zp));
            float ss = 0.f;
            int e = 0;
            for (int u0 = wave * 64; u0 < a_units; u0 += WAVES * 64, ++e)
            {
                const int u = u0 + lane;
                uintx4 raw = act[u];
                if (own_rstd && u < a_units)
                {
                    // RMSNorm without a pass of its own: every unit of the row goes through exactly one lane here
                    const uint32_t rr[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                    {
                        const half2_t hh = as_half2(rr[i]);
                        ss += (float)hh.x * (float)hh.x + (float)hh.y * (float)hh.y;
                    }
                }
                if (EPI != 0 && f.gamma)
                {
                    // fp16(a * gamma): the product of two fp16 values, rounded once
                    uintx4 g = gq[0];
#pragma unroll
                    for (int i = 1; i < GQ; ++i)
                        g = e == i ? gq[i] : g;
                    raw.x = as_u32(as_half2(raw.x) * as_half2(g.x));
                    raw.y = as_u32(as_half2(raw.y) * as_half2(g.y));
                    raw.z = as_u32(as_half2(raw.z) * as_half2(g.z));
                    raw.w = as_u32(as_half2(raw.w) * as_half2(g.w));
                }
                const uintx4 a = W8 ? raw : permute_a8(raw);
                const half2_t x = as_half2(a.x), y = as_half2(a.y), z = as_half2(a.z), w = as_half2(a.w);
                const float se = ((float)x.x + (float)x.y) + ((float)z.x + (float)z.y);
                const float so = ((float)y.x + (float)y.y) + ((float)w.x + (float)w.y);
                act[u] = a;
                corr[u] = ce * se + co * so;
                if (QZT)
                    asum_u[u] = se + so;
            }
            if (own_rstd)
            {
                ss = row16_sum(ss);
                ss += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, ss), 0x142, 0xA, 0xF, false));
                ss += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, ss), 0x143, 0xC, 0xF, false));
                if (lane == 63)
                    sum_sq[wave] = ss;
            }
        }
        lds_barrier();
        NNF_ROWS_STAMP(2); // every wavefront has prepared its share of the activations
        uintx4 areg[SEG][UPL];
        float ncorr[SEG], asum[SEG];
#pragma unroll
        for (int j = 0; j < SEG; ++j)
        {
            // 4 (8) bytes of weights per unit; a lane past the end of K gets the zeros
            const int u0 = valid[j] ? (int)((seg_byte0 + j * 1024 + lane * 16) >> (W8 ? 3 : 2)) : a_pad;
            if constexpr (W8)
            {
                const floatx2 c2 = *reinterpret_cast<const floatx2*>(corr + u0);
                ncorr[j] = c2.x + c2.y;
                if constexpr (QZT)
                {
                    const floatx2 s2 = *reinterpret_cast<const floatx2*>(asum_u + u0);
                    asum[j] = s2.x + s2.y;
                }
            }
            else
            {
                const floatx4 c4 = *reinterpret_cast<const floatx4*>(corr + u0);
                ncorr[j] = (c4.x + c4.y) + (c4.z + c4.w);
                if constexpr (QZT)
                {
                    const floatx4 s4 = *reinterpret_cast<const floatx4*>(asum_u + u0);
                    asum[j] = (s4.x + s4.y) + (s4.z + s4.w);
                }
            }
#pragma unroll
            for (int d = 0; d < UPL; ++d)
                areg[j][d] = act[u0 + d];
        }

        // ---- rows -------------------------------------------------------------------------------------
        const uint32_t lane16 = (uint32_t)lane * 16u;
        uintx4 wv[SEG];
        float sv[SEG], zv[SEG];
        auto read_slot = [&](int r, int slot) {
            const uint8_t* sc_row = scales + ((GATE && r >= n_out) ? sc_block + (r - n_out) * (G * 2) : r * (G * 2));
#pragma unroll
            for (int j = 0; j < SEG; ++j)
            {
                wv[j] = *reinterpret_cast<const uintx4*>(ring + slot * SLOT_BYTES + j * 1024 + lane16);
                sv[j] = (float)*reinterpret_cast<const half_t*>(sc_row + s_rd[j]);
                if constexpr (QZT)
                    zv[j] = (float)(((uint32_t)ring[slot * SLOT_BYTES + SEG * 1024 + z_rd[j]] >> z_sh[j]) & (W8 ? 255u : 15u));
            }
        };
        auto compute = [&](int r) {
            float v = 0.f;
#pragma unroll
            for (int j = 0; j < SEG; ++j)
            {
                const uint32_t ww[4] = {wv[j].x, wv[j].y, wv[j].z, wv[j].w};
                float t = ncorr[j];
                if constexpr (QZT)
                    t = __builtin_fmaf(-zv[j], asum[j], t);
                if constexpr (W8)
                {
                    // v_perm_b32(S0, S1, sel): selectors 0-3 pick bytes of S1, 4-7 of S0
#pragma unroll
                    for (int d = 0; d < UPL; ++d)
                    {
                        const uintx4 a = areg[j][d];
                        const uint32_t w0 = ww[2 * d], w1 = ww[2 * d + 1];
                        t = dot2(as_half2(__builtin_amdgcn_perm(0x64646464u, w0, 0x04010400u)), as_half2(a.x), t);
                        t = dot2(as_half2(__builtin_amdgcn_perm(0x64646464u, w0, 0x04030402u)), as_half2(a.y), t);
                        t = dot2(as_half2(__builtin_amdgcn_perm(0x64646464u, w1, 0x04010400u)), as_half2(a.z), t);
                        t = dot2(as_half2(__builtin_amdgcn_perm(0x64646464u, w1, 0x04030402u)), as_half2(a.w), t);
                    }
                }
                else
#pragma unroll
                for (int d = 0; d < 4; ++d)
                {
                    const uint32_t w = ww[d];
                    const uint32_t w8 = w >> 8;
                    const uintx4 a = areg[j][d];
                    t = dot2(as_half2((w & MASK_LO) | MAGIC), as_half2(a.x), t);  // 1024 + (q0, q4)
                    t = dot2(as_half2((w & MASK_HI) | MAGIC_HI), as_half2(a.y), t); // 64 + (q1, q5)
                    t = dot2(as_half2((w8 & MASK_LO) | MAGIC), as_half2(a.z), t); // 1024 + (q2, q6)
                    t = dot2(as_half2((w8 & MASK_HI) | MAGIC_HI), as_half2(a.w), t); // 64 + (q3, q7)
                }
                v = __builtin_fmaf(t, sv[j], v);
            }
            // the 16 lanes of a row, then the four rows: row_bcast:15 adds lane 15 of rows 0 and 2 into rows 1 and 3,
            // row_bcast:31 adds lane 31 into rows 2 and 3 -- lane 63 ends up with everything
            v = row16_sum(v);
            v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x142, 0xA, 0xF, false));
            v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x143, 0xC, 0xF, false));
            if (lane == 63)
                outb[(r << kshift) + kpart] = v;
        };

        // D rows are in flight at the top of every iteration; a wavefront leaves the loop when the counter has run
        // past the workgroup's rows, with D - 1 rows (all of them real) still to come.  (D > 1 is only chosen when
        // every wavefront has at least D rows.)
        // The loop body is written out once per ring slot, so that slots and the rows in them are compile-time
        // registers and addresses.
        int in_slot[D]; // the row in each ring slot
#pragma unroll
        for (int d = 0; d < D; ++d)
            in_slot[d] = widx + d * gpw;
#pragma unroll
        for (int d = D0; d < D; ++d)
            issue(in_slot[d], d);
        const uint32_t next_addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) int*)(next_row + kpart);
        if (in_slot[0] < n_rows)
        {
            int exit_slot = -1;
            while (exit_slot < 0)
            {
                static_for<0, D>([&](auto sc) {
                    constexpr int slot = decltype(sc)::value;
                    if (slot == 0 || exit_slot < 0)
                    {
                        // The counter is bumped by hand: ahead of an LDS atomic that it can see, the compiler waits
                        // for every LDS-bound load in flight.  The result is there after the wait below.
                        int nx = 0;
                        if (lane == 0)
                            asm volatile("ds_add_rtn_u32 %0, %1, %2" : "=v"(nx) : "v"(next_addr), "v"(1) : "memory");
                        __builtin_amdgcn_s_waitcnt(rows_vmcnt((D - 1) * LPR));
                        NNF_ROWS_STAMP_FIRST(3); // the first row's weights have arrived
                        read_slot(in_slot[slot], slot);
                        // the slot has been read before it is refilled
                        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(nx)::"memory");
                        nx = __builtin_amdgcn_readfirstlane(nx);
                        const bool more = nx < n_rows;
                        if (more)
                            issue(nx, slot);
                        compute(in_slot[slot]);
                        if (more)
                            in_slot[slot] = nx;
                        else
                            exit_slot = slot;
                    }
                });
            }
            // the D - 1 rows still in flight, oldest first: the slots after the one the loop was left in.  Their row
            // numbers are picked by a run-time slot: from the lanes of one register (indexed as an array they would
            // be kept in scratch memory for the whole kernel)
            int rows_by_slot = 0;
#pragma unroll
            for (int d = 0; d < D; ++d)
                rows_by_slot = lane == d ? in_slot[d] : rows_by_slot;
            static_for<0, D - 1>([&](auto tc) {
                constexpr int t = decltype(tc)::value;
                int slot = exit_slot + 1 + t;
                slot = slot >= D ? slot - D : slot;
                const int row = __builtin_amdgcn_readlane(rows_by_slot, slot);
                __builtin_amdgcn_s_waitcnt(rows_vmcnt((D - 2 - t) * LPR));
                read_slot(row, slot);
                compute(row);
            });
        }
        NNF_ROWS_STAMP(4); // this wavefront's last row is added up
        __builtin_amdgcn_s_waitcnt(rows_vmcnt(0)); // nothing may land in LDS after the workgroup is gone

        // ---- outputs ------------------------------------------------------------------------------------
        lds_barrier();
        NNF_ROWS_STAMP(5); // ... and every wavefront's
        float rs = (EPI != 0 && f.rstd) ? f.rstd[0] : 1.0f;
        if (own_rstd)
        {
            float total = 0.f;
            for (int w = 0; w * 64 < a_units && w < WAVES; ++w) // the wavefronts that fetched a share of the row
                total += sum_sq[w];
            rs = 1.0f / __builtin_sqrtf(total / (float)K + f.rms_eps);
        }
        for (int r = tid; r < n_out; r += WAVES * 64)
        {
            float y = 0.f;
            for (int kp = 0; kp < ksw; ++kp)
                y += outb[(r << kshift) + kp];
            if (EPI == 0 || QG)
                Y[out0 + r] = (half_t)y;
            else if (EPI == 1)
                Y[out0 + r] = finish_bias_residual(y * rs, f.bias, out0 + r, f.residual, (size_t)(out0 + r));
            else
            {
                float up = 0.f;
                for (int kp = 0; kp < ksw; ++kp)
                    up += outb[((r + n_out) << kshift) + kp];
                Y[out0 + r] = finish_silu_gate(y * rs, up * rs);
            }
        }
        NNF_ROWS_FLUSH(); // stamp 7: the outputs are on their way
    }
} // namespace nnf
