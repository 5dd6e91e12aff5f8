// fp16 x int4 (g128) GEMV for a single activation row (M = 1) on gfx950:  y[N] = ((Wq - zp) * S) . a
//
// With one activation row there is nothing for the matrix cores to amortise, and the kernel that is
// closest to "just read the weights once" wins.  This one is built like a streaming read:
//   * a wavefront owns whole weight rows (or, for long rows, a fixed K segment of them shared by 2..16
//     wavefronts): each wavefront-wide load takes 1 KiB of one row, in memory order, so the weight
//     matrix is read as long sequential runs;
//   * the loads go global -> LDS without passing through registers (global_load_lds_dwordx4) into a
//     private ring of D rows per wavefront, D rows ahead of their use, and are waited for with explicit
//     s_waitcnt counts: wavefronts run free of each other, there is no barrier between the prologue and
//     the final flush, and no register is held by data in flight;
//   * a lane always meets the same 32 (x SEG) activations, whatever the row: they live in registers for
//     the whole kernel, already paired and pre-scaled for the nibble trick below, and nothing but the
//     weights is read per row (plus two bytes of scale per lane and load, from LDS);
//   * nibbles become fp16 with one v_and_or_b32 per pair: (q | 0x6400) = 1024 + q and, four bits up,
//     1024 + 16 q; the dot products run on v_dot2_f32_f16 (fp32 accumulate) against (a_even, a_odd / 16),
//     and the constant part  (1024 + zp) sum a_even + (64 + zp) sum a_odd  of a lane's sum is the same
//     for every row: it is computed once and used as the negative initial accumulator;
//   * the 32 weights of a lane and load share one group scale (a group of 128 is 4 lanes); the lane's
//     partial sum is multiplied by it in fp32, the 64 lanes are added with DPP row rotations, and the
//     row's result is parked in LDS; outputs are written once, after the last row.
#include "nnf_device.h"
#include "nnf_launch.h"

#include "../nnf_workspace.h"

#include <type_traits>

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

    // LDS (bytes):  ring  [16 wavefronts][D rows][SEG] x 1 KiB
    //               scale [16 wavefronts][2 chunks] x 1 KiB: chunk = RS rows x PPR 16-byte pieces of the
    //                     wavefront's K segment (the last piece of a row is moved back to end with the segment)
    //               act   K/8 16-byte units a[8u .. 8u+8), rounded up to whole KiB: first as in memory, then
    //                     as (a0,a4) (a1,a5)/16 (a2,a6) (a3,a7)/16
    //               corr  one fp32 per unit: its part of the constant that the nibble trick adds to a row
    //               out   [rows of the workgroup][KSW] fp32
    // SEG: wavefront-wide loads (1 KiB of a row each) per row and wavefront; D: rows in flight per wavefront.
    // pack = zp | log2(KSW) << 8, KSW = wavefronts sharing a row (each a segment of SEG KiB).
    // Rows are dealt to the wavefront groups in contiguous runs: rows_q each, one more for the first rows_r.
    template <int SEG, int D>
    __global__ __launch_bounds__(1024) void w4a16_gemv_rows_kernel(const half_t* __restrict__ A,
                                                                   const uint8_t* __restrict__ Wq,
                                                                   const half_t* __restrict__ S,
                                                                   half_t* __restrict__ Y, int N, int K, int rows_q,
                                                                   int rows_r, int pack)
    {
        extern __shared__ uintx4 lds[];
        uint32_t MAGIC, MASK_LO, MASK_HI;
        asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(MAGIC));
        asm volatile("s_mov_b32 %0, 0x000F000F" : "=s"(MASK_LO));
        asm volatile("s_mov_b32 %0, 0x00F000F0" : "=s"(MASK_HI));
        constexpr int PPR = 2 * SEG;  // 16-byte scale pieces per row and segment
        constexpr int RS = 64 / PPR;  // rows per scale chunk (one wavefront-wide load)
        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int zp = pack & 0xff, kshift = pack >> 8;
        const int ksw = 1 << kshift;
        const int kpart = wave & (ksw - 1);
        const int gpw = 16 >> kshift; // wavefront groups per workgroup
        const int gid = (int)blockIdx.x * gpw + (wave >> kshift);
        const int row_start = gid * rows_q + min(gid, rows_r);
        const int count = rows_q + (gid < rows_r ? 1 : 0);
        const uint32_t row_bytes = (uint32_t)K >> 1;
        const int G = K >> 7;

        uint8_t* lds_bytes = reinterpret_cast<uint8_t*>(lds);
        uint8_t* ring = lds_bytes + wave * (D * SEG * 1024);
        uint8_t* sc_slots = lds_bytes + 16 * D * SEG * 1024 + wave * 2048;
        uintx4* act = lds + (16 * D * SEG * 1024 + 16 * 2048) / 16;
        const int a_pad = ((K >> 3) + 63) & ~63; // whole wavefront-wide loads of activations
        float* outb = reinterpret_cast<float*>(act + a_pad) + a_pad;

        // ---- activations: requested first (few loads, cache hits), once per workgroup, as they are -------
        // (also global -> LDS: a load into registers followed by an LDS write would be made to wait for
        // every LDS-bound load in flight, i.e. for the first weights)
        const int a_units = K >> 3;
        bool a_loader = false; // this wavefront fetches a share
#pragma unroll
        for (int e = 0; e < 2; ++e) // K <= 16384: at most two rounds of 1024 units
        {
            const int u0 = e * 1024 + wave * 64;
            if (u0 < a_units)
            {
                const uint32_t u = (uint32_t)min(u0 + lane, a_units - 1);
                __builtin_amdgcn_global_load_lds((global_ptr_t)(reinterpret_cast<const uint8_t*>(A) + (size_t)(u * 16u)),
                                                 (lds_ptr_t)(reinterpret_cast<uint8_t*>(act) + u0 * 16), 16, 0, 0);
                a_loader = true;
            }
        }

        // ---- this wavefront's K segment: the first rows are requested before anything else is worked out ----
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
        // weights of the wavefront's i-th row -> ring slot (rows past the end re-read the last row)
        auto issue_weights = [&](int i, int slot) {
            const int row = min(row_start + i, N - 1);
            const uint8_t* src = Wq + (size_t)row * row_bytes;
#pragma unroll
            for (int j = 0; j < SEG; ++j)
                __builtin_amdgcn_global_load_lds((global_ptr_t)(src + w_off[j]),
                                                 (lds_ptr_t)(ring + (slot * SEG + j) * 1024), 16, 0, 0);
        };
        issue_weights(0, 0);
        __builtin_amdgcn_sched_barrier(0);

        // scales of the segment: groups [seg_g0, seg_g0 + seg_groups), seg_bytes of every row of S
        const int seg_g0 = kpart * SEG * 16;
        const int seg_groups = max(min(G - seg_g0, SEG * 16), 8); // (a segment past the end of K reads the row's last ones)
        const int seg_g0c = min(seg_g0, G - seg_groups);
        const int seg_bytes = seg_groups * 2;
        const int pieces = (seg_bytes + 15) >> 4;
        const int last_piece0 = seg_bytes - 16; // byte offset of the (moved back) last piece
        // the lane's share of a scale chunk load: row r_sc of the chunk, piece p_sc
        const int r_sc = lane / PPR, p_sc = min(lane - r_sc * PPR, pieces - 1);
        const uint32_t s_src_off = (uint32_t)seg_g0c * 2u + (uint32_t)min(p_sc * 16, last_piece0);
        auto issue_scales = [&](int chunk) {
            const int row = min(row_start + chunk * RS + r_sc, N - 1);
            const uint8_t* src = reinterpret_cast<const uint8_t*>(S) + ((size_t)row * (size_t)G * 2 + s_src_off);
            __builtin_amdgcn_global_load_lds((global_ptr_t)src, (lds_ptr_t)(sc_slots + (chunk & 1) * 1024), 16, 0, 0);
        };
        // A chunk of scales travels ahead of the weights of its first row (row 0: right behind them).
        auto issue_row = [&](int i, int slot) {
            if (i % RS == 0)
                issue_scales(i / RS);
            issue_weights(i, slot);
        };
        issue_scales(0);
#pragma unroll
        for (int d = 1; d < D; ++d)
            issue_row(d, d);
        __builtin_amdgcn_sched_barrier(0);
        // where the lane finds the scale of its load j inside a row's pieces
        uint32_t s_rd[SEG];
#pragma unroll
        for (int j = 0; j < SEG; ++j)
        {
            const int g = min(seg_g0 - seg_g0c + j * 16 + (lane >> 2), seg_groups - 1);
            const int o = g * 2;
            s_rd[j] = (uint32_t)(o >= (pieces - 1) * 16 ? (pieces - 1) * 16 + (o - last_piece0) : o);
        }

        // ---- activations: prepared once per workgroup, then LDS -> registers ------------------------------
        // A lane of a fetching wavefront gets back exactly the unit it asked for (no barrier needed for that):
        // it stores the unit as (a0,a4) (a1,a5)/16 (a2,a6) (a3,a7)/16 and, next to it, the unit's part of the
        // constant  (1024 + zp) sum a_even + (64 + zp) sum a_odd  that the nibble trick adds to every row.
        // Everything this wavefront asked for after the activations may still be in flight.
        float* corr = reinterpret_cast<float*>(act + a_pad);
        if (a_loader)
        {
            __builtin_amdgcn_s_waitcnt(rows_vmcnt(D * SEG + 1));
            const half2_t sixteenth = half2_t{(half_t)0.0625f, (half_t)0.0625f};
            const float ce = -(1024.0f + (float)zp);
            const float co = -16.0f * (64.0f + (float)zp);
#pragma unroll
            for (int e = 0; e < 2; ++e)
            {
                const int u = e * 1024 + wave * 64 + lane;
                if (e * 1024 + wave * 64 < a_units)
                {
                    uintx4 a = permute_a8(act[u]);
                    a.y = as_u32(as_half2(a.y) * sixteenth);
                    a.w = as_u32(as_half2(a.w) * sixteenth);
                    const half2_t x = as_half2(a.x), y = as_half2(a.y), z = as_half2(a.z), w = as_half2(a.w);
                    const float se = ((float)x.x + (float)x.y) + ((float)z.x + (float)z.y);
                    const float so = ((float)y.x + (float)y.y) + ((float)w.x + (float)w.y);
                    act[u] = a;
                    corr[u] = ce * se + co * so;
                }
            }
        }
        lds_barrier();
        uintx4 areg[SEG][4];
        float ncorr[SEG];
#pragma unroll
        for (int j = 0; j < SEG; ++j)
        {
            const int u0 = min((int)((seg_byte0 + j * 1024 + lane * 16) >> 2), a_units - 4); // 4 bytes of weights per unit
            const floatx4 c4 = *reinterpret_cast<const floatx4*>(corr + u0);
            ncorr[j] = valid[j] ? (c4.x + c4.y) + (c4.z + c4.w) : 0.f;
#pragma unroll
            for (int d = 0; d < 4; ++d)
                areg[j][d] = valid[j] ? act[u0 + d] : uintx4{0u, 0u, 0u, 0u};
        }

        // ---- rows -------------------------------------------------------------------------------------
        const int out0 = ((int)blockIdx.x * gpw) * rows_q + min((int)blockIdx.x * gpw, rows_r); // first row of the workgroup
        const uint32_t lane16 = (uint32_t)lane * 16u;
        auto consume = [&](int i, int slot) {
            const uint8_t* sc_row = sc_slots + ((i / RS) & 1) * 1024 + (i % RS) * (PPR * 16);
            float v = 0.f;
#pragma unroll
            for (int j = 0; j < SEG; ++j)
            {
                const uintx4 w4 = *reinterpret_cast<const uintx4*>(ring + (slot * SEG + j) * 1024 + lane16);
                const float s = (float)*reinterpret_cast<const half_t*>(sc_row + s_rd[j]);
                const uint32_t ww[4] = {w4.x, w4.y, w4.z, w4.w};
                float t = ncorr[j];
#pragma unroll
                for (int d = 0; d < 4; ++d)
                {
                    const uint32_t w = ww[d];
                    const uint32_t w8 = w >> 8;
                    const uintx4 a = areg[j][d];
                    t = dot2(as_half2((w & MASK_LO) | MAGIC), as_half2(a.x), t);  // 1024 + (q0, q4)
                    t = dot2(as_half2((w & MASK_HI) | MAGIC), as_half2(a.y), t);  // 1024 + 16 (q1, q5)
                    t = dot2(as_half2((w8 & MASK_LO) | MAGIC), as_half2(a.z), t); // 1024 + (q2, q6)
                    t = dot2(as_half2((w8 & MASK_HI) | MAGIC), as_half2(a.w), t); // 1024 + 16 (q3, q7)
                }
                v = __builtin_fmaf(t, s, v);
            }
            v = row16_sum(v);
            // the four rows of 16 lanes
            const int vb = __builtin_bit_cast(int, v);
            const float total = (__builtin_bit_cast(float, __builtin_amdgcn_readlane(vb, 0)) +
                                 __builtin_bit_cast(float, __builtin_amdgcn_readlane(vb, 16))) +
                                (__builtin_bit_cast(float, __builtin_amdgcn_readlane(vb, 32)) +
                                 __builtin_bit_cast(float, __builtin_amdgcn_readlane(vb, 48)));
            if (lane == 0)
                outb[((row_start - out0 + i) << kshift) + kpart] = total;
        };

        // Exactly D rows are in flight at the top of every iteration of the first loop; the second loop
        // drains them.  The scale loads that travel with some rows only make the waits stricter.
        int slot = 0;
        int i = 0;
        for (; i + D < count; ++i)
        {
            __builtin_amdgcn_s_waitcnt(rows_vmcnt((D - 1) * SEG));
            consume(i, slot);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // the slot has been read before it is refilled
            issue_row(i + D, slot);
            slot = slot + 1 == D ? 0 : slot + 1;
        }
        static_for<0, D>([&](auto tc) {
            constexpr int t = decltype(tc)::value;
            if (i < count)
            {
                __builtin_amdgcn_s_waitcnt(rows_vmcnt((D - 1 - t) * SEG));
                consume(i, slot);
                slot = slot + 1 == D ? 0 : slot + 1;
                ++i;
            }
        });
        __builtin_amdgcn_s_waitcnt(rows_vmcnt(0)); // nothing may land in LDS after the workgroup is gone

        // ---- outputs ------------------------------------------------------------------------------------
        lds_barrier();
        const int wg_groups_end = ((int)blockIdx.x + 1) * gpw;
        const int out_end = wg_groups_end * rows_q + min(wg_groups_end, rows_r);
        for (int r = tid; r < out_end - out0; r += 1024)
        {
            float y = 0.f;
            for (int kp = 0; kp < ksw; ++kp)
                y += outb[(r << kshift) + kp];
            Y[out0 + r] = (half_t)y;
        }
    }

    namespace
    {
        using workspace::RowsPlan;

        template <int SEG, int D>
        hipError_t launch_rows(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int N, int K,
                               int zp, const RowsPlan& p, int grid)
        {
            const int n_groups = grid * (16 >> p.kshift);
            const size_t lds_total = p.lds_bytes(N, K, grid);
            if (lds_total > MAX_LDS_BYTES)
                return hipErrorInvalidValue;
            if (lds_total > 64 * 1024)
            {
                hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&w4a16_gemv_rows_kernel<SEG, D>),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_total);
                if (e != hipSuccess)
                    return e;
            }
            hipLaunchKernelGGL((w4a16_gemv_rows_kernel<SEG, D>), dim3(grid), dim3(1024), lds_total, stream, (const half_t*)A,
                               (const uint8_t*)Wq, (const half_t*)S, (half_t*)Y, N, K, N / n_groups, N % n_groups,
                               zp | (p.kshift << 8));
            return hipGetLastError();
        }
    } // namespace

    bool w4a16_gemv_rows_supported(int M, int N, int K, int num_cu)
    {
        return workspace::plan_w4a16_rows(M, N, K, num_cu).seg != 0;
    }

    hipError_t launch_w4a16_gemv_rows(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int N,
                                      int K, int zp, int num_cu)
    {
        const RowsPlan p = workspace::plan_w4a16_rows(1, N, K, num_cu);
        switch (p.seg * 10 + p.depth)
        {
#define NNF_ROWS_CASE(SEG, D)                                                                                          \
    case SEG * 10 + D: return launch_rows<SEG, D>(stream, A, Wq, S, Y, N, K, zp, p, num_cu);
            NNF_ROWS_CASE(1, 1)
            NNF_ROWS_CASE(1, 2)
            NNF_ROWS_CASE(1, 3)
            NNF_ROWS_CASE(1, 4)
            NNF_ROWS_CASE(2, 1)
            NNF_ROWS_CASE(2, 2)
            NNF_ROWS_CASE(2, 3)
            NNF_ROWS_CASE(3, 1)
            NNF_ROWS_CASE(3, 2)
#undef NNF_ROWS_CASE
        default: return hipErrorInvalidValue;
        }
    }
} // namespace nnf
