// W8A8 GEMV for a single activation row (M = 1) on gfx950:  acc[N] = W[N,K] . a  (int8 x int8 -> int32, exact),
// Y = fp16((float)acc * s_tok[0] * s_ch[n]).
//
// The int8 sibling of the row-streaming fp16 x int4 kernel (w4a16_gemv_rows.hip), with nothing to unpack:
//   * one workgroup of eight wavefronts per CU owns a contiguous run of weight rows; a wavefront works on a fixed
//     K segment of SEG KiB of whole rows (2..8 wavefronts share a row) and takes its next row from a counter in LDS;
//   * every wavefront-wide load takes 1 KiB of one row in memory order and goes global -> LDS without registers
//     (global_load_lds_dwordx4) into a private ring of D rows, waited for with explicit s_waitcnt counts;
//   * a lane meets the same 16 x SEG activations for every row: they stay in registers; the products run on
//     v_dot4_i32_i8; the 64 lanes are added with DPP (integer adds: the result does not depend on the order);
//   * results are parked in LDS; the dequantisation and the stores happen once, after the last row.
#include "nnf_device.h"
#include "nnf_launch.h"

#include "../nnf_workspace.h"

#include <type_traits>

namespace nnf
{
    namespace
    {
        // s_waitcnt with only the vector-memory counter set (gfx9 encoding: vmcnt = bits 3:0 and 15:14)
        constexpr int q8_vmcnt(int n) { return (n & 0xF) | ((n >> 4) << 14) | (0x7 << 4) | (0xF << 8); }

        template <int BEGIN, int END, class F>
        __device__ __forceinline__ void q8_static_for(F&& f)
        {
            if constexpr (BEGIN < END)
            {
                f(std::integral_constant<int, BEGIN>{});
                q8_static_for<BEGIN + 1, END>(f);
            }
        }

        typedef const void __attribute__((address_space(1))) * q8_global_ptr_t;
        typedef void __attribute__((address_space(3))) * q8_lds_ptr_t;
    } // namespace

    // LDS (bytes):  ring  [WAVES wavefronts][D rows][SEG] x 1 KiB
    //               act   the K activations as in memory, rounded up to whole KiB, then 16 bytes of zeros (what a lane
    //                     past the end of K multiplies with)
    //               out   [rows of the workgroup][KSW] int32
    //               next  [KSW] row counters
    // SEG: wavefront-wide loads (1 KiB of a row each) per row and wavefront; D: rows in flight per wavefront; WAVES:
    // wavefronts per workgroup; kshift = log2(KSW), KSW = wavefronts sharing a row.  RAW: write the int32 sums.
    // Workgroup b owns rows_q rows (one more for b < rows_r), contiguous.
    template <int SEG, int D, int WAVES, bool RAW>
    __global__ __launch_bounds__(WAVES * 64) void w8a8_gemv_rows_kernel(const int8_t* __restrict__ A,
                                                                        const int8_t* __restrict__ W,
                                                                        const float* __restrict__ s_tok,
                                                                        const float* __restrict__ s_ch,
                                                                        half_t* __restrict__ Y, int32_t* __restrict__ acc_out,
                                                                        int N, int K, int rows_q, int rows_r, int kshift)
    {
        extern __shared__ uintx4 lds[];
        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int ksw = 1 << kshift;
        const int kpart = wave & (ksw - 1);
        const int gpw = WAVES >> kshift; // wavefronts per K segment
        const int widx = wave >> kshift; // this one among them
        const int out0 = (int)blockIdx.x * rows_q + min((int)blockIdx.x, rows_r);
        const int n_rows = rows_q + ((int)blockIdx.x < rows_r ? 1 : 0); // >= 1: the grid never exceeds N
        const uint32_t row_bytes = (uint32_t)K;
        const int a_kib = (K + 1023) >> 10; // wavefront-wide loads of activations

        uint8_t* lds_bytes = reinterpret_cast<uint8_t*>(lds);
        uint8_t* ring = lds_bytes + wave * (D * SEG * 1024);
        uint8_t* act = lds_bytes + WAVES * D * SEG * 1024;
        int* outb = reinterpret_cast<int*>(act + a_kib * 1024 + 16);
        int* next_row = outb + ((rows_q + 1) << kshift);

        // ---- activations: requested first (few loads, cache hits), once per workgroup ------------------------
        for (int i = wave; i < a_kib; i += WAVES)
        {
            const uint32_t b = (uint32_t)min(i * 1024 + lane * 16, K - 16);
            __builtin_amdgcn_global_load_lds((q8_global_ptr_t)(reinterpret_cast<const uint8_t*>(A) + (size_t)b),
                                             (q8_lds_ptr_t)(act + i * 1024), 16, 0, 0);
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
        // weights of row r (relative to the workgroup's first; rows past the end re-read the last row) -> ring slot
        auto issue = [&](int r, int slot) {
            const uint8_t* src = reinterpret_cast<const uint8_t*>(W) + (size_t)(out0 + min(r, n_rows - 1)) * row_bytes;
#pragma unroll
            for (int j = 0; j < SEG; ++j)
                __builtin_amdgcn_global_load_lds((q8_global_ptr_t)(src + w_off[j]),
                                                 (q8_lds_ptr_t)(ring + (slot * SEG + j) * 1024), 16, 0, 0);
        };
#pragma unroll
        for (int d = 0; d < D; ++d)
            issue(widx + d * gpw, d);
        __builtin_amdgcn_sched_barrier(0);
        if (tid < ksw)
            next_row[tid] = gpw * D; // the counters start behind the fixed rows
        if (tid == 0)
            *reinterpret_cast<uintx4*>(act + a_kib * 1024) = uintx4{0u, 0u, 0u, 0u};

        // ---- activations: LDS -> registers; only the weights asked for above may still be in flight ----------
        __builtin_amdgcn_s_waitcnt(q8_vmcnt(D * SEG));
        lds_barrier();
        uintx4 areg[SEG];
#pragma unroll
        for (int j = 0; j < SEG; ++j)
        {
            // a lane past the end of K gets the zeros (a lane whose 16 bytes straddle the end cannot occur: K % 16 == 0)
            const uint32_t b = valid[j] ? seg_byte0 + j * 1024 + lane * 16 : (uint32_t)a_kib * 1024u;
            areg[j] = *reinterpret_cast<const uintx4*>(act + b);
        }

        // ---- rows -------------------------------------------------------------------------------------
        const uint32_t lane16 = (uint32_t)lane * 16u;
        uintx4 wv[SEG];
        auto read_slot = [&](int slot) {
#pragma unroll
            for (int j = 0; j < SEG; ++j)
                wv[j] = *reinterpret_cast<const uintx4*>(ring + (slot * SEG + j) * 1024 + lane16);
        };
        auto compute = [&](int r) {
            int v = 0;
#pragma unroll
            for (int j = 0; j < SEG; ++j)
            {
                v = __builtin_amdgcn_sdot4((int)wv[j].x, (int)areg[j].x, v, false);
                v = __builtin_amdgcn_sdot4((int)wv[j].y, (int)areg[j].y, v, false);
                v = __builtin_amdgcn_sdot4((int)wv[j].z, (int)areg[j].z, v, false);
                v = __builtin_amdgcn_sdot4((int)wv[j].w, (int)areg[j].w, v, false);
            }
            // the 16 lanes of a row (four rotations), then the four rows: row_bcast:15 adds lane 15 of rows 0 and 2
            // into rows 1 and 3, row_bcast:31 adds lane 31 into rows 2 and 3 -- lane 63 ends up with everything
            v += __builtin_amdgcn_update_dpp(0, v, 0x128, 0xF, 0xF, false);
            v += __builtin_amdgcn_update_dpp(0, v, 0x124, 0xF, 0xF, false);
            v += __builtin_amdgcn_update_dpp(0, v, 0x122, 0xF, 0xF, false);
            v += __builtin_amdgcn_update_dpp(0, v, 0x121, 0xF, 0xF, false);
            v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xA, 0xF, false);
            v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xC, 0xF, false);
            if (lane == 63)
                outb[(r << kshift) + kpart] = v;
        };

        // The loop body is written out once per ring slot.  D rows are in flight at the top of every iteration; a
        // wavefront leaves the loop when the counter has run past the workgroup's rows, with D - 1 rows (all of them
        // real) still to come.  (D > 1 is only chosen when every wavefront has at least D rows.)
        int in_slot[D]; // the row in each ring slot
#pragma unroll
        for (int d = 0; d < D; ++d)
            in_slot[d] = widx + d * gpw;
        const uint32_t next_addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) int*)(next_row + kpart);
        if (in_slot[0] < n_rows)
        {
            int exit_slot = -1;
            while (exit_slot < 0)
            {
                q8_static_for<0, D>([&](auto sc) {
                    constexpr int slot = decltype(sc)::value;
                    if (slot == 0 || exit_slot < 0)
                    {
                        // The counter is bumped by hand: ahead of an LDS atomic that it can see, the compiler waits
                        // for every LDS-bound load in flight.  The result is there after the wait below.
                        int nx = 0;
                        if (lane == 0)
                            asm volatile("ds_add_rtn_u32 %0, %1, %2" : "=v"(nx) : "v"(next_addr), "v"(1) : "memory");
                        __builtin_amdgcn_s_waitcnt(q8_vmcnt((D - 1) * SEG));
                        read_slot(slot);
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
            q8_static_for<0, D - 1>([&](auto tc) {
                constexpr int t = decltype(tc)::value;
                int slot = exit_slot + 1 + t;
                slot = slot >= D ? slot - D : slot;
                const int row = __builtin_amdgcn_readlane(rows_by_slot, slot);
                __builtin_amdgcn_s_waitcnt(q8_vmcnt((D - 2 - t) * SEG));
                read_slot(slot);
                compute(row);
            });
        }
        __builtin_amdgcn_s_waitcnt(q8_vmcnt(0)); // nothing may land in LDS after the workgroup is gone

        // ---- outputs ------------------------------------------------------------------------------------
        lds_barrier();
        for (int r = tid; r < n_rows; r += WAVES * 64)
        {
            int sum = 0;
            for (int kp = 0; kp < ksw; ++kp)
                sum += outb[(r << kshift) + kp];
            if (RAW)
            {
                acc_out[out0 + r] = sum;
            }
            else
            {
                const float t = (float)sum * s_tok[0];
                Y[out0 + r] = f32_to_f16_two_step(t * s_ch[out0 + r]);
            }
        }
    }

    namespace
    {
        using workspace::Q8RowsPlan;

        template <int SEG, int D, bool RAW>
        hipError_t launch_q8_rows(hipStream_t stream, const void* A, const void* s_tok, const void* W, const void* s_ch,
                                  void* Y, void* acc, int N, int K, const Q8RowsPlan& p, int grid)
        {
            constexpr int WAVES = workspace::ROWS_WAVES;
            const size_t lds_total = p.lds_bytes(N, K, grid);
            if (lds_total > MAX_LDS_BYTES)
                return hipErrorInvalidValue;
            if (lds_total > 64 * 1024)
            {
                static LdsGrant granted;
                const hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(&w8a8_gemv_rows_kernel<SEG, D, WAVES, RAW>),
                                                       granted, (int)MAX_LDS_BYTES);
                if (e != hipSuccess)
                    return e;
            }
            hipLaunchKernelGGL((w8a8_gemv_rows_kernel<SEG, D, WAVES, RAW>), dim3(grid), dim3(WAVES * 64), lds_total, stream,
                               (const int8_t*)A, (const int8_t*)W, (const float*)s_tok, (const float*)s_ch, (half_t*)Y,
                               (int32_t*)acc, N, K, N / grid, N % grid, p.kshift);
            return hipGetLastError();
        }

        template <bool RAW>
        hipError_t launch_q8_rows_any(hipStream_t stream, const void* A, const void* s_tok, const void* W, const void* s_ch,
                                      void* Y, void* acc, int N, int K, int num_cu)
        {
            const Q8RowsPlan p = workspace::plan_w8a8_rows(1, N, K, num_cu, 0);
            const int grid = workspace::rows_grid(N, num_cu);
            switch (p.seg * 10 + p.depth)
            {
#define NNF_Q8_ROWS_CASE(SEG, D)                                                                                       \
    case SEG * 10 + D: return launch_q8_rows<SEG, D, RAW>(stream, A, s_tok, W, s_ch, Y, acc, N, K, p, grid);
                NNF_Q8_ROWS_CASE(1, 1)
                NNF_Q8_ROWS_CASE(1, 2)
                NNF_Q8_ROWS_CASE(1, 3)
                NNF_Q8_ROWS_CASE(1, 4)
                NNF_Q8_ROWS_CASE(2, 1)
                NNF_Q8_ROWS_CASE(2, 2)
                NNF_Q8_ROWS_CASE(2, 3)
                NNF_Q8_ROWS_CASE(2, 4)
                NNF_Q8_ROWS_CASE(3, 1)
                NNF_Q8_ROWS_CASE(3, 2)
#undef NNF_Q8_ROWS_CASE
            default: return hipErrorInvalidValue;
            }
        }
    } // namespace

    bool w8a8_gemv_rows_supported(int M, int N, int K, int num_cu)
    {
        return workspace::plan_w8a8_rows(M, N, K, num_cu).seg != 0;
    }

    // acc != nullptr: the raw int32 sums, otherwise Y = fp16(acc * s_tok[0] * s_ch[n])
    hipError_t launch_w8a8_gemv_rows(hipStream_t stream, const void* A, const void* s_tok, const void* W, const void* s_ch,
                                     void* Y, void* acc, int N, int K, int num_cu)
    {
        return acc ? launch_q8_rows_any<true>(stream, A, s_tok, W, s_ch, Y, acc, N, K, num_cu)
                   : launch_q8_rows_any<false>(stream, A, s_tok, W, s_ch, Y, acc, N, K, num_cu);
    }
} // namespace nnf
