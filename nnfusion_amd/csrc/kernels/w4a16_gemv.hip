// fp16 x int4 (g128) GEMV for skinny M on gfx950: Y[M,N] = A[M,K] . ((Wq - zp) * S)^T.
//
// Bandwidth-bound: every byte of Wq and S is read exactly once with 128-bit loads, a full
// wavefront reading 1 KiB of one weight row per instruction.  One wavefront owns a weight row
// at a time over the whole K (so no cross-workgroup split-K reduction is needed when N is large);
// the 64 lanes split K, each lane keeps fp32 partial sums and the wave is reduced with DPP
// shuffles.  The activations are staged once per workgroup in LDS, already permuted into the
// pair order the nibble unpacking produces and transposed so that LDS reads are conflict free.
#include "nnf_device.h"
#include "nnf_launch.h"

#include "../nnf_workspace.h"

namespace nnf
{
    // LDS layout of the staged activations: 16-byte slots; slot(m, c, j, l) = ((m*C + c)*4 + j)*64 + l
    // holds the permuted a[m][k0..k0+7], k0 = c*2048 + l*32 + j*8.
    template <int MB>
    __global__ __launch_bounds__(256) void w4a16_gemv_kernel(const half_t* __restrict__ A,
                                                             const uint8_t* __restrict__ Wq,
                                                             const half_t* __restrict__ S,
                                                             half_t* __restrict__ Y,
                                                             int m0, int N, int K, int zp, int rows_per_wave)
    {
        extern __shared__ uintx4 a_lds[];
        const int tid = threadIdx.x;
        const int lane = tid & 63;
        const int wave = tid >> 6;
        const int C = (K + 2047) >> 11; // 2048-wide K chunks (one wave-wide 16-byte load each)
        const int G = K >> 7;           // groups of 128 per row
        const int segs_per_row = K >> 3;

        // stage A[m0 .. m0+MB) into LDS
        for (int seg = tid; seg < MB * segs_per_row; seg += 256)
        {
            int m = seg / segs_per_row;
            int k0 = (seg - m * segs_per_row) << 3;
            uintx4 a = *reinterpret_cast<const uintx4*>(A + (size_t)(m0 + m) * K + k0);
            int c = k0 >> 11;
            int l = (k0 & 2047) >> 5;
            int j = (k0 & 31) >> 3;
            a_lds[((m * C + c) * 4 + j) * 64 + l] = permute_a8(a);
        }
        __syncthreads();

        const DequantConst dq = make_dequant_const(zp);
        const int row_begin = (blockIdx.x * 4 + wave) * rows_per_wave;
        const int row_end = min(row_begin + rows_per_wave, N);

        for (int n = row_begin; n < row_end; ++n)
        {
            float acc[MB];
#pragma unroll
            for (int m = 0; m < MB; ++m)
                acc[m] = 0.0f;
            const uint8_t* wrow = Wq + (size_t)n * (K >> 1);
            const half_t* srow = S + (size_t)n * G;
#pragma unroll 2
            for (int c = 0; c < C; ++c)
            {
                int k_lane = (c << 11) + (lane << 5);
                if (k_lane < K)
                {
                    uintx4 w = __builtin_nontemporal_load(reinterpret_cast<const uintx4*>(wrow + (k_lane >> 1)));
                    float s = (float)srow[k_lane >> 7];
                    float part[MB];
#pragma unroll
                    for (int m = 0; m < MB; ++m)
                        part[m] = 0.0f;
                    uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                    {
                        half2_t q[4];
                        dequant8(ww[j], dq, q);
#pragma unroll
                        for (int m = 0; m < MB; ++m)
                        {
                            uintx4 a = a_lds[((m * C + c) * 4 + j) * 64 + lane];
                            part[m] = dot2(q[0], as_half2(a.x), part[m]);
                            part[m] = dot2(q[1], as_half2(a.y), part[m]);
                            part[m] = dot2(q[2], as_half2(a.z), part[m]);
                            part[m] = dot2(q[3], as_half2(a.w), part[m]);
                        }
                    }
#pragma unroll
                    for (int m = 0; m < MB; ++m)
                        acc[m] = __builtin_fmaf(part[m], s, acc[m]);
                }
            }
#pragma unroll
            for (int m = 0; m < MB; ++m)
            {
                float v = wave_sum(acc[m]);
                if (lane == 0)
                    Y[(size_t)(m0 + m) * N + n] = (half_t)v;
            }
        }
    }

    template <int MB>
    static hipError_t launch_gemv_mb(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y,
                                     int m0, int N, int K, int zp, int num_cu)
    {
        // aim at >= 2 workgroups (8 waves) per CU while keeping a few rows per wave
        int rows_per_wave = 1;
        while (rows_per_wave < 8 && (N + 4 * (rows_per_wave * 2) - 1) / (4 * rows_per_wave * 2) >= 4 * num_cu)
            rows_per_wave *= 2;
        int grid = (N + 4 * rows_per_wave - 1) / (4 * rows_per_wave);
        int C = (K + 2047) >> 11;
        size_t lds = (size_t)MB * C * 4 * 64 * 16;
        if (lds > 64 * 1024)
        {
            static LdsGrant granted;
            const hipError_t e = allow_dynamic_lds(reinterpret_cast<const void*>(&w4a16_gemv_kernel<MB>),
                                                   granted, (int)MAX_LDS_BYTES);
            if (e != hipSuccess)
                return e;
        }
        hipLaunchKernelGGL(w4a16_gemv_kernel<MB>, dim3(grid), dim3(256), lds, stream,
                           (const half_t*)A, (const uint8_t*)Wq, (const half_t*)S, (half_t*)Y, m0, N, K, zp,
                           rows_per_wave);
        return hipGetLastError();
    }

    bool w4a16_gemv_supported(int M, int K)
    {
        return workspace::w4a16_gemv_valu_fits(M, K);
    }

    // M rows are processed in passes of 4/2/1 rows (each pass re-reads the weights; the MFMA
    // skinny path takes over for larger M).
    hipError_t launch_w4a16_gemv(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y,
                                 int M, int N, int K, int zp, int num_cu)
    {
        int m0 = 0;
        hipError_t err = hipSuccess;
        while (m0 < M && err == hipSuccess)
        {
            int left = M - m0;
            if (left >= 4)
            {
                err = launch_gemv_mb<4>(stream, A, Wq, S, Y, m0, N, K, zp, num_cu);
                m0 += 4;
            }
            else if (left >= 2)
            {
                err = launch_gemv_mb<2>(stream, A, Wq, S, Y, m0, N, K, zp, num_cu);
                m0 += 2;
            }
            else
            {
                err = launch_gemv_mb<1>(stream, A, Wq, S, Y, m0, N, K, zp, num_cu);
                m0 += 1;
            }
        }
        return err;
    }
} // namespace nnf
