// Stand-alone kernels for the nodes around a quantized product that no fusion pattern absorbed: RMSNorm, the
// element-wise operators of the MLP block (Add, Multiply, Sigmoid, Swish) and Dequantize.
//
// The reference emits these nodes through its element-wise emitter
// (src/nnfusion/core/kernels/cuda_gpu/kernels/elementwise.cpp with the CudaOpMap entries of
// cuda_gpu/cuda_kernelops.hpp:408 Add, :416 Multiply, :447-451 Sigmoid = 1 / (1 + expf(-x0))), LayerNorm through
// cuda_gpu/kernels/layer_norm.cpp (rsqrt(sigma2 + epsilon), cuda_langunit.cpp:618), and defines Dequantize as
// static_cast<REAL>(in - offset) * scale (core/kernels/cpu/reference/kernels.cpp:601-623).  Here: fp16 tensors,
// arithmetic in fp32, one rounding to fp16 per node -- what the fused kernels reproduce.  All HBM bound, 16-byte accesses
// where the tensors allow it.
#include "nnf_device.h"
#include "nnf_launch.h"

namespace nnf
{
    namespace
    {
        __device__ __forceinline__ float ew_apply(int op, float a, float b)
        {
            switch (op)
            {
            case EW_ADD: return a + b;
            case EW_MULTIPLY: return a * b;
            case EW_SIGMOID: return 1.0f / (1.0f + __expf(-a));
            default: return a * (1.0f / (1.0f + __expf(-a))); // EW_SWISH
            }
        }

        // y[r, c] = op(a[r, c], b[r, c] or b[c]); eight consecutive columns per thread (cols a multiple of 8) or one
        template <bool VEC>
        __global__ __launch_bounds__(256) void elementwise_kernel(int op, const half_t* __restrict__ a, const half_t* b,
                                                                  half_t* y, long long total, int cols, int b_is_row)
        {
            const long long i = ((long long)blockIdx.x * 256 + threadIdx.x) * (VEC ? 8 : 1);
            if (i >= total)
                return;
            const bool binary = op == EW_ADD || op == EW_MULTIPLY;
            if constexpr (VEC)
            {
                const half8_t va = *reinterpret_cast<const half8_t*>(a + i);
                half8_t vb = va;
                if (binary)
                    vb = *reinterpret_cast<const half8_t*>(b + (b_is_row ? i % cols : i));
                half8_t out;
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    out[e] = (half_t)ew_apply(op, (float)va[e], (float)vb[e]);
                *reinterpret_cast<half8_t*>(y + i) = out;
            }
            else
            {
                const float fb = binary ? (float)b[b_is_row ? i % cols : i] : 0.f;
                y[i] = (half_t)ew_apply(op, (float)a[i], fb);
            }
        }

        // W[n, k] = fp16((q[n, k] - z[n, k / group]) * s[n, k / group]); eight consecutive k per thread
        template <int BITS>
        __global__ __launch_bounds__(256) void dequantize_kernel(const uint8_t* __restrict__ Wq, const half_t* __restrict__ S,
                                                                 const uint8_t* __restrict__ zps, half_t* __restrict__ W, int N, int K,
                                                                 int group_shift, int zp)
        {
            const long long i = ((long long)blockIdx.x * 256 + threadIdx.x) * 8;
            if (i >= (long long)N * K)
                return;
            const int n = (int)(i / K), k = (int)(i - (long long)n * K);
            const int G = K >> group_shift, g = k >> group_shift;
            int z = zp;
            if (zps)
            {
                if (BITS == 4)
                {
                    const uint8_t byte = zps[(size_t)n * ((G + 1) >> 1) + (g >> 1)];
                    z = (g & 1) ? (byte >> 4) : (byte & 0xF);
                }
                else
                    z = zps[(size_t)n * G + g];
            }
            const float s = (float)S[(size_t)n * G + g];
            int q[8];
            if (BITS == 4)
            {
                const uint32_t w = *reinterpret_cast<const uint32_t*>(Wq + (size_t)n * (K >> 1) + (k >> 1));
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    q[e] = (int)((w >> (4 * e)) & 0xFu);
            }
            else
            {
                const uintx2 w = *reinterpret_cast<const uintx2*>(Wq + (size_t)n * K + k);
#pragma unroll
                for (int e = 0; e < 4; ++e)
                {
                    q[e] = (int)((w.x >> (8 * e)) & 0xFFu);
                    q[4 + e] = (int)((w.y >> (8 * e)) & 0xFFu);
                }
            }
            half8_t out;
#pragma unroll
            for (int e = 0; e < 8; ++e)
                out[e] = (half_t)((float)(q[e] - z) * s); // integer subtract, cast, multiply: exact in fp32, one rounding
            *reinterpret_cast<half8_t*>(W + i) = out;
        }
    } // namespace

    hipError_t launch_elementwise(hipStream_t stream, int op, const void* a, const void* b, void* y, long long rows, int cols,
                                  bool b_is_row)
    {
        const long long total = rows * cols;
        const bool aligned = ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(y)) & 15) == 0;
        if ((cols & 7) == 0 && aligned)
        {
            const long long blocks = (total / 8 + 255) / 256;
            hipLaunchKernelGGL(elementwise_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, stream, op, (const half_t*)a,
                               (const half_t*)b, (half_t*)y, total, cols, b_is_row ? 1 : 0);
        }
        else
        {
            const long long blocks = (total + 255) / 256;
            hipLaunchKernelGGL(elementwise_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, stream, op, (const half_t*)a,
                               (const half_t*)b, (half_t*)y, total, cols, b_is_row ? 1 : 0);
        }
        return hipGetLastError();
    }

    hipError_t launch_dequantize(hipStream_t stream, const void* Wq, const void* S, const void* zero_points, void* W, int N, int K,
                                 int bits, int group_shift, int zp)
    {
        const long long blocks = ((long long)N * K / 8 + 255) / 256;
        if (bits == 4)
            hipLaunchKernelGGL(dequantize_kernel<4>, dim3((unsigned)blocks), dim3(256), 0, stream, (const uint8_t*)Wq, (const half_t*)S,
                               (const uint8_t*)zero_points, (half_t*)W, N, K, group_shift, zp);
        else
            hipLaunchKernelGGL(dequantize_kernel<8>, dim3((unsigned)blocks), dim3(256), 0, stream, (const uint8_t*)Wq, (const half_t*)S,
                               (const uint8_t*)zero_points, (half_t*)W, N, K, group_shift, zp);
        return hipGetLastError();
    }
} // namespace nnf
