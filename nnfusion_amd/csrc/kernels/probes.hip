// Measurement probes (not part of the public ABI): how fast the matrix cores run on their own --
// no memory traffic at all -- as a function of the operand VALUES.  The chip is power managed: the
// same MFMA loop is clocked lower when the operand bits toggle more, so the attainable MFMA rate of a
// GEMM depends on its data.  bench.py --mfma-probe prints the figures.
#include "nnf_device.h"

#include <hip/hip_runtime.h>

namespace nnf
{
    namespace
    {
        // per-lane operand table: 512 lanes x 6 operands x 16 bytes
        __device__ __attribute__((aligned(16))) uint32_t g_probe_tab[512 * 6 * 4];

        __device__ __forceinline__ uint32_t mix(uint32_t x)
        {
            x ^= x >> 16;
            x *= 0x7feb352dU;
            x ^= x >> 15;
            x *= 0x846ca68bU;
            x ^= x >> 16;
            return x;
        }

        // kind 0: fp16 values, kind 1: int8 values.  mode 0: all ones, 1: N(0,1) fp16 / uniform int8 in
        // [-127, 127], 2: small integers in [-7, 7]
        __global__ void probe_fill_kernel(uint32_t* tab, int kind, int mode)
        {
            const int i = blockIdx.x * blockDim.x + threadIdx.x; // one 32-bit word each
            if (i >= 512 * 6 * 4)
                return;
            uint32_t word = 0;
            const int per_word = kind == 0 ? 2 : 4;
            for (int e = 0; e < per_word; ++e)
            {
                const uint32_t r1 = mix((uint32_t)(i * 4 + e) * 2654435761U + 12345U), r2 = mix(r1 + 0x9e3779b9U);
                float v;
                if (mode == 0)
                    v = 1.0f;
                else if (mode == 2)
                    v = (float)((int)(r1 % 15U) - 7);
                else if (kind == 0)
                {
                    const float u1 = ((float)(r1 >> 8) + 1.0f) / 16777217.0f, u2 = (float)(r2 >> 8) / 16777216.0f;
                    v = __builtin_sqrtf(-2.0f * __logf(u1)) * __cosf(6.2831853f * u2);
                }
                else
                    v = (float)((int)(r1 % 255U) - 127);
                if (kind == 0)
                {
                    half_t hv = (half_t)v;
                    word |= (uint32_t)__builtin_bit_cast(uint16_t, hv) << (16 * e);
                }
                else
                    word |= ((uint32_t)(int)v & 0xFFu) << (8 * e);
            }
            tab[i] = word;
        }

        // eight independent 32x32 accumulators per wavefront (4 A operands x 2 B operands), two wavefronts
        // per SIMD: the arrangement of the GEMM kernels, minus everything but the MFMAs
        // shader clock cycles and 100 MHz wall-clock ticks spent by workgroup 0 (their ratio is the shader clock)
        __device__ unsigned long long g_probe_clocks[2];

        __global__ __launch_bounds__(512) void probe_f16_kernel(const uint32_t* tab, float* out, int iters)
        {
            const unsigned long long c0 = clock64(), w0 = wall_clock64();
            const uintx4* t = reinterpret_cast<const uintx4*>(tab) + threadIdx.x * 6;
            half8_t a[4], b[2];
            for (int i = 0; i < 4; ++i)
                a[i] = __builtin_bit_cast(half8_t, t[i]);
            for (int i = 0; i < 2; ++i)
                b[i] = __builtin_bit_cast(half8_t, t[4 + i]);
            floatx16 acc[8];
            for (int i = 0; i < 8; ++i)
                for (int e = 0; e < 16; ++e)
                    acc[i][e] = 0.f;
            for (int it = 0; it < iters; ++it)
            {
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        acc[j * 4 + i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], b[j], acc[j * 4 + i], 0, 0, 0);
            }
            float s = 0.f;
            for (int i = 0; i < 8; ++i)
                for (int e = 0; e < 16; ++e)
                    s += acc[i][e];
            if (s == 1234.5f)
                out[0] = s;
            if (blockIdx.x == 0 && threadIdx.x == 0)
            {
                g_probe_clocks[0] = clock64() - c0;
                g_probe_clocks[1] = wall_clock64() - w0;
            }
        }

        __global__ __launch_bounds__(512) void probe_i8_kernel(const uint32_t* tab, float* out, int iters)
        {
            const unsigned long long c0 = clock64(), w0 = wall_clock64();
            const intx4* t = reinterpret_cast<const intx4*>(tab) + threadIdx.x * 6;
            intx4 a[4], b[2];
            for (int i = 0; i < 4; ++i)
                a[i] = t[i];
            for (int i = 0; i < 2; ++i)
                b[i] = t[4 + i];
            intx16 acc[8];
            for (int i = 0; i < 8; ++i)
                for (int e = 0; e < 16; ++e)
                    acc[i][e] = 0;
            for (int it = 0; it < iters; ++it)
            {
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        acc[j * 4 + i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[j], acc[j * 4 + i], 0, 0, 0);
            }
            int s = 0;
            for (int i = 0; i < 8; ++i)
                for (int e = 0; e < 16; ++e)
                    s += acc[i][e];
            if (s == 123457)
                out[0] = (float)s;
            if (blockIdx.x == 0 && threadIdx.x == 0)
            {
                g_probe_clocks[0] = clock64() - c0;
                g_probe_clocks[1] = wall_clock64() - w0;
            }
        }
    } // namespace
} // namespace nnf

// Runs `iters` rounds of 8 MFMAs per wavefront on one workgroup of 8 wavefronts per CU and returns the
// rate in tera-operations per second through *tops (fp16: 32x32x16, int8: 32x32x32) and the shader clock
// during the run through *shader_mhz.  Returns a hipError_t.
extern "C" int nnf_internal_mfma_probe(int kind, int mode, int iters, int num_cu, double* tops, double* shader_mhz)
{
    using namespace nnf;
    uint32_t* tab = nullptr;
    hipError_t e = hipGetSymbolAddress((void**)&tab, HIP_SYMBOL(g_probe_tab));
    if (e != hipSuccess)
        return (int)e;
    hipLaunchKernelGGL(probe_fill_kernel, dim3((512 * 6 * 4 + 255) / 256), dim3(256), 0, 0, tab, kind, mode);
    float* out = reinterpret_cast<float*>(tab); // never written: the guard values cannot occur
    hipEvent_t e0, e1;
    if ((e = hipEventCreate(&e0)) != hipSuccess || (e = hipEventCreate(&e1)) != hipSuccess)
        return (int)e;
    for (int rep = 0; rep < 2; ++rep) // the first run warms up clocks and code
    {
        if ((e = hipEventRecord(e0, 0)) != hipSuccess)
            return (int)e;
        if (kind == 0)
            hipLaunchKernelGGL(probe_f16_kernel, dim3(num_cu), dim3(512), 0, 0, tab, out, iters);
        else
            hipLaunchKernelGGL(probe_i8_kernel, dim3(num_cu), dim3(512), 0, 0, tab, out, iters);
        if ((e = hipEventRecord(e1, 0)) != hipSuccess || (e = hipEventSynchronize(e1)) != hipSuccess)
            return (int)e;
    }
    float ms = 0.f;
    if ((e = hipEventElapsedTime(&ms, e0, e1)) != hipSuccess)
        return (int)e;
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    const double ops_per_mfma = kind == 0 ? 32768.0 : 65536.0;
    *tops = (double)num_cu * 8 * (double)iters * 8 * ops_per_mfma / ((double)ms * 1e9);
    unsigned long long clocks[2] = {0, 0};
    e = hipMemcpyFromSymbol(clocks, HIP_SYMBOL(g_probe_clocks), sizeof(clocks));
    if (e != hipSuccess)
        return (int)e;
    *shader_mhz = clocks[1] ? (double)clocks[0] / (double)clocks[1] * 100.0 : 0.0;
    return (int)hipGetLastError();
}
