// TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
//
// CPU restatement of the arithmetic that microsoft/nnfusion's CPU code path would
// perform for a quantized linear layer: dequantize the constant weight, then an fp32
// Dot (GEMM) as cpu::DotMlas emits it, then element-wise ops.  Only tests, the smoke
// check and the cpu_baseline leg of bench.py may load this library; the shipped
// library (libnnf_hip_kernels.so) never links or calls it.
//
// Reference sources each function follows (paths relative to the nnfusion tree):
//   oracle_dequantize_w4 / _wn   src/nnfusion/core/kernels/cpu/reference/kernels.cpp:601-623
//                                (integer subtract of the offset, cast to REAL, multiply by scale)
//   oracle_dot_f32               src/nnfusion/core/kernels/cpu/mlas/dot.cpp:25-102
//                                (M/N/K, lda = transA ? M : K, ldb = transB ? K : N, ldc = N,
//                                 alpha = 1, beta = 0, row-major) and the K-blocking of 128 of
//                                thirdparty/mlas/lib/mlasi.h:119-120
//   oracle_dot_general           src/nnfusion/core/operators/op_define/dot.cpp:43-135 (shape rule),
//                                src/nnfusion/core/kernels/cpu/reference/kernels.cpp:1532-1621
//                                (naive definition, sequential k order, accumulate in T)
//   oracle_sigmoid               src/nnfusion/core/kernels/cpu/reference/kernels.cpp:934-943
//                                (1 / (1 + exp(-x)))
//   oracle_time_dot_f32          src/nnfusion/engine/pass/codegen/cpu_codegen_pass.cpp:301-335
//                                (warm-ups, then timed iterations with std::chrono, mean)
// The quantized layouts (nibble order, scale layout, W8A8 epilogue order) are not defined by
// the reference; they are fixed in include/nnf_hip_kernels.h and restated here.
//
// Pinning status (see tests/test_oracle_*.py):
//   fp32 Dot: reference known-answer vectors (test/nnfusion/inventory/dot.cpp, ONNX gemm/matmul
//             vectors), MLAS built from the reference tree (oracle/_ref), fp64 brute force.
//   dequantize, W8A8, RMSNorm, SiLU: the reference holds no test for quantized arithmetic;
//             pinned by closed forms, invariants and brute force in int64/fp64.

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

namespace
{
    // IEEE binary16 <-> binary32, round-to-nearest-even, NaN/Inf/subnormals handled.
    inline float h2f(uint16_t h)
    {
        uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
        uint32_t exp = (h >> 10) & 0x1Fu;
        uint32_t man = h & 0x3FFu;
        uint32_t bits;
        if (exp == 0)
        {
            if (man == 0)
            {
                bits = sign;
            }
            else
            {
                // subnormal: normalise
                int e = -1;
                do
                {
                    man <<= 1;
                    ++e;
                } while ((man & 0x400u) == 0);
                man &= 0x3FFu;
                bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
            }
        }
        else if (exp == 31)
        {
            bits = sign | 0x7F800000u | (man << 13);
        }
        else
        {
            bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
        }
        float f;
        std::memcpy(&f, &bits, 4);
        return f;
    }

    inline uint16_t f2h(float f)
    {
        uint32_t x;
        std::memcpy(&x, &f, 4);
        uint32_t sign = (x >> 16) & 0x8000u;
        uint32_t abs = x & 0x7FFFFFFFu;
        if (abs >= 0x7F800000u)
        {
            // Inf / NaN (keep a quiet NaN payload bit)
            return (uint16_t)(sign | 0x7C00u | (abs > 0x7F800000u ? (0x200u | ((abs >> 13) & 0x3FFu)) : 0));
        }
        if (abs >= 0x477FF000u)
        {
            // >= 65520 rounds to infinity
            return (uint16_t)(sign | 0x7C00u);
        }
        if (abs < 0x33000001u)
        {
            // <= 2^-25 rounds to zero (exactly 2^-25 ties to even = 0)
            return (uint16_t)sign;
        }
        int32_t e = (int32_t)(abs >> 23) - 127;
        uint32_t man = (abs & 0x7FFFFFu) | 0x800000u; // 24-bit significand
        int shift;                                     // bits dropped from the 24-bit significand
        uint32_t hexp;
        if (e < -14)
        {
            shift = 13 + (-14 - e);
            hexp = 0;
        }
        else
        {
            shift = 13;
            hexp = (uint32_t)(e + 15);
        }
        uint32_t kept = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1);
        if (rem > half || (rem == half && (kept & 1u)))
            ++kept;
        uint32_t out;
        if (hexp == 0)
            out = kept; // subnormal (a carry into bit 10 yields the smallest normal, as wanted)
        else
            out = ((hexp - 1) << 10) + kept; // kept carries the implicit bit: adds 1 to the exponent
        return (uint16_t)(sign | out);
    }

    inline int clamp_threads(int nthreads)
    {
#ifdef _OPENMP
        int hw = omp_get_num_procs();
        if (nthreads <= 0 || nthreads > hw)
            nthreads = hw;
        return nthreads;
#else
        (void)nthreads;
        return 1;
#endif
    }

    // One output element of C = A . B^T restricted to K-block [k0,k1): 16 independent partial
    // sums in a fixed order, reduced pairwise -- the shape of a SIMD FMA micro-kernel.
    inline float dot_block(const float* a, const float* b, int len)
    {
        float acc[16];
        for (int j = 0; j < 16; ++j)
            acc[j] = 0.0f;
        int k = 0;
        for (; k + 16 <= len; k += 16)
            for (int j = 0; j < 16; ++j)
                acc[j] = std::fma(a[k + j], b[k + j], acc[j]);
        for (int j = 0; k < len; ++k, ++j)
            acc[j] = std::fma(a[k], b[k], acc[j]);
        for (int w = 8; w >= 1; w >>= 1)
            for (int j = 0; j < w; ++j)
                acc[j] += acc[j + w];
        return acc[0];
    }

    const int KBLOCK = 128; // MLAS_SGEMM_STRIDEK

    // C[M,N] = A[M,K] . Bt[N,K]^T, fp32 accumulate, K in blocks of 128, rows of Bt split over threads.
    void gemm_nt(const float* A, const float* Bt, float* C, int M, int N, int K, int nthreads)
    {
        nthreads = clamp_threads(nthreads);
#pragma omp parallel for schedule(static) num_threads(nthreads)
        for (int n = 0; n < N; ++n)
        {
            const float* b = Bt + (size_t)n * K;
            for (int m = 0; m < M; ++m)
            {
                const float* a = A + (size_t)m * K;
                float c = 0.0f;
                for (int k0 = 0; k0 < K; k0 += KBLOCK)
                    c += dot_block(a + k0, b + k0, std::min(KBLOCK, K - k0));
                C[(size_t)m * N + n] = c;
            }
        }
    }
} // namespace

extern "C" {

int oracle_version()
{
    return 1;
}

int oracle_max_threads()
{
    return clamp_threads(0);
}

void oracle_f16_to_f32(const uint16_t* in, float* out, size_t n)
{
    for (size_t i = 0; i < n; ++i)
        out[i] = h2f(in[i]);
}

void oracle_f32_to_f16(const float* in, uint16_t* out, size_t n)
{
    for (size_t i = 0; i < n; ++i)
        out[i] = f2h(in[i]);
}

// Unpack + dequantize unsigned 4-bit weights.  wq is [N, K/2] bytes, the low nibble of byte b
// of a row holds k = 2b and the high nibble k = 2b+1; scales is fp16 [N, K/group]; the offset
// is the scalar zero point.  out is fp32 [N, K]:  REAL(q - offset) * scale.
void oracle_dequantize_w4(const uint8_t* wq, const uint16_t* scales, int N, int K, int group, int zp, float* out)
{
    const int G = K / group;
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n)
        for (int k = 0; k < K; ++k)
        {
            uint8_t byte = wq[(size_t)n * (K / 2) + k / 2];
            int q = (k & 1) ? (byte >> 4) : (byte & 0xF);
            float s = h2f(scales[(size_t)n * G + k / group]);
            out[(size_t)n * K + k] = static_cast<float>(q - zp) * s;
        }
}

// The same dequantisation with the block parameters of the reference's signature left open
// (cpu_reference_dequantize, kernels.cpp:601-623: per-block offset and scale, the integer subtract done before
// the cast): `bits` 4 (two weights per byte as above) or 8 (one byte per weight, wq [N, K]); `group` any divisor
// of K; zero points either the scalar `zp` (zps == nullptr) or one per (row, group): u8, row stride
// ceil(G * bits / 8) bytes, bits = 4 packed two per byte along the groups, low nibble = even group -- the packing of
// ONNX com.microsoft::MatMulNBits' zero_points input.
void oracle_dequantize_wn(const uint8_t* wq, const uint16_t* scales, const uint8_t* zps, int N, int K, int bits,
                          int group, int zp, float* out)
{
    const int G = K / group;
    const size_t w_stride = (size_t)K * bits / 8;
    const size_t z_stride = ((size_t)G * bits + 7) / 8;
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n)
        for (int k = 0; k < K; ++k)
        {
            int q;
            if (bits == 4)
            {
                const uint8_t byte = wq[(size_t)n * w_stride + k / 2];
                q = (k & 1) ? (byte >> 4) : (byte & 0xF);
            }
            else
                q = wq[(size_t)n * w_stride + k];
            const int g = k / group;
            int z = zp;
            if (zps)
            {
                if (bits == 4)
                {
                    const uint8_t byte = zps[(size_t)n * z_stride + g / 2];
                    z = (g & 1) ? (byte >> 4) : (byte & 0xF);
                }
                else
                    z = zps[(size_t)n * z_stride + g];
            }
            out[(size_t)n * K + k] = static_cast<float>(q - z) * h2f(scales[(size_t)n * G + g]);
        }
}

// The 2-D Dot as cpu::DotMlas hands it to MlasGemm: C[M,N] = op(A) . op(B), row-major,
// op(A) is [M,K] (stored [K,M] with lda = M when transA), op(B) is [K,N] (stored [N,K] with
// ldb = K when transB), alpha 1, beta 0.
void oracle_dot_f32(const float* A, const float* B, float* C, int M, int N, int K, int transA, int transB, int nthreads)
{
    std::vector<float> a_tmp, b_tmp;
    const float* a = A;
    const float* bt = B;
    if (transA)
    {
        a_tmp.resize((size_t)M * K);
        for (int k = 0; k < K; ++k)
            for (int m = 0; m < M; ++m)
                a_tmp[(size_t)m * K + k] = A[(size_t)k * M + m];
        a = a_tmp.data();
    }
    if (!transB)
    {
        b_tmp.resize((size_t)N * K);
        for (int k = 0; k < K; ++k)
            for (int n = 0; n < N; ++n)
                b_tmp[(size_t)n * K + k] = B[(size_t)k * N + n];
        bt = b_tmp.data();
    }
    gemm_nt(a, bt, C, M, N, K, nthreads);
}

// Naive Dot with the reduction-axes rule of op::Dot: the last `r` axes of arg0 are contracted
// with the first `r` axes of arg1; output dims = free dims of arg0 then free dims of arg1.
// Sequential k order, accumulation in float.  Scalars are rank-0 (rank = 0, dims ignored).
void oracle_dot_general(const float* a, const int64_t* a_dims, int a_rank,
                        const float* b, const int64_t* b_dims, int b_rank,
                        int r, float* out)
{
    if (a_rank == 0 || b_rank == 0)
    {
        // scalar times tensor
        size_t na = 1, nb = 1;
        for (int i = 0; i < a_rank; ++i)
            na *= (size_t)a_dims[i];
        for (int i = 0; i < b_rank; ++i)
            nb *= (size_t)b_dims[i];
        if (a_rank == 0)
            for (size_t i = 0; i < nb; ++i)
                out[i] = a[0] * b[i];
        else
            for (size_t i = 0; i < na; ++i)
                out[i] = a[i] * b[0];
        return;
    }
    size_t Mf = 1, Kf = 1, Nf = 1;
    for (int i = 0; i < a_rank - r; ++i)
        Mf *= (size_t)a_dims[i];
    for (int i = a_rank - r; i < a_rank; ++i)
        Kf *= (size_t)a_dims[i];
    for (int i = r; i < b_rank; ++i)
        Nf *= (size_t)b_dims[i];
    for (size_t m = 0; m < Mf; ++m)
        for (size_t n = 0; n < Nf; ++n)
        {
            float sum = 0.0f;
            for (size_t k = 0; k < Kf; ++k)
                sum += a[m * Kf + k] * b[k * Nf + n];
            out[m * Nf + n] = sum;
        }
}

// fp64-accumulated twin of the NT GEMM, for error analysis in tests (tiny/medium shapes).
void oracle_gemm_nt_f64(const float* A, const float* Bt, double* C, int M, int N, int K)
{
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n)
        for (int m = 0; m < M; ++m)
        {
            double s = 0.0;
            for (int k = 0; k < K; ++k)
                s += (double)A[(size_t)m * K + k] * (double)Bt[(size_t)n * K + k];
            C[(size_t)m * N + n] = s;
        }
}

// Y = A . ((W - zp) * scale)^T : dequantize to fp32, fp32-accumulated GEMM, fp32 result.
void oracle_w4a16_gemm_f32(const uint16_t* A, const uint8_t* wq, const uint16_t* scales, float* Y,
                           int M, int N, int K, int group, int zp, int nthreads)
{
    std::vector<float> a((size_t)M * K), w((size_t)N * K);
    oracle_f16_to_f32(A, a.data(), (size_t)M * K);
    oracle_dequantize_w4(wq, scales, N, K, group, zp, w.data());
    gemm_nt(a.data(), w.data(), Y, M, N, K, nthreads);
}

// Same, with the result rounded (nearest even) to fp16 as the output tensor type asks.
void oracle_w4a16_gemm(const uint16_t* A, const uint8_t* wq, const uint16_t* scales, uint16_t* Y,
                       int M, int N, int K, int group, int zp, int nthreads)
{
    std::vector<float> y((size_t)M * N);
    oracle_w4a16_gemm_f32(A, wq, scales, y.data(), M, N, K, group, zp, nthreads);
    oracle_f32_to_f16(y.data(), Y, (size_t)M * N);
}

// Y = A . dequantize_wn(W)^T, fp32-accumulated, fp32 result (f16_out == 0) or rounded to fp16 (Y then holds uint16).
void oracle_wna16_gemm(const uint16_t* A, const uint8_t* wq, const uint16_t* scales, const uint8_t* zps, void* Y, int M,
                       int N, int K, int bits, int group, int zp, int f16_out, int nthreads)
{
    std::vector<float> a((size_t)M * K), w((size_t)N * K), y;
    oracle_f16_to_f32(A, a.data(), (size_t)M * K);
    oracle_dequantize_wn(wq, scales, zps, N, K, bits, group, zp, w.data());
    if (!f16_out)
    {
        gemm_nt(a.data(), w.data(), static_cast<float*>(Y), M, N, K, nthreads);
        return;
    }
    y.resize((size_t)M * N);
    gemm_nt(a.data(), w.data(), y.data(), M, N, K, nthreads);
    oracle_f32_to_f16(y.data(), static_cast<uint16_t*>(Y), (size_t)M * N);
}

// Raw int32 accumulators of the W8A8 product: acc[m,n] = sum_k A[m,k] * W[n,k].
void oracle_w8a8_acc(const int8_t* A, const int8_t* W, int32_t* acc, int M, int N, int K, int nthreads)
{
    nthreads = clamp_threads(nthreads);
#pragma omp parallel for schedule(static) num_threads(nthreads)
    for (int n = 0; n < N; ++n)
        for (int m = 0; m < M; ++m)
        {
            const int8_t* a = A + (size_t)m * K;
            const int8_t* w = W + (size_t)n * K;
            int32_t s = 0;
            for (int k = 0; k < K; ++k)
                s += (int32_t)a[k] * (int32_t)w[k];
            acc[(size_t)m * N + n] = s;
        }
}

// int64 brute-force twin (pins oracle_w8a8_acc against overflow or widening mistakes).
void oracle_w8a8_acc_i64(const int8_t* A, const int8_t* W, int64_t* acc, int M, int N, int K)
{
    for (int n = 0; n < N; ++n)
        for (int m = 0; m < M; ++m)
        {
            int64_t s = 0;
            for (int k = 0; k < K; ++k)
                s += (int64_t)A[(size_t)m * K + k] * (int64_t)W[(size_t)n * K + k];
            acc[(size_t)m * N + n] = s;
        }
}

// Epilogue of W8A8: Y = fp16( (float)acc * s_tok[m] * s_ch[n] ), evaluated left to right in fp32.
void oracle_w8a8_epilogue(const int32_t* acc, const float* s_tok, const float* s_ch, uint16_t* Y, int M, int N)
{
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n)
        {
            volatile float t = (float)acc[(size_t)m * N + n] * s_tok[m];
            volatile float u = t * s_ch[n];
            Y[(size_t)m * N + n] = f2h(u);
        }
}

void oracle_w8a8_gemm(const int8_t* A, const float* s_tok, const int8_t* W, const float* s_ch, uint16_t* Y,
                      int M, int N, int K, int nthreads)
{
    std::vector<int32_t> acc((size_t)M * N);
    oracle_w8a8_acc(A, W, acc.data(), M, N, K, nthreads);
    oracle_w8a8_epilogue(acc.data(), s_tok, s_ch, Y, M, N);
}

float oracle_sigmoid(float x)
{
    return 1.0f / (1.0f + std::exp(-x));
}

// RMSNorm over the last axis: out = fp16( x * rsqrt(mean(x^2) + eps) * gamma ), fp32 math on
// fp16 data (the sum of squares is accumulated in fp64 so the oracle is order-independent).
void oracle_rmsnorm_f16(const uint16_t* x, const uint16_t* gamma, float eps, uint16_t* out, int M, int K)
{
    for (int m = 0; m < M; ++m)
    {
        double ss = 0.0;
        for (int k = 0; k < K; ++k)
        {
            double v = h2f(x[(size_t)m * K + k]);
            ss += v * v;
        }
        float r = 1.0f / std::sqrt((float)(ss / K) + eps);
        for (int k = 0; k < K; ++k)
            out[(size_t)m * K + k] = f2h(h2f(x[(size_t)m * K + k]) * r * h2f(gamma[k]));
    }
}

// h = fp16( g * sigmoid(g) * u ) element-wise on fp16 tensors, fp32 math.
void oracle_silu_mul_f16(const uint16_t* g, const uint16_t* u, uint16_t* out, size_t n)
{
    for (size_t i = 0; i < n; ++i)
    {
        float gv = h2f(g[i]);
        out[i] = f2h(gv * oracle_sigmoid(gv) * h2f(u[i]));
    }
}

void oracle_add_f16(const uint16_t* a, const uint16_t* b, uint16_t* out, size_t n)
{
    for (size_t i = 0; i < n; ++i)
        out[i] = f2h(h2f(a[i]) + h2f(b[i]));
}

// Llama-style MLP block as an unfused graph with fp16 tensors between the nodes:
//   xn = RMSNorm(x, gamma, eps); gu = QuantDot(xn, Wgu) (rows 0..I-1 = gate, I..2I-1 = up);
//   h = SiLU(gate) * up; d = QuantDot(h, Wd); out = d + x.
// h_out (optional, [M, I] fp16) receives the intermediate.
void oracle_fused_mlp_w4a16(const uint16_t* x, const uint16_t* gamma, float eps,
                            const uint8_t* wgu, const uint16_t* sgu,
                            const uint8_t* wd, const uint16_t* sd,
                            uint16_t* out, uint16_t* h_out,
                            int M, int H, int I, int group, int zp, int nthreads)
{
    std::vector<uint16_t> xn((size_t)M * H), gu((size_t)M * 2 * I), g((size_t)M * I), u((size_t)M * I),
        h((size_t)M * I), d((size_t)M * H);
    oracle_rmsnorm_f16(x, gamma, eps, xn.data(), M, H);
    oracle_w4a16_gemm(xn.data(), wgu, sgu, gu.data(), M, 2 * I, H, group, zp, nthreads);
    for (int m = 0; m < M; ++m)
    {
        std::memcpy(&g[(size_t)m * I], &gu[(size_t)m * 2 * I], (size_t)I * 2);
        std::memcpy(&u[(size_t)m * I], &gu[(size_t)m * 2 * I + I], (size_t)I * 2);
    }
    oracle_silu_mul_f16(g.data(), u.data(), h.data(), (size_t)M * I);
    if (h_out)
        std::memcpy(h_out, h.data(), (size_t)M * I * 2);
    oracle_w4a16_gemm(h.data(), wd, sd, d.data(), M, H, I, group, zp, nthreads);
    oracle_add_f16(d.data(), x, out, (size_t)M * H);
}

// Timing loop of the generated CPU main_test: `warmup` untimed calls, then `iters` timed calls
// with std::chrono; returns the mean in milliseconds and writes the minimum to *min_ms.
// B is the already-dequantized fp32 weight [N,K] (constants are folded at init, untimed).
double oracle_time_dot_f32(const float* A, const float* Bt, float* C, int M, int N, int K,
                           int warmup, int iters, int nthreads, double* min_ms)
{
    for (int i = 0; i < warmup; ++i)
        gemm_nt(A, Bt, C, M, N, K, nthreads);
    double total = 0.0, best = 1e300;
    for (int i = 0; i < iters; ++i)
    {
        auto t0 = std::chrono::high_resolution_clock::now();
        gemm_nt(A, Bt, C, M, N, K, nthreads);
        auto t1 = std::chrono::high_resolution_clock::now();
        double ms = std::chrono::duration<double, std::milli>(t1 - t0).count();
        total += ms;
        best = std::min(best, ms);
    }
    if (min_ms)
        *min_ms = best;
    return total / std::max(iters, 1);
}

double oracle_time_w8a8_acc(const int8_t* A, const int8_t* W, int32_t* acc, int M, int N, int K,
                            int warmup, int iters, int nthreads, double* min_ms)
{
    for (int i = 0; i < warmup; ++i)
        oracle_w8a8_acc(A, W, acc, M, N, K, nthreads);
    double total = 0.0, best = 1e300;
    for (int i = 0; i < iters; ++i)
    {
        auto t0 = std::chrono::high_resolution_clock::now();
        oracle_w8a8_acc(A, W, acc, M, N, K, nthreads);
        auto t1 = std::chrono::high_resolution_clock::now();
        double ms = std::chrono::duration<double, std::milli>(t1 - t0).count();
        total += ms;
        best = std::min(best, ms);
    }
    if (min_ms)
        *min_ms = best;
    return total / std::max(iters, 1);
}

} // extern "C"
