// Internal launch functions behind the C ABI (one per kernel family).  Each validates nothing:
// nnf_api.hip checks shapes, alignment and workspace before calling in.
#pragma once

#include <hip/hip_runtime.h>
#include <atomic>
#include <stddef.h>
#include <stdint.h>

namespace nnf
{
    // largest dynamic LDS a workgroup may ask for on gfx950 (160 KiB per CU)
    constexpr size_t MAX_LDS_BYTES = 160 * 1024;

    // Lifts a kernel's dynamic-LDS limit to `bytes`, once per (kernel, device): `granted` is a static of the calling
    // template instantiation (one per kernel).  Racing first calls at worst set the attribute twice.
    struct LdsGrant
    {
        std::atomic<int> bytes[64] = {};
    };
    inline hipError_t allow_dynamic_lds(const void* kernel, LdsGrant& granted, int bytes)
    {
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess)
            return e;
        const bool cached = dev >= 0 && dev < 64;
        if (cached && granted.bytes[dev].load(std::memory_order_relaxed) >= bytes)
            return hipSuccess;
        e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        if (e == hipSuccess && cached)
            granted.bytes[dev].store(bytes, std::memory_order_relaxed);
        return e;
    }

    // Optional prologue and epilogue of the row-streaming GEMV kernels (every pointer may be null), applied as the unfused
    // graph would on fp16 tensors: y = fp16(rstd[m] * sum); gate: y = fp16(silu(y_gate) * y_up); y = fp16(y + bias[n]);
    // y = fp16(y + residual[m, n]).
    struct GemvFusion
    {
        const void* gamma = nullptr;    // fp16 [K]: RMSNorm weight, multiplied onto the activations on the way in ...
        const float* rstd = nullptr;    // fp32 [M]: ... with the sums of row m scaled by rstd[m] on the way out
        float rms_eps = 0.f;            // gamma without rstd (the row-streaming kernels with a fixed K): rstd computed inside the kernel with this eps
        const void* bias = nullptr;     // fp16 [N]
        const void* residual = nullptr; // fp16 [M, N]; may be the output buffer itself
        bool gate = false;              // N outputs from 2 N weight rows (gate rows, then up rows): SiLU(gate) * up
        bool any() const { return gamma || rstd || bias || residual || gate; }
    };

    // What a call fixes about its launch (all zero: the library's own choice by shape).  Filled from the variant and
    // plan arguments of the C ABI and passed down by value: the library keeps no dispatch state between calls.
    struct LaunchChoice
    {
        int path = 0;      // the nnf_w4a16_variant / nnf_w8a8_variant values: 1 VALU GEMV, 2 MFMA GEMV over K ranges,
                           // 3 tile GEMM, 4 row-streaming kernels
        int tile_rows = 0; // tile GEMM: rows of an output tile (256, 128, 64; fp16 x int4 also 32)
        int k_parts = 0;   // tile GEMM: workgroups that share an output tile (fp16 x int4) / ranges of K (W8A8)
        int tile_cols = 0; // W8A8 tile GEMM with 256-row tiles: 256 or 128 columns
        // fp16 x int4 tile GEMM in one launch: zeroed words the workgroups that share a tile synchronise through (left
        // zero again), their size, and how many polls a workgroup waits for the others (0: DEFAULT_SPIN_LIMIT)
        void* sync_flags = nullptr;
        size_t sync_bytes = 0;
        int spin_limit = 0;
    };
    // a poll is an atomic load from device memory and a short sleep, about a microsecond: a workgroup that has waited some
    // ten milliseconds hands its share to the last arriver
    constexpr int DEFAULT_SPIN_LIMIT = 1 << 13;

    hipError_t launch_w4a16_gemv(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y,
                                 int M, int N, int K, int zp, int num_cu);
    // true when launch_w4a16_gemv can stage the activations of one pass in LDS
    bool w4a16_gemv_supported(int M, int K);

    // one activation row (M = 1): the row-streaming kernel
    // (N: outputs; with fusion.gate from 2 N weight rows)
    hipError_t launch_w4a16_gemv_rows(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int N,
                                      int K, int zp, int num_cu, const GemvFusion& fusion = GemvFusion());
    bool w4a16_gemv_rows_supported(int M, int N, int K, int num_cu, bool gate = false);
    // the same kernel for 4- or 8-bit weights with groups of 2^group_shift = 32 / 64 / 128 and a scalar zero point or
    // (zero_points != null) one per (row, group): 4 bits: u8 [N, (K / group + 1) / 2], even group in the low nibble;
    // 8 bits: u8 [N, K / group]
    hipError_t launch_w4a16_gemv_rows_q(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int N,
                                        int K, int group_shift, int zp, const void* zero_points, int num_cu, int bits = 4);
    bool w4a16_gemv_rows_q_supported(int M, int N, int K, int group_shift, bool zero_points, int num_cu, int bits = 4);

    // 2 <= M <= 16, K = 1024 / 2048 / 4096 / 8192: weights streamed through LDS rings, activations in registers
    // (N: outputs; gate / fusion.gate: from 2 N weight rows)
    // the same kernel for groups of 2^group_shift = 32 / 64 / 128 and a scalar zero point or (zero_points != null) one per
    // (row, group): 2 <= M <= 16, K = 2048 / 4096 / 8192, no fused parts
    hipError_t launch_w4a16_mrows_q(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M, int N,
                                    int K, int group_shift, int zp, const void* zero_points, int num_cu);
    bool w4a16_mrows_q_supported(int M, int N, int K, int group_shift, bool zero_points, int num_cu);
    // ... for 8-bit weights (u8 [N, K]; zero points u8 [N, K / group]): 2 <= M <= 16 (32 up to K = 4096), K = 2048 (groups of 32 / 64) / 4096 /
    // 8192
    hipError_t launch_w8a16_mrows_q(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M, int N,
                                    int K, int group_shift, int zp, const void* zero_points, int num_cu);
    bool w8a16_mrows_q_supported(int M, int N, int K, int group_shift, bool zero_points, int num_cu);
    // ... with K any other multiple of 256 (2 <= M <= 16).  w4a16_mrows_q_any_ranges: 0 does not apply; 1: results to Y;
    // more: fp32 sums of each range of K to partial[ranges][M][N], Y is not written (launch_wna16_reduce adds them up)
    int w4a16_mrows_q_any_ranges(int M, int N, int K, int group_shift, bool zero_points, int num_cu);
    hipError_t launch_w4a16_mrows_q_any(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, float* partial,
                                        int M, int N, int K, int group_shift, int zp, const void* zero_points, int num_cu);
    // Y [M, N] = fp16(sum over the ranges of partial[ranges][M][N])
    hipError_t launch_wna16_reduce(hipStream_t stream, const float* partial, int ranges, void* Y, int M, int N);
    hipError_t launch_w4a16_mrows(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M, int N,
                                  int K, int zp, int num_cu, const GemvFusion& fusion = GemvFusion());
    bool w4a16_mrows_supported(int M, int N, int K, int num_cu, bool gate = false);
    bool w4a16_mrows_preferred(int M, int N, int K, int num_cu, bool gate = false); // where the library picks it without being told
    // K above 8192: the same kernel over ranges of K, fp32 sums to partial[ranges][M][N] for the reduction pass
    int w4a16_mrows_ksplits(int M, int N, int K, int num_cu); // 0: does not apply
    // (gamma: fp16 [K] or null, the RMSNorm weight multiplied onto the activations)
    // sync: w4a16_mrows_split_sync_bytes() of zeroed words (zero again afterwards): the launch adds the ranges up itself, in
    // order, and writes epilogue(sums) to Y (rstd, bias, residual of `epilogue`; no gate): no reduction pass follows
    size_t w4a16_mrows_split_sync_bytes(int num_cu);
    hipError_t launch_w4a16_mrows_split(hipStream_t stream, const void* A, const void* Wq, const void* S, float* partial,
                                        int M, int N, int K, int zp, int num_cu, const void* gamma = nullptr, void* Y = nullptr,
                                        const GemvFusion* epilogue = nullptr, uint32_t* sync = nullptr);

    hipError_t launch_w4a16_skinny(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M,
                                   int N, int K, int zp, int num_cu);
    // true when one workgroup can hold the activations (M <= 16 rows of K) in LDS
    bool w4a16_skinny_supported(int M, int N, int K);

    // M <= 16 with activations too large for LDS: the same kernel over `ksplits` ranges of K, fp32 partial sums
    // [ksplits][M][N] (to be added by the GEMM's reduction pass); w4a16_skinny_ksplits returns 0 when not applicable
    int w4a16_skinny_ksplits(int M, int N, int K);
    hipError_t launch_w4a16_skinny_split(hipStream_t stream, const void* A, const void* Wq, const void* S, float* partial,
                                         int M, int N, int K, int zp, int ksplits, int num_cu);

    // Y = epilogue(prologue(A) . W^T) through the kernel that nnf::workspace::route_w4a16 names for the shape, the fused
    // parts and choice: the RMSNorm prologue and the bias / residual / SiLU-gate epilogues inside the row-streaming
    // kernels and the tile GEMM, in the reduction pass behind a GEMV kernel over ranges of K, or (MFMA GEMV kernel) as a
    // pre-pass and an element-wise kernel.  rms_ws / partial_ws: the route's rms_bytes / partial_bytes (null when 0).
    // the tile GEMM for groups of 2^group_shift = 32 / 64 / 128 and a scalar zero point or (zero_points != null) one per
    // (row, group): M > 16, K a multiple of 256; partial_ws: workspace::wna16_gemm bytes (0: not needed)
    bool w4a16_gemm_q_supported(int M, int N, int K, int group_shift);
    hipError_t launch_w4a16_gemm_q(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M, int N,
                                   int K, int group_shift, int zp, const void* zero_points, void* partial_ws, int num_cu,
                                   const LaunchChoice& choice = LaunchChoice());
    hipError_t launch_w4a16_gemm(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M,
                                 int N, int K, int zp, const void* rms_gamma, float rms_eps, const void* bias,
                                 const void* residual, int act, void* rms_ws, void* partial_ws, int num_cu,
                                 const LaunchChoice& choice = LaunchChoice());

    // ---- the nodes around a product as kernels of their own (elementwise.hip, w4a16_gemm.hip) --------------------------
    enum ElementwiseOp { EW_ADD = 0, EW_MULTIPLY = 1, EW_SIGMOID = 2, EW_SWISH = 3 }; // values of nnf_elementwise_op
    // y[r, c] = fp16(op(a[r, c], b[r, c] or (b_is_row) b[c])), fp32 arithmetic; unary operators ignore b
    hipError_t launch_elementwise(hipStream_t stream, int op, const void* a, const void* b, void* y, long long rows, int cols,
                                  bool b_is_row);
    // W fp16 [N, K] = fp16((q - z) * s): bits 4 / 8, groups of 2^group_shift, zero_points (or null: zp) as nnf_wna16_gemm takes them
    hipError_t launch_dequantize(hipStream_t stream, const void* Wq, const void* S, const void* zero_points, void* W, int N, int K,
                                 int bits, int group_shift, int zp);
    // Xn fp16 [M, K] = fp16(x * rsqrt(mean_k(x^2) + eps) * gamma[k]); K a multiple of 8
    hipError_t launch_rms_norm(hipStream_t stream, const void* X, const void* gamma, void* Xn, int M, int K, float eps);
    // Y [M, N] = fp16(SiLU(T[m, n]) * T[m, N + n]) from T fp16 [M, 2N]
    hipError_t launch_silu_gate(hipStream_t stream, const void* T, void* Y, int M, int N);
    // Y [M, N] = fp16(fp16(T + bias[n]) + residual[m, n]) (either may be null); T and residual may be Y
    hipError_t launch_bias_residual(hipStream_t stream, const void* T, void* Y, const void* bias, const void* residual, int M, int N);

    // fp16 activations x 4- or 8-bit weights, groups of 32 / 64 / 128, a scalar zero point or one per (row, group)
    // (zero_points: u8 [N, ceil(K/group * bits / 8)], 4-bit ones two to a byte, even group low): wna16_generic.hip
    bool wna16_supported(int M, int N, int K, int bits, int group);
    hipError_t launch_wna16_generic(hipStream_t stream, const void* A, const void* Wq, const void* S, void* Y, int M, int N,
                                    int K, int bits, int group, int zp, const void* zero_points, int num_cu);

    // W8A8: acc != nullptr writes the raw int32 accumulators, otherwise Y = fp16(acc * s_tok * s_ch).
    // partial_ws: w8a8_partial_bytes(...) bytes
    hipError_t launch_w8a8(hipStream_t stream, const void* A, const void* s_tok, const void* W, const void* s_ch,
                           void* Y, void* acc, int M, int N, int K, int num_cu, void* partial_ws, size_t partial_bytes,
                           const LaunchChoice& choice = LaunchChoice());
    // bytes launch_w8a8 writes at partial_ws for this call (0: the kernel it picks needs none)
    size_t w8a8_partial_bytes(int M, int N, int K, int num_cu, const LaunchChoice& choice = LaunchChoice());
    // true: the kernel it picks runs without those bytes as well (another way round, a little slower)
    bool w8a8_partial_optional(int M, int N, int K, int num_cu, const LaunchChoice& choice = LaunchChoice());
    // whether the kernel family `path` names can serve the shape
    bool w8a8_path_supported(int M, int N, int K, int num_cu, int path);
    // the MFMA GEMM behind launch_w8a8 (any M)
    hipError_t launch_w8a8_gemm(hipStream_t stream, const void* A, const void* s_tok, const void* W, const void* s_ch,
                                void* Y, void* acc, int M, int N, int K, void* partial_ws,
                                const LaunchChoice& choice = LaunchChoice());
    bool w8a8_skinny_supported(int M, int K);
    // one activation row (M = 1): the row-streaming kernel; acc != nullptr writes the raw int32 sums
    hipError_t launch_w8a8_gemv_rows(hipStream_t stream, const void* A, const void* s_tok, const void* W, const void* s_ch,
                                     void* Y, void* acc, int N, int K, int num_cu);
    bool w8a8_gemv_rows_supported(int M, int N, int K, int num_cu);
    // 2 <= M <= 32, K = 2048, 4096, 6144 or 8192: the row-streaming MFMA kernel (w8a8_mrows.hip)
    // partial_ws (workspace::w8a8_mrows_ranges_bytes(...)) and sync (workspace::mrows_split_sync_bytes(num_cu), zeroed, left
    // zero): what the form over two ranges of K needs; without either, one pass over K
    hipError_t launch_w8a8_mrows(hipStream_t stream, const void* A, const void* s_tok, const void* W, const void* s_ch,
                                 void* Y, void* acc, int M, int N, int K, int num_cu, void* partial_ws = nullptr,
                                 size_t partial_bytes = 0, uint32_t* sync = nullptr, size_t sync_bytes = 0);
    bool w8a8_mrows_supported(int M, int N, int K, int num_cu);
    bool w8a8_mrows_preferred(int M, int N, int K, int num_cu); // where the library picks it without being told

} // namespace nnf
