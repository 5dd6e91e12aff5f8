/*
 * nnf_hip_kernels.h -- C ABI of the gfx950 (MI355X) low-bit GEMM/GEMV launcher library
 * (libnnf_hip_kernels.so).
 *
 * These entry points are what an nnfusion kernel emitter for the quantized Dot/MatMul node
 * puts in its emitted function body, in the place where the reference's cuda::Dot emitter
 * puts a cuBLAS call (src/nnfusion/core/kernels/cuda_gpu/kernels/dot.cpp:128-205 for fp32,
 * :271-363 for fp16) and where FunctionFile emits the `extern void <kernel>_Call(grids, blocks,
 * mem, stream, args...)` host wrappers (src/nnfusion/engine/pass/codegen/codegenerator_helper.cpp:
 * 143-177).  Every function
 *   - takes plain device pointers and sizes (no C++ types, no torch types),
 *   - is stream ordered: it enqueues on `stream` and returns without synchronising,
 *   - never allocates: scratch memory is passed in (`workspace`, 16-byte aligned), sized by the
 *     matching `*_workspace_bytes` query -- pure host arithmetic on the shape, an upper bound, 0 for
 *     shapes that need none -- so that an emitter can reserve it at compile time with
 *     KernelEmitter::allocate_tensor (src/nnfusion/core/kernels/kernel_emitter.cpp:282-319).
 *     It holds, as the shape requires: the normalised activations of the RMSNorm prologue, the
 *     fp32 / int32 partial sums of a GEMM whose K range is split across workgroups, the MLP's h,
 *   - never throws: it returns NNF_OK (0), a negative NNF_ERR_* code for a rejected call, or a
 *     positive hipError_t value reported by the HIP runtime.
 *
 * Tensor layouts (all dense, row-major, base pointers 16-byte aligned; the reference's memory
 * planner aligns every tensor to 64 bytes, src/nnfusion/engine/device/rocm.cpp:86):
 *   A       fp16  [M, K]            activations
 *   Wq      u8    [N, K/2]          unsigned 4-bit weights, two per byte along K:
 *                                   low nibble of byte b of a row = k 2b, high nibble = k 2b+1
 *   scales  fp16  [N, K/group]      one scale per output channel and K-group (group = 128)
 *   zp      int   scalar            zero point (8): W[n,k] = (q[n,k] - zp) * scales[n, k/group]
 *   Y       fp16  [M, N]            Y = A . W^T, accumulated in fp32, rounded to nearest even
 * Input range: any finite fp16 activations, subnormals included.  No kernel rescales the activations; the
 * 4-bit weights are decoded to exact fp16 integers (q - zp, or q plus a constant that is removed from the fp32
 * sum), so a product a * (q - zp) is exact in fp32 whatever the magnitude of a.  The scales are applied in fp32
 * (GEMV kernels: to the fp32 sum of a group) or as fp16((q - zp) * scale) weights (tile GEMM); a result beyond
 * the fp16 range becomes +-inf as in any fp16 tensor.
 *   W8A8:   A i8 [M,K], s_tok f32 [M], W i8 [N,K], s_ch f32 [N], acc i32 [M,N] (exact),
 *           Y = fp16( (float)acc * s_tok[m] * s_ch[n] ) evaluated left to right in fp32
 */
#ifndef NNF_HIP_KERNELS_H
#define NNF_HIP_KERNELS_H

#include <stddef.h>
#include <stdint.h>

/* The library is built with hidden visibility; these declarations are its whole exported surface. */
#ifndef NNF_API
#define NNF_API __attribute__((visibility("default")))
#endif

#ifdef __cplusplus
extern "C" {
#endif

/* A hipStream_t, passed as an opaque pointer so that this header needs no HIP include. */
typedef void* nnf_stream_t;

enum nnf_status
{
    NNF_OK = 0,
    NNF_ERR_INVALID_ARGUMENT = -1, /* null pointer, non-positive size, misaligned pointer */
    NNF_ERR_UNSUPPORTED_SHAPE = -2, /* K % group != 0, group != 128, K % 32 != 0, zp outside 0..15 ... */
    NNF_ERR_WORKSPACE_TOO_SMALL = -3,
    NNF_ERR_NO_DEVICE = -4, /* no gfx950 device is current */
    NNF_ERR_STATIC_SCRATCH_LIMIT = -5 /* nnf_w4a16_gemm_static_scratch: the shape needs more than NNF_STATIC_SCRATCH_BYTES */
};

/* ABI version of this header (bumped on any signature change). */
NNF_API int nnf_abi_version(void);

/* Human-readable text for a status returned by any function below (static storage). */
NNF_API const char* nnf_status_string(int status);

/* ---------------------------------------------------------------------------------------------
 * fp16 x int4 (group-scaled) GEMM / GEMV:  Y[M,N] = A[M,K] . ((Wq - zp) * scales)^T
 * Replaces the cublasHgemm / cublasSgemm call of cuda::Dot (cuda_gpu/kernels/dot.cpp:128-205,
 * :271-363) for a weight-quantized Dot node with transpose_B = true.  By shape: M = 1 the row-streaming
 * GEMV kernel; 2 <= M <= 32 (40 for long K) the row-streaming MFMA kernel, over ranges of K (partial sums in
 * `workspace`, then a reduction pass) where the activations exceed one workgroup's registers; other M <= 16
 * shapes the MFMA GEMV kernel over K ranges; everything else the MFMA tile GEMM, whose work is split evenly
 * over the CUs (tiles shared by several workgroups are summed through `workspace` by a second launch).
 * ------------------------------------------------------------------------------------------- */
NNF_API size_t nnf_w4a16_gemm_workspace_bytes(int M, int N, int K, int group);

NNF_API int nnf_w4a16_gemm(nnf_stream_t stream,
                   const void* A, const void* Wq, const void* scales, void* Y,
                   int M, int N, int K, int group, int zp,
                   void* workspace, size_t workspace_bytes);

/* nnf_w4a16_gemm for callers that can neither allocate nor pass a workspace (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same kernels and
 * results as nnf_w4a16_gemm (the tile GEMM in its one-launch form, see nnf_plan::sync_flags, with synchronisation
 * words of the library's own); the partial sums of a GEMM whose K range is split go to a buffer of
 * NNF_STATIC_SCRATCH_BYTES that the library holds in device memory (a static __device__ array: each GPU the
 * library is used on keeps its own copy until the process ends).  Calls no hipMalloc / hipFree.  A shape whose
 * nnf_w4a16_gemm_workspace_bytes exceeds the buffer is rejected with NNF_ERR_STATIC_SCRATCH_LIMIT.  All calls
 * on one GPU share the buffer: calls that overlap on one GPU (different streams) race; calls on one stream
 * are ordered and safe.  The first call of this entry point on a device looks the buffer's address up
 * (hipGetSymbolAddress): make that call outside stream capture. */
#define NNF_STATIC_SCRATCH_BYTES ((size_t)32 << 20)
NNF_API int nnf_w4a16_gemm_static_scratch(nnf_stream_t stream,
                                  const void* A, const void* Wq, const void* scales, void* Y,
                                  int M, int N, int K, int group, int zp);

/* The kernels behind nnf_w4a16_gemm as separate, selectable variants: what several registered emitters
 * for one operator are to ProfilingBasedKernelSelector::profiling_best
 * (engine/pass/graph/kernel_selection.cpp:21-73), which times every emitter that accepts the node and keeps
 * the fastest.  NNF_W4A16_AUTO is nnf_w4a16_gemm itself (a built-in choice by shape). */
enum nnf_w4a16_variant
{
    NNF_W4A16_AUTO = 0,
    NNF_W4A16_GEMV_VALU = 1, /* M <= 16: v_dot2 GEMV, exact (q - zp) unpacking; cross-check implementation */
    NNF_W4A16_GEMV_MFMA = 2, /* M <= 16: MFMA 16x16x32 weight-streaming kernel (activations held per workgroup; over ranges
                                of K with partial sums in the workspace when they exceed its LDS) */
    NNF_W4A16_GEMM_MFMA = 3, /* any M: MFMA 32x32x16 tile GEMM (may split K: workspace) */
    NNF_W4A16_GEMV_ROWS = 4  /* row-streaming kernels, one workgroup per CU: M = 1 (K a multiple of 256, 1024 .. 16384),
                                M = 2 .. 16 on MFMA (K a multiple of 256, 1024 .. 8192, N >= 16), M = 17 .. 32 up to K = 4096;
                                longer K (to 65536; M = 33 .. 40: 2048 < K <= 4096) over ranges of K with partial sums
                                in the workspace */
};
/* What else a candidate may fix about the tile GEMM (variant NNF_*_GEMM_MFMA; ignored by the other variants).
 * Passed per call: the library keeps no dispatch state, calls with different plans may run concurrently.
 * NULL, or a field that is 0: the library's own choice for the shape. */
#define NNF_MAX_K_PARTS 64
/* Synchronisation words for the one-launch forms of the fp16 x int4 kernels: two 32-bit words per output tile of the
 * tile GEMM and two more; a buffer of NNF_SYNC_FLAGS_BYTES serves every shape up to 8191 tiles (a launch with more
 * tiles than the buffer given takes the two-launch form). */
#define NNF_SYNC_FLAGS_BYTES ((size_t)64 << 10)
typedef struct nnf_plan
{
    int tile_rows; /* rows of an output tile: 256, 128, 64 (fp16 x int4 also 32); see tile_cols for their width
                      (W8A8 128-row tiles: 128 columns, 64-row tiles: 256) */
    int k_parts;   /* fp16 x int4: workgroups that share one output tile, each a contiguous part of K, summed by a
                      second launch (the grid is tiles x k_parts, work split evenly); W8A8: ranges of K, int32
                      partial sums added exactly by a reduction pass.  At most NNF_MAX_K_PARTS (and never more
                      workgroups than the product has units of 256 k). */
    int tile_cols; /* columns of an output tile, 256 or 128 (0: the library's choice): W8A8 with 256-row tiles;
                      fp16 x int4 with 64-, 128- or 256-row tiles and no SiLU-gate (the gate | up halves need the
                      256 weight rows of a full tile); ignored elsewhere */
    /* fp16 x int4 products in one launch (any variant that ends up on one of the kernels below; ignored by every other
     * kernel; W8A8: see the last sentence).
     * The work of the GEMM is split evenly over the CUs, so most output tiles of a mid-sized product are shared by
     * several workgroups.  Without sync_flags their parts are added up by a second launch.  With sync_flags the
     * workgroups count themselves in at their tiles there, and each adds up and finishes its share of a tile's rows
     * once all that hold a part have arrived -- same summation order, bit-identical results, one launch less.
     * (A plan whose grid has more workgroups than the device has CUs keeps the second launch: workgroups that wait
     * for one another must all be running.)
     * Two more launches go the same way: a fused RMSNorm's rstd[] is computed by the GEMM launch itself (every
     * workgroup a few rows before its first tile; no pass of its own), and the row-streaming kernel for a few
     * activation rows and K above 8192, which works on ranges of K, adds the ranges up itself (the last workgroup to
     * arrive at a group of columns, in the order of the ranges; no reduction pass).  W8A8 with 8 .. 32 rows and K from
     * 8192 runs its row-streaming kernel over two ranges of K the same way (int32 sums: exact), given sync_flags and
     * nnf_w8a8_gemm_variant_workspace_bytes of workspace; without either, in one pass over K (same bits, ~1 us more).
     *   sync_flags: device memory, 16-byte aligned, ALL ZERO before the first call that uses it; every call leaves it
     *     all zero again, so it needs clearing once (when it is allocated), not per call.  It must not be scratch
     *     memory that other kernels write between calls, and calls that may overlap on the device (different
     *     streams) need buffers of their own.  The reference's counterpart is the persistent, zero-initialised
     *     `be_state_buffer` tensor of its BlockFusion kernels
     *     (src/nnfusion/engine/pass/graph/blockfusion/blockfusion_codegen.cpp:295-304): an emitter reserves it
     *     with KernelEmitter::allocate_tensor + set_memset(true, 0) + set_persistent(true).
     *   sync_flags_bytes: its size; NNF_SYNC_FLAGS_BYTES always suffices.
     *   spin_limit: how many times (about a microsecond each) a workgroup polls for the other arrivals before it hands
     *     its share of the rows to the last workgroup to arrive, which never waits (so a launch whose workgroups are
     *     not all resident at once still ends).  0: the library's default (some ten milliseconds); negative: do not
     *     wait at all (every tile is then finished by its last arriver; for tests of that path). */
    void* sync_flags;
    size_t sync_flags_bytes;
    int spin_limit;
} nnf_plan;
/* 1 when the variant can serve the shape (decided on the host, for a 256-CU device), else 0. */
NNF_API int nnf_w4a16_variant_supported(int M, int N, int K, int group, int variant);
/* Upper bound for a 256-CU device; the call itself checks what its launch writes on the device at hand. */
NNF_API size_t nnf_w4a16_gemm_variant_workspace_bytes(int M, int N, int K, int group, int variant, const nnf_plan* plan);
/* As nnf_w4a16_gemm through the given variant; NNF_ERR_UNSUPPORTED_SHAPE when it cannot serve the shape,
 * NNF_ERR_INVALID_ARGUMENT for a variant or plan value outside the ones listed. */
NNF_API int nnf_w4a16_gemm_variant(nnf_stream_t stream,
                           const void* A, const void* Wq, const void* scales, void* Y,
                           int M, int N, int K, int group, int zp, int variant, const nnf_plan* plan,
                           void* workspace, size_t workspace_bytes);

/* The same product with every block parameter the reference's dequantisation takes: its Dequantize scales and
 * offsets are tensors over blocks of any shape (core/kernels/cpu/reference/kernels.cpp:601-623: integer subtract of
 * the offset, cast, multiply by the scale), and the ONNX operator that carries such weights (MatMulNBits) stores
 * `bits`, `block_size` and an optional zero-point tensor.
 *   w[n,k] = (q[n,k] - z[n, k / group]) * scales[n, k / group]
 *   bits = 4 : Wq u8 [N, K/2], weight k in the low (k even) or high (k odd) nibble of byte k/2
 *   bits = 8 : Wq u8 [N, K]
 *   zero_points == NULL : z = zero_point everywhere (0 .. 2^bits - 1)
 *   zero_points != NULL : u8 [N, ceil(K/group * bits / 8)], one per (row, group); 4-bit ones packed two to a byte along
 *                         the groups of a row, even group in the low nibble
 * bits 4, group 128 and no zero-point tensor is nnf_w4a16_gemm itself (same kernels, same workspace).  For every other
 * combination (group 32 / 64 / 128, K a multiple of group) 4-bit weights run on the kernels of nnf_w4a16_gemm where
 * those apply: the row-streaming kernels for M = 1 with K a multiple of 256 from 1024 to 16384 and for 2 <= M <= 16
 * with K a multiple of 256 from about 2560 on (2048 / 4096 also up to 32 rows; above K = 8192 over ranges of K with a
 * reduction pass), and the tile GEMM for the other shapes above 16 rows with K a multiple of 256 and zero_points
 * 4-byte aligned.  The ranges of K and the tile GEMM want nnf_wna16_gemm_workspace_bytes of workspace; called with
 * less (or NULL) the product runs on a plain kernel instead, at about half the rate.
 * Everything else runs on plain kernels that need no workspace: a row-per-wavefront GEMV for M = 1, an MFMA kernel
 * with the operands fetched straight into registers for 2 <= M <= 16, MFMA tiles through LDS above. */
typedef struct nnf_quant
{
    int bits;                /* 4 or 8 */
    int group;               /* 32, 64 or 128 */
    int zero_point;          /* used when zero_points is NULL */
    const void* zero_points; /* device pointer or NULL */
} nnf_quant;
/* 1 when nnf_wna16_gemm serves the shape with these parameters (zero_points is not read), else 0. */
NNF_API int nnf_wna16_supported(int M, int N, int K, const nnf_quant* q);
NNF_API size_t nnf_wna16_gemm_workspace_bytes(int M, int N, int K, const nnf_quant* q);
NNF_API int nnf_wna16_gemm(nnf_stream_t stream,
                   const void* A, const void* Wq, const void* scales, void* Y,
                   int M, int N, int K, const nnf_quant* q,
                   void* workspace, size_t workspace_bytes);
/* The same with an nnf_plan (NULL: nnf_wna16_gemm): its sync_flags make the tile GEMM of these parameters a single
 * launch, as they do for nnf_w4a16_gemm_variant (same contract: all zero before the first call, left all zero by every
 * call); the tile fields apply to 4 bits / 128 / no zero-point tensor only (the other parameters keep the library's tile
 * shapes).  Same results bit for bit. */
NNF_API int nnf_wna16_gemm_planned(nnf_stream_t stream,
                   const void* A, const void* Wq, const void* scales, void* Y,
                   int M, int N, int K, const nnf_quant* q, const nnf_plan* plan,
                   void* workspace, size_t workspace_bytes);

/* ---------------------------------------------------------------------------------------------
 * The nodes around a quantized product, for graphs in which no fusion pattern absorbed them (a gate
 * product with a second consumer, a normalisation that feeds something else as well, ...): fp16
 * tensors, fp32 arithmetic, one rounding to fp16 per node.  The reference emits such nodes through its
 * element-wise emitter (cuda_gpu/kernels/elementwise.cpp; the operators' bodies are the CudaOpMap entries
 * of cuda_gpu/cuda_kernelops.hpp:408 Add, :416 Multiply, :447-451 Sigmoid) and layer_norm.cpp.
 * ------------------------------------------------------------------------------------------- */
enum nnf_elementwise_op
{
    NNF_EW_ADD = 0,      /* a + b */
    NNF_EW_MULTIPLY = 1, /* a * b */
    NNF_EW_SIGMOID = 2,  /* 1 / (1 + exp(-a)) */
    NNF_EW_SWISH = 3     /* a * sigmoid(a) */
};
/* y[r, c] = op(a[r, c], b[r, c]) over fp16 [rows, cols]; b_is_row != 0: b is [cols], the same for every row
 * (a bias).  Unary operators ignore b.  y may be a or b. */
NNF_API int nnf_elementwise_f16(nnf_stream_t stream, int op, const void* a, const void* b, void* y,
                        size_t rows, int cols, int b_is_row);
/* y[m, :] = x[m, :] * rsqrt(mean_k(x[m, k]^2) + eps) * gamma  (rsqrt(x + eps) as in the reference's LayerNorm,
 * cuda_gpu/cuda_langunit.cpp:618; the reference has no RMSNorm operator).  K a multiple of 8. */
NNF_API int nnf_rms_norm_f16(nnf_stream_t stream, const void* x, const void* gamma, void* y, int M, int K, float eps);
/* W fp16 [N, K] = (q - zero point) * scale per block of `group` weights along K: the reference's Dequantize
 * (core/kernels/cpu/reference/kernels.cpp:601-623: integer subtract, cast, multiply) for the weight layouts of
 * nnf_wna16_gemm.  For a Dequantize node that does not feed a product (one that does is folded into it). */
NNF_API int nnf_dequantize_f16(nnf_stream_t stream, const void* Wq, const void* scales, void* W, int N, int K, const nnf_quant* q);

/* Epilogue / prologue selectors for nnf_w4a16_gemm_fused. */
enum nnf_activation
{
    NNF_ACT_NONE = 0,
    /* Wq/scales hold 2N rows: rows [0,N) are the gate projection, rows [N,2N) the up projection;
       Y[M,N] = SiLU(gate) * up with SiLU(g) = g * 1/(1+exp(-g))
       (sigmoid as in cuda_gpu/cuda_kernelops.hpp:447-451, multiply :416). */
    NNF_ACT_SILU_GATE = 1
};

/* Same GEMM with prologue / epilogue in one call.  They run inside the kernel that serves the shape: the
 * row-streaming kernels (M = 1; M <= 32) and the tile GEMM multiply gamma in on the way in, rstd[m] and the
 * epilogue at their end.  The row-streaming kernels add up the squares of the activations they hold themselves
 * (K a multiple of 1024 up to 8192; M = 1: any K they take): one launch in all; the tile GEMM and the other
 * forms take rstd from a small pre-pass over A (fp32 [M] in `workspace`); a GEMV kernel over ranges of K
 * leaves rstd and the epilogue to its reduction pass.  Only the MFMA GEMV kernel (M <= 16 with K not a
 * multiple of 256) reads normalised activations written to `workspace` by a pre-pass and leaves its
 * products to one element-wise kernel.
 *   rms_gamma != NULL : A is replaced by RMSNorm(A) = A * rsqrt(mean_k(A^2) + rms_eps) * gamma[k]
 *                       (rsqrt(x + eps) as in LayerNorm, cuda_gpu/cuda_langunit.cpp:618)
 *   bias      != NULL : fp16 [N], added to every row (MatMulAdd precedent,
 *                       cuda_gpu/kernels/matmuladd.cpp:29-93)
 *   residual  != NULL : fp16 [M,N], added element-wise (Add, cuda_kernelops.hpp:408);
 *                       may alias Y
 *   act               : nnf_activation
 */
NNF_API size_t nnf_w4a16_gemm_fused_workspace_bytes(int M, int N, int K, int group, int act);

NNF_API int nnf_w4a16_gemm_fused(nnf_stream_t stream,
                         const void* A, const void* Wq, const void* scales, void* Y,
                         int M, int N, int K, int group, int zp,
                         const void* rms_gamma, float rms_eps,
                         const void* bias, const void* residual, int act,
                         void* workspace, size_t workspace_bytes);

/* nnf_w4a16_gemm_fused as a selectable candidate: any variant but NNF_W4A16_GEMV_VALU (which has no fused form:
 * NNF_ERR_UNSUPPORTED_SHAPE, as for a variant that cannot serve the shape); `plan` for the tile GEMM.
 * A workspace of nnf_w4a16_gemm_fused_workspace_bytes + nnf_w4a16_gemm_variant_workspace_bytes(.., plan) of the
 * weight rows (2N with NNF_ACT_SILU_GATE) always suffices. */
NNF_API int nnf_w4a16_gemm_fused_variant(nnf_stream_t stream,
                                 const void* A, const void* Wq, const void* scales, void* Y,
                                 int M, int N, int K, int group, int zp,
                                 const void* rms_gamma, float rms_eps,
                                 const void* bias, const void* residual, int act,
                                 int variant, const nnf_plan* plan,
                                 void* workspace, size_t workspace_bytes);

/* nnf_w4a16_gemm_fused for every block parameter of nnf_wna16_gemm (act == NNF_ACT_SILU_GATE: Wq, scales and the zero
 * points hold 2N rows).  4 bits / groups of 128 / a scalar zero point is nnf_w4a16_gemm_fused itself; the other
 * combinations run the nodes one after the other -- RMSNorm (into `workspace`), the product on nnf_wna16_gemm's
 * kernels, one element-wise kernel for the epilogue -- with the fp16 tensors of the unfused graph between them. */
NNF_API size_t nnf_wna16_gemm_fused_workspace_bytes(int M, int N, int K, const nnf_quant* q, int act);
NNF_API int nnf_wna16_gemm_fused(nnf_stream_t stream,
                         const void* A, const void* Wq, const void* scales, void* Y,
                         int M, int N, int K, const nnf_quant* q,
                         const void* rms_gamma, float rms_eps,
                         const void* bias, const void* residual, int act,
                         void* workspace, size_t workspace_bytes);

/* ---------------------------------------------------------------------------------------------
 * W8A8: int8 x int8 -> int32 on the int8 MFMA, then the per-token / per-channel dequantisation.
 * The reference has no emitter for this; the nearest routine in its tree is MLAS's u8 x s8
 * MlasGemm (thirdparty/mlas/inc/mlas.h:147-163).
 * ------------------------------------------------------------------------------------------- */
NNF_API size_t nnf_w8a8_gemm_workspace_bytes(int M, int N, int K);

/* Y fp16 [M,N] = fp16((float)acc * s_tok[m] * s_ch[n]) */
NNF_API int nnf_w8a8_gemm(nnf_stream_t stream,
                  const void* A, const void* s_tok, const void* W, const void* s_ch, void* Y,
                  int M, int N, int K,
                  void* workspace, size_t workspace_bytes);

/* Raw accumulators: acc i32 [M,N] = A . W^T (exact). */
NNF_API int nnf_w8a8_gemm_acc(nnf_stream_t stream,
                      const void* A, const void* W, void* acc,
                      int M, int N, int K,
                      void* workspace, size_t workspace_bytes);

/* The kernels behind nnf_w8a8_gemm as selectable variants (see nnf_w4a16_variant); `plan` as above (tile_rows, tile_cols and
 * k_parts for the tile GEMM; sync_flags for the row-streaming kernel over two ranges of K). */
enum nnf_w8a8_variant
{
    NNF_W8A8_AUTO = 0,
    NNF_W8A8_GEMV_MFMA = 1, /* M <= 16: int8 MFMA kernel over ranges of K inside one workgroup */
    NNF_W8A8_GEMM_MFMA = 2, /* any M: int8 MFMA 32x32x32 tile GEMM (may split K: workspace) */
    NNF_W8A8_GEMV_ROWS = 3  /* row-streaming kernels: M = 1; M = 2 .. 32 on MFMA (K a multiple of 256, 1024 .. 16384) */
};
NNF_API int nnf_w8a8_variant_supported(int M, int N, int K, int variant);
NNF_API size_t nnf_w8a8_gemm_variant_workspace_bytes(int M, int N, int K, int variant, const nnf_plan* plan);
/* Exactly one of Y (with s_tok, s_ch) and acc is non-NULL: the fp16 result or the raw int32 accumulators. */
NNF_API int nnf_w8a8_gemm_variant(nnf_stream_t stream,
                          const void* A, const void* s_tok, const void* W, const void* s_ch, void* Y, void* acc,
                          int M, int N, int K, int variant, const nnf_plan* plan,
                          void* workspace, size_t workspace_bytes);

/* ---------------------------------------------------------------------------------------------
 * Fused Llama-style MLP block (one emitted function for the sub-graph
 *   RMSNorm -> QuantDot(gate|up) -> SiLU*mul -> QuantDot(down) -> Add(residual) ):
 *   out[M,H] = x + W_down . ( SiLU(W_gate . n) * (W_up . n) ),  n = RMSNorm(x, gamma, eps)
 * Wgu u8 [2I, H/2] (gate rows then up rows), Sgu fp16 [2I, H/group], Wd u8 [H, I/2],
 * Sd fp16 [H, I/group].  Intermediates in `workspace`: rstd fp32 [M] (RMSNorm(x) itself is never
 * written: gamma is multiplied in inside the first product's kernel, rstd at its end), h fp16 [M, I],
 * and the partial sums of a product that several workgroups share; SiLU, the gate product and the
 * residual add touch no memory of their own.  (Shapes that only the MFMA GEMV kernel serves -- up to
 * 16 rows with K not a multiple of 256 -- still go through RMSNorm(x) fp16 [M, H] and gate | up
 * fp16 [M, 2I] in the workspace.)
 * `out` may be `x` itself (the residual is then added in place); no other buffers may overlap.
 * The element-wise semantics follow the reference's ops (Sigmoid, Multiply, Add, Rsqrt:
 * cuda_gpu/cuda_kernelops.hpp:206-210,408,416,447-451); the reference has no RMSNorm op.
 * ------------------------------------------------------------------------------------------- */
NNF_API size_t nnf_fused_mlp_w4a16_workspace_bytes(int M, int H, int I, int group);

NNF_API int nnf_fused_mlp_w4a16(nnf_stream_t stream,
                        const void* x, const void* gamma, float eps,
                        const void* Wgu, const void* Sgu, const void* Wd, const void* Sd,
                        void* out,
                        int M, int H, int I, int group, int zp,
                        void* workspace, size_t workspace_bytes);

/* The same block with an nnf_plan for each of its two products (NULL: the library's own choice): the tile shapes a
 * profiling selector wants to try, and the sync_flags that make each tile GEMM a single launch (both plans may name
 * the same buffer: the two products run one after the other on `stream`).  A plan that fixes a tile shape or k_parts
 * puts that product on the tile GEMM.  Workspace: nnf_fused_mlp_w4a16_workspace_bytes for NULL plans or plans that
 * only carry sync_flags; with a fixed tile shape add nnf_w4a16_gemm_variant_workspace_bytes of that product
 * (gate | up: M x 2I x H; down: M x H x I). */
NNF_API int nnf_fused_mlp_w4a16_planned(nnf_stream_t stream,
                                const void* x, const void* gamma, float eps,
                                const void* Wgu, const void* Sgu, const void* Wd, const void* Sd,
                                void* out,
                                int M, int H, int I, int group, int zp,
                                const nnf_plan* gate_up_plan, const nnf_plan* down_plan,
                                void* workspace, size_t workspace_bytes);

/* The same block for every block parameter of nnf_wna16_gemm, one nnf_quant per weight matrix (their zero-point
 * tensors differ).  Both plain (4 bits, groups of 128, the same scalar zero point): nnf_fused_mlp_w4a16 itself;
 * otherwise the nodes one after the other, as nnf_wna16_gemm_fused does. */
NNF_API size_t nnf_fused_mlp_wna16_workspace_bytes(int M, int H, int I, const nnf_quant* q_gate_up, const nnf_quant* q_down);
NNF_API int nnf_fused_mlp_wna16(nnf_stream_t stream,
                        const void* x, const void* gamma, float eps,
                        const void* Wgu, const void* Sgu, const void* Wd, const void* Sd,
                        void* out,
                        int M, int H, int I, const nnf_quant* q_gate_up, const nnf_quant* q_down,
                        void* workspace, size_t workspace_bytes);

#ifdef __cplusplus
}
#endif

#endif /* NNF_HIP_KERNELS_H */
