// C ABI of libnnf_hip_kernels.so: argument checks, dispatch by shape, error mapping.
// Declarations and the contract of each entry point are in include/nnf_hip_kernels.h.
#include "nnf_hip_kernels.h"
#include "kernels/nnf_launch.h"
#include "nnf_workspace.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <mutex>

namespace
{
    struct DeviceInfo
    {
        int num_cu = 0;
    };

    // Scratch memory owned by the library, for nnf_w4a16_gemm_static_scratch (callers that cannot allocate): parked
    // tiles / partial sums, and the synchronisation words of the one-launch tile GEMM (zero when the module is
    // loaded, and every launch leaves them zero).  Every device the library runs on holds its own copy, at its own
    // address, until the process ends.  In host code the arrays' names are only handles: the device addresses come
    // from hipGetSymbolAddress, once per device, at that entry point's first call there.
    constexpr size_t STATIC_SCRATCH_BYTES = NNF_STATIC_SCRATCH_BYTES;
    static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];
    static __device__ __align__(256) unsigned int scratch_sync[NNF_SYNC_FLAGS_BYTES / sizeof(unsigned int)];

    constexpr int MAX_DEVICES = 64;
    // Lazily cached properties of each device (with the arrays above, the only global state of the library).  A slot is
    // written once, under its once_flag, and only read afterwards.
    struct DeviceSlot
    {
        std::once_flag once;
        int status = NNF_ERR_NO_DEVICE;
        DeviceInfo info;
    };
    DeviceSlot g_dev[MAX_DEVICES];
    struct ScratchSlot
    {
        std::once_flag once;
        int status = NNF_ERR_NO_DEVICE;
        void* scratch = nullptr;
        void* sync = nullptr;
    };
    ScratchSlot g_scratch[MAX_DEVICES];

    int current_device(int& dev)
    {
        dev = -1;
        const hipError_t e = hipGetDevice(&dev);
        return (e != hipSuccess || dev < 0 || dev >= MAX_DEVICES) ? NNF_ERR_NO_DEVICE : NNF_OK;
    }

    int current_device_info(DeviceInfo& out)
    {
        int dev;
        if (current_device(dev) != NNF_OK)
            return NNF_ERR_NO_DEVICE;
        DeviceSlot& slot = g_dev[dev];
        std::call_once(slot.once, [&] {
            hipDeviceProp_t prop;
            const hipError_t e = hipGetDeviceProperties(&prop, dev);
            slot.info.num_cu = prop.multiProcessorCount;
            slot.status = e == hipSuccess ? NNF_OK : (int)e;
        });
        out = slot.info;
        return slot.status;
    }

    // the current device's copies of `scratch` and `scratch_sync` (that device is current here: the addresses are
    // those of its own copies)
    int current_static_scratch(void*& scratch_ptr, void*& sync_ptr)
    {
        int dev;
        if (current_device(dev) != NNF_OK)
            return NNF_ERR_NO_DEVICE;
        ScratchSlot& slot = g_scratch[dev];
        std::call_once(slot.once, [&] {
            hipError_t e = hipGetSymbolAddress(&slot.scratch, HIP_SYMBOL(scratch));
            if (e == hipSuccess)
                e = hipGetSymbolAddress(&slot.sync, HIP_SYMBOL(scratch_sync));
            slot.status = e == hipSuccess ? NNF_OK : (int)e;
        });
        scratch_ptr = slot.scratch;
        sync_ptr = slot.sync;
        return slot.status;
    }

    inline bool aligned16(const void* p)
    {
        return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
    }

    int check_w4a16(const void* A, const void* Wq, const void* S, const void* Y, int M, int N, int K, int group,
                    int zp)
    {
        if (!A || !Wq || !S || !Y || M <= 0 || N <= 0 || K <= 0)
            return NNF_ERR_INVALID_ARGUMENT;
        if (!aligned16(A) || !aligned16(Wq) || !aligned16(S) || !aligned16(Y))
            return NNF_ERR_INVALID_ARGUMENT;
        if (group != 128 || K % group != 0 || zp < 0 || zp > 15)
            return NNF_ERR_UNSUPPORTED_SHAPE;
        return NNF_OK;
    }
} // namespace

extern "C" {

int nnf_abi_version(void)
{
    return 4;
}

const char* nnf_status_string(int status)
{
    switch (status)
    {
    case NNF_OK: return "ok";
    case NNF_ERR_INVALID_ARGUMENT: return "invalid argument (null/misaligned pointer or non-positive size)";
    case NNF_ERR_UNSUPPORTED_SHAPE: return "unsupported shape or quantisation parameters";
    case NNF_ERR_WORKSPACE_TOO_SMALL: return "workspace too small";
    case NNF_ERR_NO_DEVICE: return "no current HIP device";
    case NNF_ERR_STATIC_SCRATCH_LIMIT:
        return "shape needs more scratch memory than the library's static buffer holds (NNF_STATIC_SCRATCH_BYTES)";
    default: break;
    }
    if (status > 0)
        return hipGetErrorString((hipError_t)status);
    return "unknown nnf status";
}

} // extern "C"

namespace
{
    // the caller's variant and plan arguments as the launchers take them; false: not a valid request
    bool make_choice(int variant, const nnf_plan* plan, int max_variant, nnf::LaunchChoice& out)
    {
        if (variant < 0 || variant > max_variant)
            return false;
        out.path = variant;
        if (plan)
        {
            const int r = plan->tile_rows;
            const int c = plan->tile_cols;
            if ((r != 0 && r != 32 && r != 64 && r != 128 && r != 256) || plan->k_parts < 0 || plan->k_parts > NNF_MAX_K_PARTS ||
                (c != 0 && c != 128 && c != 256))
                return false;
            if (plan->sync_flags && (!aligned16(plan->sync_flags) || plan->sync_flags_bytes < 8))
                return false;
            out.tile_rows = r;
            out.k_parts = plan->k_parts;
            out.tile_cols = c;
            out.sync_flags = plan->sync_flags;
            out.sync_bytes = plan->sync_flags ? plan->sync_flags_bytes : 0;
            out.spin_limit = plan->spin_limit;
        }
        return true;
    }

    // the parameters of the specialised fp16 x int4 kernels
    bool is_plain_w4a16(const nnf_quant* q) { return q->bits == 4 && q->group == 128 && !q->zero_points; }
    int group_shift_of(int group) { return group == 32 ? 5 : group == 64 ? 6 : 7; }

    // nnf_w8a8_variant -> the launchers' numbering of kernel families (that of nnf_w4a16_variant)
    int w8a8_path(int variant) { return variant == NNF_W8A8_AUTO ? 0 : variant + 1; }

    bool workspace_ok(size_t need, const void* workspace, size_t workspace_bytes)
    {
        return need == 0 || (workspace && aligned16(workspace) && workspace_bytes >= need);
    }

    int w4a16_gemm_checked(nnf_stream_t stream, const void* A, const void* Wq, const void* scales, void* Y, int M, int N,
                           int K, int group, int zp, const nnf::LaunchChoice& choice, void* workspace,
                           size_t workspace_bytes)
    {
        int st = check_w4a16(A, Wq, scales, Y, M, N, K, group, zp);
        if (st != NNF_OK)
            return st;
        DeviceInfo dev;
        st = current_device_info(dev);
        if (st != NNF_OK)
            return st;
        const hipStream_t s = (hipStream_t)stream;
        if (choice.path == NNF_W4A16_GEMV_VALU)
        {
            if (M > 16 || !nnf::w4a16_gemv_supported(M, K))
                return NNF_ERR_UNSUPPORTED_SHAPE;
            return (int)nnf::launch_w4a16_gemv(s, A, Wq, scales, Y, M, N, K, zp, dev.num_cu);
        }
        const nnf::workspace::W4A16Route route =
            nnf::workspace::route_w4a16(M, N, K, false, false, false, dev.num_cu, choice.path, choice.tile_rows, choice.k_parts,
                                        choice.tile_cols);
        if (route.kind == nnf::workspace::W4A16Route::NONE)
            return NNF_ERR_UNSUPPORTED_SHAPE;
        // the GEMV kernels over ranges of K and the tile GEMM park partial sums in scratch memory; the check is for
        // what this launch writes on this device
        if (!workspace_ok(route.partial_bytes, workspace, workspace_bytes))
            return NNF_ERR_WORKSPACE_TOO_SMALL;
        return (int)nnf::launch_w4a16_gemm(s, A, Wq, scales, Y, M, N, K, zp, nullptr, 0.f, nullptr, nullptr, NNF_ACT_NONE,
                                           nullptr, workspace, dev.num_cu, choice);
    }
} // namespace

extern "C" {

size_t nnf_w4a16_gemm_workspace_bytes(int M, int N, int K, int group)
{
    return nnf::workspace::w4a16_gemm(M, N, K, group);
}

int nnf_w4a16_gemm(nnf_stream_t stream, const void* A, const void* Wq, const void* scales, void* Y, int M, int N,
                   int K, int group, int zp, void* workspace, size_t workspace_bytes)
{
    return w4a16_gemm_checked(stream, A, Wq, scales, Y, M, N, K, group, zp, nnf::LaunchChoice(), workspace,
                              workspace_bytes);
}

int nnf_w4a16_gemm_static_scratch(nnf_stream_t stream, const void* A, const void* Wq, const void* scales, void* Y,
                                  int M, int N, int K, int group, int zp)
{
    int st = check_w4a16(A, Wq, scales, Y, M, N, K, group, zp);
    if (st != NNF_OK)
        return st;
    DeviceInfo dev;
    st = current_device_info(dev);
    if (st != NNF_OK)
        return st;
    // what the launch parks on this device
    const nnf::workspace::W4A16Route route = nnf::workspace::route_w4a16(M, N, K, false, false, false, dev.num_cu);
    if (route.kind == nnf::workspace::W4A16Route::NONE)
        return NNF_ERR_UNSUPPORTED_SHAPE;
    if (route.partial_bytes > STATIC_SCRATCH_BYTES)
        return NNF_ERR_STATIC_SCRATCH_LIMIT;
    void *buffer = nullptr, *sync = nullptr;
    st = current_static_scratch(buffer, sync);
    if (st != NNF_OK)
        return st;
    // Same kernels, with the device's static buffer in the place of the caller's workspace.  Nothing in it has to
    // start at zero: every partial sum is written before it is read.  The synchronisation words are the library's
    // own as well (zero at load, left zero by every launch): tiles shared between workgroups need no second launch.
    nnf::LaunchChoice choice;
    choice.sync_flags = sync;
    choice.sync_bytes = NNF_SYNC_FLAGS_BYTES;
    st = w4a16_gemm_checked(stream, A, Wq, scales, Y, M, N, K, group, zp, choice, buffer, STATIC_SCRATCH_BYTES);
    return st == NNF_ERR_WORKSPACE_TOO_SMALL ? NNF_ERR_STATIC_SCRATCH_LIMIT : st;
}

int nnf_wna16_supported(int M, int N, int K, const nnf_quant* q)
{
    if (!q || q->zero_point < 0 || q->zero_point >= (1 << (q->bits == 8 ? 8 : 4)))
        return 0;
    return nnf::wna16_supported(M, N, K, q->bits, q->group) ? 1 : 0;
}

size_t nnf_wna16_gemm_workspace_bytes(int M, int N, int K, const nnf_quant* q)
{
    if (!q)
        return 0;
    if (is_plain_w4a16(q))
        return nnf::workspace::w4a16_gemm(M, N, K, q->group);
    // 4-bit weights above 16 rows: the tile GEMM where tiles are shared between workgroups (without it: the plain tile kernel)
    return nnf_wna16_supported(M, N, K, q) ? nnf::workspace::wna16_gemm(M, N, K, q->bits, q->group) : 0;
}

int nnf_wna16_gemm(nnf_stream_t stream, const void* A, const void* Wq, const void* scales, void* Y, int M, int N, int K,
                   const nnf_quant* q, void* workspace, size_t workspace_bytes)
{
    return nnf_wna16_gemm_planned(stream, A, Wq, scales, Y, M, N, K, q, nullptr, workspace, workspace_bytes);
}

int nnf_wna16_gemm_planned(nnf_stream_t stream, const void* A, const void* Wq, const void* scales, void* Y, int M, int N, int K,
                           const nnf_quant* q, const nnf_plan* plan, void* workspace, size_t workspace_bytes)
{
    if (!q)
        return NNF_ERR_INVALID_ARGUMENT;
    if (is_plain_w4a16(q))
        return plan ? nnf_w4a16_gemm_variant(stream, A, Wq, scales, Y, M, N, K, q->group, q->zero_point, NNF_W4A16_AUTO, plan, workspace,
                                             workspace_bytes)
                    : nnf_w4a16_gemm(stream, A, Wq, scales, Y, M, N, K, q->group, q->zero_point, workspace, workspace_bytes);
    // (of a plan only the synchronisation words apply to these parameters)
    nnf::LaunchChoice choice;
    if (!make_choice(NNF_W4A16_AUTO, plan, NNF_W4A16_GEMV_ROWS, choice))
        return NNF_ERR_INVALID_ARGUMENT;
    choice.tile_rows = choice.k_parts = choice.tile_cols = 0;
    if (!A || !Wq || !scales || !Y || M <= 0 || N <= 0 || K <= 0)
        return NNF_ERR_INVALID_ARGUMENT;
    if (!aligned16(A) || !aligned16(Wq) || !aligned16(scales) || !aligned16(Y))
        return NNF_ERR_INVALID_ARGUMENT;
    if (!nnf_wna16_supported(M, N, K, q))
        return NNF_ERR_UNSUPPORTED_SHAPE;
    DeviceInfo dev;
    const int st = current_device_info(dev);
    if (st != NNF_OK)
        return st;
    // 4-bit weights, 2 .. 16 rows, a K the fixed-K row-streaming kernel does not take: its run-time-K form, above K = 8192
    // over ranges of K with the reduction pass (given the workspace for the sums of the ranges)
    const int gs = group_shift_of(q->group);
    if (q->bits == 4 && M >= 2 && M <= 16 && !nnf::w4a16_mrows_q_supported(M, N, K, gs, q->zero_points != nullptr, dev.num_cu))
    {
        const int ranges = nnf::w4a16_mrows_q_any_ranges(M, N, K, gs, q->zero_points != nullptr, dev.num_cu);
        if (ranges == 1)
            return (int)nnf::launch_w4a16_mrows_q_any((hipStream_t)stream, A, Wq, scales, Y, nullptr, M, N, K, gs, q->zero_point,
                                                      q->zero_points, dev.num_cu);
        if (ranges > 1 && workspace && aligned16(workspace) && workspace_bytes >= (size_t)ranges * M * N * sizeof(float))
        {
            const hipError_t e = nnf::launch_w4a16_mrows_q_any((hipStream_t)stream, A, Wq, scales, nullptr, (float*)workspace, M, N, K,
                                                               gs, q->zero_point, q->zero_points, dev.num_cu);
            if (e != hipSuccess)
                return (int)e;
            return (int)nnf::launch_wna16_reduce((hipStream_t)stream, (const float*)workspace, ranges, Y, M, N);
        }
    }
    // 4-bit weights above 16 rows: the stream-K tile GEMM, given the workspace its plan on this device needs (and
    // zero points it can fetch four bytes at a time)
    if (q->bits == 4 && nnf::w4a16_gemm_q_supported(M, N, K, group_shift_of(q->group)) &&
        !nnf::w4a16_mrows_q_supported(M, N, K, group_shift_of(q->group), q->zero_points != nullptr, dev.num_cu) &&
        (reinterpret_cast<uintptr_t>(q->zero_points) & 3) == 0)
    {
        const size_t need = nnf::workspace::wna16_gemm(M, N, K, q->bits, q->group, dev.num_cu);
        if (need == 0 || (workspace && aligned16(workspace) && workspace_bytes >= need))
            return (int)nnf::launch_w4a16_gemm_q((hipStream_t)stream, A, Wq, scales, Y, M, N, K, group_shift_of(q->group),
                                                 q->zero_point, q->zero_points, workspace, dev.num_cu, choice);
    }
    return (int)nnf::launch_wna16_generic((hipStream_t)stream, A, Wq, scales, Y, M, N, K, q->bits, q->group, q->zero_point,
                                          q->zero_points, dev.num_cu);
}

// ---- the nodes around a product as calls of their own ------------------------------------------------------------------
int nnf_elementwise_f16(nnf_stream_t stream, int op, const void* a, const void* b, void* y, size_t rows, int cols, int b_is_row)
{
    if (op < NNF_EW_ADD || op > NNF_EW_SWISH || !a || !y || rows == 0 || cols <= 0)
        return NNF_ERR_INVALID_ARGUMENT;
    const bool binary = op == NNF_EW_ADD || op == NNF_EW_MULTIPLY;
    if (binary && !b)
        return NNF_ERR_INVALID_ARGUMENT;
    if (rows > ((size_t)1 << 40) / (size_t)cols)
        return NNF_ERR_UNSUPPORTED_SHAPE;
    return (int)nnf::launch_elementwise((hipStream_t)stream, op, a, binary ? b : a, y, (long long)rows, cols, binary && b_is_row != 0);
}

int nnf_rms_norm_f16(nnf_stream_t stream, const void* x, const void* gamma, void* y, int M, int K, float eps)
{
    if (!x || !gamma || !y || M <= 0 || K <= 0 || !aligned16(x) || !aligned16(gamma) || !aligned16(y))
        return NNF_ERR_INVALID_ARGUMENT;
    if (K % 8 != 0)
        return NNF_ERR_UNSUPPORTED_SHAPE;
    return (int)nnf::launch_rms_norm((hipStream_t)stream, x, gamma, y, M, K, eps);
}

int nnf_dequantize_f16(nnf_stream_t stream, const void* Wq, const void* scales, void* W, int N, int K, const nnf_quant* q)
{
    if (!Wq || !scales || !W || !q || N <= 0 || K <= 0 || !aligned16(Wq) || !aligned16(W))
        return NNF_ERR_INVALID_ARGUMENT;
    if ((q->bits != 4 && q->bits != 8) || (q->group != 32 && q->group != 64 && q->group != 128) || K % q->group != 0 ||
        q->zero_point < 0 || q->zero_point >= (1 << q->bits))
        return NNF_ERR_UNSUPPORTED_SHAPE;
    return (int)nnf::launch_dequantize((hipStream_t)stream, Wq, scales, q->zero_points, W, N, K, q->bits, group_shift_of(q->group),
                                       q->zero_point);
}

// The fused product with other block parameters: the plain product between the kernels of the nodes around it, as the
// unfused graph would run them.  workspace = [ RMSNorm(A): M x K fp16 ][ product: M x rows fp16 ][ the product's own ]
size_t nnf_wna16_gemm_fused_workspace_bytes(int M, int N, int K, const nnf_quant* q, int act)
{
    if (!q || M <= 0 || N <= 0 || K <= 0)
        return 0;
    if (is_plain_w4a16(q))
        return nnf::workspace::w4a16_gemm_fused(M, N, K, q->group, act);
    return nnf::workspace::wna16_fused_layout(M, N, K, q->bits, q->group, true, act == NNF_ACT_SILU_GATE, true).total();
}

int nnf_wna16_gemm_fused(nnf_stream_t stream, const void* A, const void* Wq, const void* scales, void* Y, int M, int N, int K,
                         const nnf_quant* q, const void* rms_gamma, float rms_eps, const void* bias, const void* residual, int act,
                         void* workspace, size_t workspace_bytes)
{
    if (!q)
        return NNF_ERR_INVALID_ARGUMENT;
    if (is_plain_w4a16(q))
        return nnf_w4a16_gemm_fused(stream, A, Wq, scales, Y, M, N, K, q->group, q->zero_point, rms_gamma, rms_eps, bias, residual, act,
                                    workspace, workspace_bytes);
    if (!A || !Wq || !scales || !Y || M <= 0 || N <= 0 || K <= 0 || (act != NNF_ACT_NONE && act != NNF_ACT_SILU_GATE))
        return NNF_ERR_INVALID_ARGUMENT;
    if ((rms_gamma && !aligned16(rms_gamma)) || (bias && !aligned16(bias)) || (residual && !aligned16(residual)))
        return NNF_ERR_INVALID_ARGUMENT;
    const bool gate = act == NNF_ACT_SILU_GATE, rms = rms_gamma != nullptr;
    if ((gate && (bias || residual)) || (rms && K % 8 != 0))
        return NNF_ERR_UNSUPPORTED_SHAPE;
    const int rows = gate ? 2 * N : N;
    if (!nnf_wna16_supported(M, rows, K, q))
        return NNF_ERR_UNSUPPORTED_SHAPE;
    // a residual that is the output buffer itself must not be overwritten by the product
    const nnf::workspace::QFusedLayout l = nnf::workspace::wna16_fused_layout(M, N, K, q->bits, q->group, rms, gate, residual == Y);
    if (l.total() > 0 && (!workspace || !aligned16(workspace) || workspace_bytes < l.total()))
        return NNF_ERR_WORKSPACE_TOO_SMALL;
    uint8_t* ws = (uint8_t*)workspace;
    const hipStream_t s = (hipStream_t)stream;
    if (rms)
    {
        const hipError_t e = nnf::launch_rms_norm(s, A, rms_gamma, ws, M, K, rms_eps);
        if (e != hipSuccess)
            return (int)e;
        A = ws;
    }
    void* product = l.product ? (void*)(ws + l.xn) : Y;
    const int st = nnf_wna16_gemm(stream, A, Wq, scales, product, M, rows, K, q, l.gemm ? ws + l.xn + l.product : nullptr, l.gemm);
    if (st != NNF_OK)
        return st;
    if (gate)
        return (int)nnf::launch_silu_gate(s, product, Y, M, N);
    if (bias || residual)
        return (int)nnf::launch_bias_residual(s, product, Y, bias, residual, M, N);
    return NNF_OK;
}

int nnf_w4a16_variant_supported(int M, int N, int K, int group, int variant)
{
    return (group == 128 && nnf::workspace::w4a16_variant_fits(M, N, K, variant)) ? 1 : 0;
}

size_t nnf_w4a16_gemm_variant_workspace_bytes(int M, int N, int K, int group, int variant, const nnf_plan* plan)
{
    nnf::LaunchChoice choice;
    if (M <= 0 || N <= 0 || K < 128 || !make_choice(variant, plan, NNF_W4A16_GEMV_ROWS, choice))
        return 0;
    if (variant == NNF_W4A16_GEMV_VALU || group != 128)
        return 0;
    return nnf::workspace::route_w4a16(M, N, K, false, false, false, nnf::workspace::PLAN_CUS, variant, choice.tile_rows,
                                       choice.k_parts, choice.tile_cols)
        .partial_bytes;
}

int nnf_w4a16_gemm_variant(nnf_stream_t stream, const void* A, const void* Wq, const void* scales, void* Y, int M,
                           int N, int K, int group, int zp, int variant, const nnf_plan* plan, void* workspace,
                           size_t workspace_bytes)
{
    nnf::LaunchChoice choice;
    if (!make_choice(variant, plan, NNF_W4A16_GEMV_ROWS, choice))
        return NNF_ERR_INVALID_ARGUMENT;
    return w4a16_gemm_checked(stream, A, Wq, scales, Y, M, N, K, group, zp, choice, workspace, workspace_bytes);
}

size_t nnf_w4a16_gemm_fused_workspace_bytes(int M, int N, int K, int group, int act)
{
    // room for the normalised activations of the RMSNorm prologue whether or not the call uses it
    return nnf::workspace::w4a16_gemm_fused(M, N, K, group, act);
}

int nnf_w4a16_gemm_fused_variant(nnf_stream_t stream, const void* A, const void* Wq, const void* scales, void* Y, int M,
                                 int N, int K, int group, int zp, const void* rms_gamma, float rms_eps, const void* bias,
                                 const void* residual, int act, int variant, const nnf_plan* plan, void* workspace,
                                 size_t workspace_bytes)
{
    int st = check_w4a16(A, Wq, scales, Y, M, N, K, group, zp);
    if (st != NNF_OK)
        return st;
    nnf::LaunchChoice choice;
    if ((act != NNF_ACT_NONE && act != NNF_ACT_SILU_GATE) || !make_choice(variant, plan, NNF_W4A16_GEMV_ROWS, choice))
        return NNF_ERR_INVALID_ARGUMENT;
    if ((rms_gamma && !aligned16(rms_gamma)) || (bias && !aligned16(bias)) || (residual && !aligned16(residual)))
        return NNF_ERR_INVALID_ARGUMENT;
    // combinations without a fused kernel: the gate product with a bias or residual; the VALU GEMV
    if ((act == NNF_ACT_SILU_GATE && (bias || residual)) || variant == NNF_W4A16_GEMV_VALU)
        return NNF_ERR_UNSUPPORTED_SHAPE;
    DeviceInfo dev;
    st = current_device_info(dev);
    if (st != NNF_OK)
        return st;
    const nnf::workspace::W4A16Route route =
        nnf::workspace::route_w4a16(M, N, K, act == NNF_ACT_SILU_GATE, rms_gamma != nullptr, residual == Y, dev.num_cu,
                                    choice.path, choice.tile_rows, choice.k_parts, choice.tile_cols);
    if (route.kind == nnf::workspace::W4A16Route::NONE)
        return NNF_ERR_UNSUPPORTED_SHAPE;
    // [ RMSNorm scratch ][ what this launch parks, on this device ]
    if (!workspace_ok(route.rms_bytes + route.partial_bytes, workspace, workspace_bytes))
        return NNF_ERR_WORKSPACE_TOO_SMALL;
    uint8_t* ws = (uint8_t*)workspace;
    return (int)nnf::launch_w4a16_gemm((hipStream_t)stream, A, Wq, scales, Y, M, N, K, zp, rms_gamma, rms_eps, bias,
                                       residual, act, route.rms_bytes ? ws : nullptr,
                                       route.partial_bytes ? ws + route.rms_bytes : nullptr, dev.num_cu, choice);
}

int nnf_w4a16_gemm_fused(nnf_stream_t stream, const void* A, const void* Wq, const void* scales, void* Y, int M, int N,
                         int K, int group, int zp, const void* rms_gamma, float rms_eps, const void* bias,
                         const void* residual, int act, void* workspace, size_t workspace_bytes)
{
    return nnf_w4a16_gemm_fused_variant(stream, A, Wq, scales, Y, M, N, K, group, zp, rms_gamma, rms_eps, bias, residual,
                                        act, NNF_W4A16_AUTO, nullptr, workspace, workspace_bytes);
}

// ---- W8A8 ---------------------------------------------------------------------------------------
size_t nnf_w8a8_gemm_workspace_bytes(int M, int N, int K)
{
    return nnf::workspace::w8a8_gemm(M, N, K);
}

static int check_w8a8(const void* A, const void* W, const void* out, int M, int N, int K)
{
    if (!A || !W || !out || M <= 0 || N <= 0 || K <= 0)
        return NNF_ERR_INVALID_ARGUMENT;
    if (!aligned16(A) || !aligned16(W) || !aligned16(out))
        return NNF_ERR_INVALID_ARGUMENT;
    // rows must be whole 128-byte K tiles; the exact int32 sum needs K * 127 * 127 < 2^31
    if (K % 128 != 0 || K > 133000)
        return NNF_ERR_UNSUPPORTED_SHAPE;
    return NNF_OK;
}

int nnf_w8a8_variant_supported(int M, int N, int K, int variant)
{
    if (M <= 0 || N <= 0 || K <= 0 || K % 128 != 0 || K > 133000 || variant < NNF_W8A8_AUTO || variant > NNF_W8A8_GEMV_ROWS)
        return 0;
    return nnf::w8a8_path_supported(M, N, K, nnf::workspace::PLAN_CUS, w8a8_path(variant)) ? 1 : 0;
}

size_t nnf_w8a8_gemm_variant_workspace_bytes(int M, int N, int K, int variant, const nnf_plan* plan)
{
    nnf::LaunchChoice choice;
    if (!make_choice(variant, plan, NNF_W8A8_GEMV_ROWS, choice) || !nnf_w8a8_variant_supported(M, N, K, variant))
        return 0;
    choice.path = w8a8_path(variant);
    return nnf::w8a8_partial_bytes(M, N, K, nnf::workspace::PLAN_CUS, choice);
}

int nnf_w8a8_gemm_variant(nnf_stream_t stream, const void* A, const void* s_tok, const void* W, const void* s_ch, void* Y,
                          void* acc, int M, int N, int K, int variant, const nnf_plan* plan, void* workspace,
                          size_t workspace_bytes)
{
    // exactly one of the two outputs
    if ((Y != nullptr) == (acc != nullptr))
        return NNF_ERR_INVALID_ARGUMENT;
    int st = check_w8a8(A, W, Y ? Y : acc, M, N, K);
    if (st != NNF_OK)
        return st;
    nnf::LaunchChoice choice;
    if ((Y && (!s_tok || !s_ch)) || !make_choice(variant, plan, NNF_W8A8_GEMV_ROWS, choice))
        return NNF_ERR_INVALID_ARGUMENT;
    choice.path = w8a8_path(variant);
    DeviceInfo dev;
    st = current_device_info(dev);
    if (st != NNF_OK)
        return st;
    if (!nnf::w8a8_path_supported(M, N, K, dev.num_cu, choice.path))
        return NNF_ERR_UNSUPPORTED_SHAPE;
    if (!workspace_ok(nnf::w8a8_partial_bytes(M, N, K, dev.num_cu, choice), workspace, workspace_bytes))
    {
        if (!nnf::w8a8_partial_optional(M, N, K, dev.num_cu, choice))
            return NNF_ERR_WORKSPACE_TOO_SMALL;
        workspace = nullptr, workspace_bytes = 0;
    }
    return (int)nnf::launch_w8a8((hipStream_t)stream, A, Y ? s_tok : nullptr, W, Y ? s_ch : nullptr, Y, acc, M, N, K,
                                 dev.num_cu, workspace, workspace_bytes, choice);
}

int nnf_w8a8_gemm(nnf_stream_t stream, const void* A, const void* s_tok, const void* W, const void* s_ch, void* Y,
                  int M, int N, int K, void* workspace, size_t workspace_bytes)
{
    if (!Y)
        return NNF_ERR_INVALID_ARGUMENT;
    return nnf_w8a8_gemm_variant(stream, A, s_tok, W, s_ch, Y, nullptr, M, N, K, NNF_W8A8_AUTO, nullptr, workspace,
                                 workspace_bytes);
}

int nnf_w8a8_gemm_acc(nnf_stream_t stream, const void* A, const void* W, void* acc, int M, int N, int K,
                      void* workspace, size_t workspace_bytes)
{
    if (!acc)
        return NNF_ERR_INVALID_ARGUMENT;
    return nnf_w8a8_gemm_variant(stream, A, nullptr, W, nullptr, nullptr, acc, M, N, K, NNF_W8A8_AUTO, nullptr, workspace,
                                 workspace_bytes);
}

// ---- fused MLP block ------------------------------------------------------------------------------
// workspace = [ RMSNorm(x): M x H fp16 ][ h: M x I fp16 ][ split-K partial sums of either GEMM ]
size_t nnf_fused_mlp_w4a16_workspace_bytes(int M, int H, int I, int group)
{
    return nnf::workspace::fused_mlp_w4a16(M, H, I, group);
}

int nnf_fused_mlp_w4a16(nnf_stream_t stream, const void* x, const void* gamma, float eps, const void* Wgu,
                        const void* Sgu, const void* Wd, const void* Sd, void* out, int M, int H, int I, int group,
                        int zp, void* workspace, size_t workspace_bytes)
{
    return nnf_fused_mlp_w4a16_planned(stream, x, gamma, eps, Wgu, Sgu, Wd, Sd, out, M, H, I, group, zp, nullptr, nullptr,
                                       workspace, workspace_bytes);
}

int nnf_fused_mlp_w4a16_planned(nnf_stream_t stream, const void* x, const void* gamma, float eps, const void* Wgu,
                                const void* Sgu, const void* Wd, const void* Sd, void* out, int M, int H, int I, int group,
                                int zp, const nnf_plan* gate_up_plan, const nnf_plan* down_plan, void* workspace,
                                size_t workspace_bytes)
{
    nnf::LaunchChoice choice_gu, choice_d;
    if (!make_choice(NNF_W4A16_AUTO, gate_up_plan, NNF_W4A16_GEMV_ROWS, choice_gu) ||
        !make_choice(NNF_W4A16_AUTO, down_plan, NNF_W4A16_GEMV_ROWS, choice_d))
        return NNF_ERR_INVALID_ARGUMENT;
    // a plan that fixes the tile shape or the split means the tile GEMM
    if (choice_gu.tile_rows || choice_gu.k_parts || choice_gu.tile_cols)
        choice_gu.path = NNF_W4A16_GEMM_MFMA;
    if (choice_d.tile_rows || choice_d.k_parts || choice_d.tile_cols)
        choice_d.path = NNF_W4A16_GEMM_MFMA;
    if (!x || !gamma || !Wgu || !Sgu || !Wd || !Sd || !out || M <= 0 || H <= 0 || I <= 0)
        return NNF_ERR_INVALID_ARGUMENT;
    if (!aligned16(x) || !aligned16(gamma) || !aligned16(Wgu) || !aligned16(Sgu) || !aligned16(Wd) ||
        !aligned16(Sd) || !aligned16(out) || !aligned16(workspace))
        return NNF_ERR_INVALID_ARGUMENT;
    if (group != 128 || H % group != 0 || I % group != 0 || zp < 0 || zp > 15)
        return NNF_ERR_UNSUPPORTED_SHAPE;
    DeviceInfo dev;
    int st = current_device_info(dev);
    if (st != NNF_OK)
        return st;
    // workspace = [ rstd of the first product ][ h: M x I fp16 ][ what either launch parks, on this device ] (the down
    // projection's residual is x: in place when the caller passes out == x)
    const nnf::workspace::W4A16Route route_gu = nnf::workspace::route_w4a16(
        M, I, H, true, true, false, dev.num_cu, choice_gu.path, choice_gu.tile_rows, choice_gu.k_parts, choice_gu.tile_cols);
    const nnf::workspace::W4A16Route route_d = nnf::workspace::route_w4a16(
        M, H, I, false, false, out == x, dev.num_cu, choice_d.path, choice_d.tile_rows, choice_d.k_parts, choice_d.tile_cols);
    if (route_gu.kind == nnf::workspace::W4A16Route::NONE || route_d.kind == nnf::workspace::W4A16Route::NONE)
        return NNF_ERR_UNSUPPORTED_SHAPE;
    const size_t h_offset = route_gu.rms_bytes;
    const size_t partial_offset = h_offset + nnf::workspace::align256((size_t)M * I * 2);
    const size_t parked = route_gu.partial_bytes > route_d.partial_bytes ? route_gu.partial_bytes : route_d.partial_bytes;
    if (!workspace || workspace_bytes < partial_offset + parked)
        return NNF_ERR_WORKSPACE_TOO_SMALL;
    uint8_t* ws = (uint8_t*)workspace;
    void* h = ws + h_offset;
    void* partial = ws + partial_offset;
    // h = SiLU(gate) * up, gate|up = RMSNorm(x) . Wgu^T : one GEMM with the gate and up projections as the two halves
    // of every N tile, the RMSNorm weight and rstd inside it
    hipError_t e = nnf::launch_w4a16_gemm((hipStream_t)stream, x, Wgu, Sgu, h, M, I, H, zp, gamma, eps, nullptr,
                                          nullptr, NNF_ACT_SILU_GATE, ws, partial, dev.num_cu, choice_gu);
    if (e != hipSuccess)
        return (int)e;
    // out = h . Wd^T + x
    e = nnf::launch_w4a16_gemm((hipStream_t)stream, h, Wd, Sd, out, M, H, I, zp, nullptr, 0.f, nullptr, x, NNF_ACT_NONE,
                               nullptr, partial, dev.num_cu, choice_d);
    return (int)e;
}

// workspace = [ RMSNorm(x): M x H fp16 ][ gate | up products: M x 2I fp16, then the down product: M x H fp16 ][ h: M x I fp16 ]
//             [ the products' own ]
size_t nnf_fused_mlp_wna16_workspace_bytes(int M, int H, int I, const nnf_quant* q_gate_up, const nnf_quant* q_down)
{
    if (!q_gate_up || !q_down || M <= 0 || H <= 0 || I <= 0)
        return 0;
    if (is_plain_w4a16(q_gate_up) && is_plain_w4a16(q_down) && q_gate_up->zero_point == q_down->zero_point)
        return nnf::workspace::fused_mlp_w4a16(M, H, I, 128);
    const int bits = q_gate_up->bits, group = q_gate_up->group;
    return nnf::workspace::fused_mlp_wna16(M, H, I, bits, group);
}

int nnf_fused_mlp_wna16(nnf_stream_t stream, const void* x, const void* gamma, float eps, const void* Wgu, const void* Sgu,
                        const void* Wd, const void* Sd, void* out, int M, int H, int I, const nnf_quant* q_gate_up,
                        const nnf_quant* q_down, void* workspace, size_t workspace_bytes)
{
    if (!q_gate_up || !q_down)
        return NNF_ERR_INVALID_ARGUMENT;
    if (is_plain_w4a16(q_gate_up) && is_plain_w4a16(q_down) && q_gate_up->zero_point == q_down->zero_point)
        return nnf_fused_mlp_w4a16(stream, x, gamma, eps, Wgu, Sgu, Wd, Sd, out, M, H, I, 128, q_gate_up->zero_point, workspace,
                                   workspace_bytes);
    if (!x || !gamma || !Wgu || !Sgu || !Wd || !Sd || !out || M <= 0 || H <= 0 || I <= 0)
        return NNF_ERR_INVALID_ARGUMENT;
    if (!aligned16(x) || !aligned16(gamma) || !aligned16(out) || !aligned16(workspace))
        return NNF_ERR_INVALID_ARGUMENT;
    if (H % 8 != 0 || q_gate_up->bits != q_down->bits || q_gate_up->group != q_down->group ||
        !nnf_wna16_supported(M, 2 * I, H, q_gate_up) || !nnf_wna16_supported(M, H, I, q_down))
        return NNF_ERR_UNSUPPORTED_SHAPE;
    if (!workspace || workspace_bytes < nnf_fused_mlp_wna16_workspace_bytes(M, H, I, q_gate_up, q_down))
        return NNF_ERR_WORKSPACE_TOO_SMALL;
    const size_t wide = (size_t)(2 * I > H ? 2 * I : H);
    uint8_t* xn = (uint8_t*)workspace;
    uint8_t* product = xn + nnf::workspace::align256((size_t)M * H * 2);
    uint8_t* h = product + nnf::workspace::align256((size_t)M * wide * 2);
    uint8_t* own = h + nnf::workspace::align256((size_t)M * I * 2);
    const size_t own_bytes = workspace_bytes - (size_t)(own - xn);
    const hipStream_t s = (hipStream_t)stream;
    // the nodes of the block, one after the other, fp16 tensors between them
    hipError_t e = nnf::launch_rms_norm(s, x, gamma, xn, M, H, eps);
    if (e != hipSuccess)
        return (int)e;
    int st = nnf_wna16_gemm(stream, xn, Wgu, Sgu, product, M, 2 * I, H, q_gate_up, own, own_bytes);
    if (st != NNF_OK)
        return st;
    e = nnf::launch_silu_gate(s, product, h, M, I);
    if (e != hipSuccess)
        return (int)e;
    st = nnf_wna16_gemm(stream, h, Wd, Sd, product, M, H, I, q_down, own, own_bytes);
    if (st != NNF_OK)
        return st;
    return (int)nnf::launch_bias_residual(s, product, out, nullptr, x, M, H); // out may be x
}

} // extern "C"
