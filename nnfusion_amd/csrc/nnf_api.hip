// C ABI of libnnf_hip_kernels.so: argument checks, dispatch by shape, error mapping.
// Declarations and the contract of each entry point are in include/nnf_hip_kernels.h.
#include "nnf_hip_kernels.h"
#include "kernels/nnf_launch.h"
#include "nnf_workspace.h"

#include <hip/hip_runtime.h>

namespace
{
    struct DeviceInfo
    {
        int valid = 0;
        int num_cu = 0;
        void* static_scratch = nullptr; // this device's copy of `scratch` below
    };

    // Scratch memory owned by the library, for nnf_w4a16_gemm_static_scratch (callers that cannot allocate).
    // Every device the library runs on holds its own copy, at its own address, until the process ends.  In host
    // code the array's name is only a handle: the device address comes from hipGetSymbolAddress, once per device.
    constexpr size_t STATIC_SCRATCH_BYTES = NNF_STATIC_SCRATCH_BYTES;
    static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

    // Lazily cached properties of each device (with `scratch`, the only global state of the library).
    DeviceInfo g_dev[64];

    int current_device_info(DeviceInfo& out)
    {
        int dev = -1;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess || dev < 0 || dev >= 64)
            return NNF_ERR_NO_DEVICE;
        if (!g_dev[dev].valid)
        {
            hipDeviceProp_t prop;
            e = hipGetDeviceProperties(&prop, dev);
            if (e != hipSuccess)
                return (int)e;
            g_dev[dev].num_cu = prop.multiProcessorCount;
            // device `dev` is current here: the address is that of its own copy
            void* ptr = nullptr;
            e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
            if (e != hipSuccess)
                return (int)e;
            g_dev[dev].static_scratch = ptr;
            g_dev[dev].valid = 1;
        }
        out = g_dev[dev];
        return NNF_OK;
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

namespace nnf
{
    Tuning g_tuning;
}

extern "C" {

// experiment hook, deliberately absent from the public header
int nnf_internal_tune(int key, int value)
{
    switch (key)
    {
    case 0: nnf::g_tuning.force_path = value; return 0;
    case 1: nnf::g_tuning.skinny_cps = value; return 0;
    case 2: nnf::g_tuning.skinny_wg_per_cu = value; return 0;
    case 3: nnf::g_tuning.gemm_tile = value; return 0;
    case 4: nnf::g_tuning.gemm_splits = value; return 0;
    case 5: nnf::workspace::skinny_min_splits() = value; return 0;
    case 6: nnf::skinny_direct_min_rows() = value > 0 ? value : 6; return 0;
    case 7: nnf::workspace::mrows_forced_ranges() = value; return 0;
    default: return -1;
    }
}

int nnf_abi_version(void)
{
    return 1;
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
    // partial-sum bytes of the GEMM plan in force (the automatic one unless an experiment overrides it)
    // fused: a call that may run the GEMV kernel into scratch (fp16 [M, N or 2N]) ahead of an element-wise epilogue
    size_t tuned_partial_bytes(int M, int N, int K, bool gate, bool fused = false)
    {
        static const int forced_rows[5] = {0, 256, 128, 64, 32};
        const int f_rows = forced_rows[nnf::g_tuning.gemm_tile >= 0 && nnf::g_tuning.gemm_tile <= 4 ? nnf::g_tuning.gemm_tile : 0];
        const size_t a =
            nnf::workspace::plan_w4a16_sk_with(M, N, K, gate, nnf::workspace::PLAN_CUS, f_rows, nnf::g_tuning.gemm_splits).bytes();
        // the M <= 16 kernels over ranges of K write partial sums too
        const size_t b = nnf::workspace::skinny_split_bytes(M, gate ? 2 * N : N, K);
        const size_t c = nnf::workspace::mrows_split_bytes(M, gate ? 2 * N : N, K);
        const size_t d = fused ? nnf::workspace::gemv_scratch_bytes(M, gate ? 2 * N : N) : 0;
        const size_t bc = b > c ? b : c, ad = a > d ? a : d;
        return ad > bc ? ad : bc;
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
    int st = check_w4a16(A, Wq, scales, Y, M, N, K, group, zp);
    if (st != NNF_OK)
        return st;
    DeviceInfo dev;
    st = current_device_info(dev);
    if (st != NNF_OK)
        return st;
    const int force = nnf::g_tuning.force_path;
    if ((force == 0 || force == 4) && nnf::w4a16_gemv_rows_supported(M, N, K, dev.num_cu))
        return (int)nnf::launch_w4a16_gemv_rows((hipStream_t)stream, A, Wq, scales, Y, N, K, zp, dev.num_cu);
    if ((force == 5 && nnf::w4a16_mrows_supported(M, N, K, dev.num_cu)) ||
        (force == 0 && nnf::w4a16_mrows_preferred(M, N, K, dev.num_cu)))
        return (int)nnf::launch_w4a16_mrows((hipStream_t)stream, A, Wq, scales, Y, M, N, K, zp, dev.num_cu);
    if ((force == 0 || force == 2 || force == 4 || force == 5) && M <= 16 && nnf::w4a16_skinny_supported(M, N, K))
        return (int)nnf::launch_w4a16_skinny((hipStream_t)stream, A, Wq, scales, Y, M, N, K, zp, dev.num_cu);
    if (force == 1 && M <= 16 && nnf::w4a16_gemv_supported(M, K))
        return (int)nnf::launch_w4a16_gemv((hipStream_t)stream, A, Wq, scales, Y, M, N, K, zp, dev.num_cu);
    // the MFMA GEMM may split K and then needs room for its partial sums (the GEMV kernels need none)
    const size_t need = tuned_partial_bytes(M, N, K, false);
    if (need > 0 && (!workspace || !aligned16(workspace) || workspace_bytes < need))
        return NNF_ERR_WORKSPACE_TOO_SMALL;
    return (int)nnf::launch_w4a16_gemm((hipStream_t)stream, A, Wq, scales, Y, M, N, K, zp, nullptr, 0.f, nullptr,
                                       nullptr, NNF_ACT_NONE, nullptr, workspace, dev.num_cu);
}

int nnf_w4a16_gemm_static_scratch(nnf_stream_t stream, const void* A, const void* Wq, const void* scales, void* Y,
                                  int M, int N, int K, int group, int zp)
{
    int st = check_w4a16(A, Wq, scales, Y, M, N, K, group, zp);
    if (st != NNF_OK)
        return st;
    // the partial sums of every path nnf_w4a16_gemm may take for this shape
    if (nnf::workspace::w4a16_gemm(M, N, K, group) > STATIC_SCRATCH_BYTES)
        return NNF_ERR_STATIC_SCRATCH_LIMIT;
    DeviceInfo dev;
    st = current_device_info(dev);
    if (st != NNF_OK)
        return st;
    // Same kernels, with the device's static buffer in the place of the caller's workspace.  Nothing in it has to
    // start at zero: every partial sum is written by the GEMM kernel before the reduction pass reads it.
    return nnf_w4a16_gemm(stream, A, Wq, scales, Y, M, N, K, group, zp, dev.static_scratch, STATIC_SCRATCH_BYTES);
}

int nnf_w4a16_variant_supported(int M, int N, int K, int group, int variant)
{
    return (group == 128 && nnf::workspace::w4a16_variant_fits(M, N, K, variant)) ? 1 : 0;
}

size_t nnf_w4a16_gemm_variant_workspace_bytes(int M, int N, int K, int group, int variant)
{
    if (M <= 0 || N <= 0 || K < 128)
        return 0;
    if (variant == NNF_W4A16_GEMM_MFMA)
        return nnf::workspace::plan_w4a16_sk(M, N, K, false, nnf::workspace::PLAN_CUS).bytes();
    if (variant == NNF_W4A16_AUTO)
        return nnf::workspace::w4a16_gemm(M, N, K, group);
    return 0;
}

int nnf_w4a16_gemm_variant(nnf_stream_t stream, const void* A, const void* Wq, const void* scales, void* Y, int M,
                           int N, int K, int group, int zp, int variant, void* workspace, size_t workspace_bytes)
{
    if (variant == NNF_W4A16_AUTO)
        return nnf_w4a16_gemm(stream, A, Wq, scales, Y, M, N, K, group, zp, workspace, workspace_bytes);
    int st = check_w4a16(A, Wq, scales, Y, M, N, K, group, zp);
    if (st != NNF_OK)
        return st;
    if (variant < NNF_W4A16_AUTO || variant > NNF_W4A16_GEMV_ROWS)
        return NNF_ERR_INVALID_ARGUMENT;
    DeviceInfo dev;
    st = current_device_info(dev);
    if (st != NNF_OK)
        return st;
    switch (variant)
    {
    case NNF_W4A16_GEMV_ROWS:
        if (M > 1 && nnf::w4a16_mrows_supported(M, N, K, dev.num_cu))
            return (int)nnf::launch_w4a16_mrows((hipStream_t)stream, A, Wq, scales, Y, M, N, K, zp, dev.num_cu);
        if (!nnf::w4a16_gemv_rows_supported(M, N, K, dev.num_cu))
            return NNF_ERR_UNSUPPORTED_SHAPE;
        return (int)nnf::launch_w4a16_gemv_rows((hipStream_t)stream, A, Wq, scales, Y, N, K, zp, dev.num_cu);
    case NNF_W4A16_GEMV_MFMA:
        if (!nnf::workspace::w4a16_skinny_fits(M, N, K))
            return NNF_ERR_UNSUPPORTED_SHAPE;
        return (int)nnf::launch_w4a16_skinny((hipStream_t)stream, A, Wq, scales, Y, M, N, K, zp, dev.num_cu);
    case NNF_W4A16_GEMV_VALU:
        if (M > 16 || !nnf::w4a16_gemv_supported(M, K))
            return NNF_ERR_UNSUPPORTED_SHAPE;
        return (int)nnf::launch_w4a16_gemv((hipStream_t)stream, A, Wq, scales, Y, M, N, K, zp, dev.num_cu);
    default: break;
    }
    const size_t need = nnf_w4a16_gemm_variant_workspace_bytes(M, N, K, group, NNF_W4A16_GEMM_MFMA);
    if (need > 0 && (!workspace || !aligned16(workspace) || workspace_bytes < need))
        return NNF_ERR_WORKSPACE_TOO_SMALL;
    return (int)nnf::launch_w4a16_gemm((hipStream_t)stream, A, Wq, scales, Y, M, N, K, zp, nullptr, 0.f, nullptr,
                                       nullptr, NNF_ACT_NONE, nullptr, workspace, dev.num_cu, true);
}

size_t nnf_w4a16_gemm_fused_workspace_bytes(int M, int N, int K, int group, int act)
{
    // room for the normalised activations of the RMSNorm prologue whether or not the call uses it
    return nnf::workspace::w4a16_gemm_fused(M, N, K, group, act);
}

int nnf_w4a16_gemm_fused(nnf_stream_t stream, const void* A, const void* Wq, const void* scales, void* Y, int M, int N,
                         int K, int group, int zp, const void* rms_gamma, float rms_eps, const void* bias,
                         const void* residual, int act, void* workspace, size_t workspace_bytes)
{
    int st = check_w4a16(A, Wq, scales, Y, M, N, K, group, zp);
    if (st != NNF_OK)
        return st;
    if (act != NNF_ACT_NONE && act != NNF_ACT_SILU_GATE)
        return NNF_ERR_INVALID_ARGUMENT;
    if ((rms_gamma && !aligned16(rms_gamma)) || (bias && !aligned16(bias)) || (residual && !aligned16(residual)))
        return NNF_ERR_INVALID_ARGUMENT;
    // combinations without a fused kernel (see launch_w4a16_gemm)
    if (act == NNF_ACT_SILU_GATE && (bias || residual))
        return NNF_ERR_UNSUPPORTED_SHAPE;
    const size_t need = (rms_gamma ? nnf::workspace::rms_rows(M, K) : 0) + tuned_partial_bytes(M, N, K, act == NNF_ACT_SILU_GATE, true);
    if (need > 0 && (!workspace || !aligned16(workspace) || workspace_bytes < need))
        return NNF_ERR_WORKSPACE_TOO_SMALL;
    DeviceInfo dev;
    st = current_device_info(dev);
    if (st != NNF_OK)
        return st;
    uint8_t* ws = (uint8_t*)workspace;
    return (int)nnf::launch_w4a16_gemm((hipStream_t)stream, A, Wq, scales, Y, M, N, K, zp, rms_gamma, rms_eps, bias,
                                       residual, act, ws, ws ? ws + (rms_gamma ? nnf::workspace::rms_rows(M, K) : 0) : nullptr,
                                       dev.num_cu);
}

// ---- W8A8 ---------------------------------------------------------------------------------------
size_t nnf_w8a8_gemm_workspace_bytes(int M, int N, int K)
{
    return nnf::workspace::w8a8_gemm(M, N, K);
}

// room for the int32 partial sums when the MFMA GEMM serves the shape (the M <= 16 kernel needs none)
static int check_w8a8_workspace(int M, int N, int K, int num_cu, const void* workspace, size_t workspace_bytes)
{
    if ((nnf::g_tuning.force_path == 0 || nnf::g_tuning.force_path == 4) && nnf::w8a8_gemv_rows_supported(M, N, K, num_cu))
        return NNF_OK;
    if ((nnf::g_tuning.force_path == 5 && nnf::w8a8_mrows_supported(M, N, K, num_cu)) ||
        (nnf::g_tuning.force_path == 0 && nnf::w8a8_mrows_preferred(M, N, K, num_cu)))
        return NNF_OK;
    if (nnf::g_tuning.force_path != 3 && nnf::w8a8_skinny_supported(M, K))
        return NNF_OK;
    const size_t need = nnf::workspace::gemm_partial_bytes(
        M, N, false, nnf::workspace::plan_w8a8_gemm(M, N, K, nnf::g_tuning.gemm_tile - 1, nnf::g_tuning.gemm_splits));
    if (need > 0 && (!workspace || !aligned16(workspace) || workspace_bytes < need))
        return NNF_ERR_WORKSPACE_TOO_SMALL;
    return NNF_OK;
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

int nnf_w8a8_gemm(nnf_stream_t stream, const void* A, const void* s_tok, const void* W, const void* s_ch, void* Y,
                  int M, int N, int K, void* workspace, size_t workspace_bytes)
{
    int st = check_w8a8(A, W, Y, M, N, K);
    if (st != NNF_OK)
        return st;
    if (!s_tok || !s_ch)
        return NNF_ERR_INVALID_ARGUMENT;
    DeviceInfo dev;
    st = current_device_info(dev);
    if (st != NNF_OK)
        return st;
    st = check_w8a8_workspace(M, N, K, dev.num_cu, workspace, workspace_bytes);
    if (st != NNF_OK)
        return st;
    return (int)nnf::launch_w8a8((hipStream_t)stream, A, s_tok, W, s_ch, Y, nullptr, M, N, K, dev.num_cu, workspace);
}

int nnf_w8a8_gemm_acc(nnf_stream_t stream, const void* A, const void* W, void* acc, int M, int N, int K,
                      void* workspace, size_t workspace_bytes)
{
    int st = check_w8a8(A, W, acc, M, N, K);
    if (st != NNF_OK)
        return st;
    DeviceInfo dev;
    st = current_device_info(dev);
    if (st != NNF_OK)
        return st;
    st = check_w8a8_workspace(M, N, K, dev.num_cu, workspace, workspace_bytes);
    if (st != NNF_OK)
        return st;
    return (int)nnf::launch_w8a8((hipStream_t)stream, A, nullptr, W, nullptr, nullptr, acc, M, N, K, dev.num_cu,
                                 workspace);
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
    if (!x || !gamma || !Wgu || !Sgu || !Wd || !Sd || !out || M <= 0 || H <= 0 || I <= 0)
        return NNF_ERR_INVALID_ARGUMENT;
    if (!aligned16(x) || !aligned16(gamma) || !aligned16(Wgu) || !aligned16(Sgu) || !aligned16(Wd) ||
        !aligned16(Sd) || !aligned16(out) || !aligned16(workspace))
        return NNF_ERR_INVALID_ARGUMENT;
    if (group != 128 || H % group != 0 || I % group != 0 || zp < 0 || zp > 15)
        return NNF_ERR_UNSUPPORTED_SHAPE;
    {
        const size_t a = tuned_partial_bytes(M, I, H, true, true), b = tuned_partial_bytes(M, H, I, false);
        if (!workspace || workspace_bytes < nnf::workspace::fused_mlp_partial_offset(M, H, I) + (a > b ? a : b))
            return NNF_ERR_WORKSPACE_TOO_SMALL;
    }
    DeviceInfo dev;
    int st = current_device_info(dev);
    if (st != NNF_OK)
        return st;
    uint8_t* ws = (uint8_t*)workspace;
    void* h = ws + nnf::workspace::fused_mlp_h_offset(M, H);
    void* partial = ws + nnf::workspace::fused_mlp_partial_offset(M, H, I);
    // h = SiLU(gate) * up, gate|up = RMSNorm(x) . Wgu^T : the normalisation pre-pass, then one GEMM with the
    // gate and up projections as the two halves of every N tile
    hipError_t e = nnf::launch_w4a16_gemm((hipStream_t)stream, x, Wgu, Sgu, h, M, I, H, zp, gamma, eps, nullptr,
                                          nullptr, NNF_ACT_SILU_GATE, ws, partial, dev.num_cu);
    if (e != hipSuccess)
        return (int)e;
    // out = h . Wd^T + x
    e = nnf::launch_w4a16_gemm((hipStream_t)stream, h, Wd, Sd, out, M, H, I, zp, nullptr, 0.f, nullptr, x, NNF_ACT_NONE,
                               nullptr, partial, dev.num_cu);
    return (int)e;
}

} // extern "C"
