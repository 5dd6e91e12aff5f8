"""ctypes loaders for the native libraries.  There is no fallback: a missing library raises."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.join(_HERE, "lib")
KERNELS_SO = os.path.join(LIB_DIR, "libnnf_hip_kernels.so")
HOST_SO = os.path.join(LIB_DIR, "libnnf_host.so")

_kernels = None
_host = None

_c_int = ctypes.c_int
_c_vp = ctypes.c_void_p
_c_sz = ctypes.c_size_t
_c_f = ctypes.c_float


class NativeLibraryMissing(RuntimeError):
    pass


def _load(path):
    if not os.path.exists(path):
        raise NativeLibraryMissing(
            f"{path} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
            "(or `make -C nnfusion_amd/csrc`). There is no CPU or PyTorch fallback for this path.")
    return ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)


# name -> (restype, argtypes): exactly the declarations of include/nnf_hip_kernels.h
KERNEL_ABI = {
    "nnf_abi_version": (_c_int, []),
    "nnf_status_string": (ctypes.c_char_p, [_c_int]),
    "nnf_w4a16_gemm_workspace_bytes": (_c_sz, [_c_int] * 4),
    "nnf_w4a16_gemm": (_c_int, [_c_vp] * 5 + [_c_int] * 5 + [_c_vp, _c_sz]),
    "nnf_w4a16_gemm_static_scratch": (_c_int, [_c_vp] * 5 + [_c_int] * 5),
    "nnf_w4a16_variant_supported": (_c_int, [_c_int] * 5),
    "nnf_w4a16_gemm_variant_workspace_bytes": (_c_sz, [_c_int] * 5 + [_c_vp]),
    "nnf_w4a16_gemm_variant": (_c_int, [_c_vp] * 5 + [_c_int] * 6 + [_c_vp, _c_vp, _c_sz]),
    "nnf_wna16_supported": (_c_int, [_c_int] * 3 + [_c_vp]),
    "nnf_wna16_gemm_workspace_bytes": (_c_sz, [_c_int] * 3 + [_c_vp]),
    "nnf_wna16_gemm": (_c_int, [_c_vp] * 5 + [_c_int] * 3 + [_c_vp, _c_vp, _c_sz]),
    "nnf_wna16_gemm_planned": (_c_int, [_c_vp] * 5 + [_c_int] * 3 + [_c_vp, _c_vp, _c_vp, _c_sz]),
    "nnf_w4a16_gemm_fused_workspace_bytes": (_c_sz, [_c_int] * 5),
    "nnf_w4a16_gemm_fused": (_c_int, [_c_vp] * 5 + [_c_int] * 5 + [_c_vp, _c_f, _c_vp, _c_vp, _c_int, _c_vp, _c_sz]),
    "nnf_w4a16_gemm_fused_variant": (_c_int, [_c_vp] * 5 + [_c_int] * 5 + [_c_vp, _c_f, _c_vp, _c_vp, _c_int, _c_int, _c_vp,
                                              _c_vp, _c_sz]),
    "nnf_w8a8_variant_supported": (_c_int, [_c_int] * 4),
    "nnf_w8a8_gemm_variant_workspace_bytes": (_c_sz, [_c_int] * 4 + [_c_vp]),
    "nnf_w8a8_gemm_variant": (_c_int, [_c_vp] * 7 + [_c_int] * 4 + [_c_vp, _c_vp, _c_sz]),
    "nnf_w8a8_gemm_workspace_bytes": (_c_sz, [_c_int] * 3),
    "nnf_w8a8_gemm": (_c_int, [_c_vp] * 6 + [_c_int] * 3 + [_c_vp, _c_sz]),
    "nnf_w8a8_gemm_acc": (_c_int, [_c_vp] * 4 + [_c_int] * 3 + [_c_vp, _c_sz]),
    "nnf_fused_mlp_w4a16_workspace_bytes": (_c_sz, [_c_int] * 4),
    "nnf_fused_mlp_w4a16": (_c_int, [_c_vp, _c_vp, _c_vp, _c_f] + [_c_vp] * 5 + [_c_int] * 5 + [_c_vp, _c_sz]),
    "nnf_elementwise_f16": (_c_int, [_c_vp, _c_int, _c_vp, _c_vp, _c_vp, _c_sz, _c_int, _c_int]),
    "nnf_rms_norm_f16": (_c_int, [_c_vp] * 4 + [_c_int, _c_int, _c_f]),
    "nnf_dequantize_f16": (_c_int, [_c_vp] * 4 + [_c_int, _c_int, _c_vp]),
    "nnf_wna16_gemm_fused_workspace_bytes": (_c_sz, [_c_int] * 3 + [_c_vp, _c_int]),
    "nnf_wna16_gemm_fused": (_c_int, [_c_vp] * 5 + [_c_int] * 3 + [_c_vp, _c_vp, _c_f, _c_vp, _c_vp, _c_int, _c_vp, _c_sz]),
    "nnf_fused_mlp_wna16_workspace_bytes": (_c_sz, [_c_int] * 3 + [_c_vp, _c_vp]),
    "nnf_fused_mlp_wna16": (_c_int, [_c_vp, _c_vp, _c_vp, _c_f] + [_c_vp] * 5 + [_c_int] * 3 + [_c_vp, _c_vp, _c_vp, _c_sz]),
    "nnf_fused_mlp_w4a16_planned": (_c_int, [_c_vp, _c_vp, _c_vp, _c_f] + [_c_vp] * 5 + [_c_int] * 5 + [_c_vp, _c_vp, _c_vp, _c_sz]),
}


def kernels():
    """libnnf_hip_kernels.so with argtypes set (loads on a CPU-only host too; calls need a GPU)."""
    global _kernels
    if _kernels is None:
        lib = _load(KERNELS_SO)
        for name, (res, args) in KERNEL_ABI.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _kernels = lib
    return _kernels


def host():
    """libnnf_host.so (pure host C++)."""
    global _host
    if _host is None:
        lib = _load(HOST_SO)
        u64, dbl = ctypes.c_uint64, ctypes.c_double
        lib.nnf_gen_normal_f16.argtypes = [u64, u64, dbl, dbl, _c_vp, _c_sz]
        lib.nnf_gen_uniform_f16.argtypes = [u64, u64, dbl, dbl, _c_vp, _c_sz]
        lib.nnf_gen_uniform_f32.argtypes = [u64, u64, dbl, dbl, _c_vp, _c_sz]
        lib.nnf_gen_uniform_u4_packed.argtypes = [u64, u64, _c_vp, _c_sz]
        lib.nnf_gen_uniform_i8.argtypes = [u64, u64, _c_int, _c_int, _c_vp, _c_sz]
        for fn in (lib.nnf_gen_normal_f16, lib.nnf_gen_uniform_f16, lib.nnf_gen_uniform_f32,
                   lib.nnf_gen_uniform_u4_packed, lib.nnf_gen_uniform_i8):
            fn.restype = None
        lib.nnf_f32_to_f16_bits.argtypes = [_c_f]
        lib.nnf_f32_to_f16_bits.restype = ctypes.c_uint16
        lib.nnf_f16_bits_to_f32.argtypes = [ctypes.c_uint16]
        lib.nnf_f16_bits_to_f32.restype = _c_f
        _host = lib
    return _host
