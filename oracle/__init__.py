"""TEST INFRASTRUCTURE: ctypes front of the CPU oracle (oracle/liboracle.so) and, when it has been
built, of the reference's own MLAS (oracle/_ref/libmlas_ref.so).  Only tests/, the smoke check and
the cpu_baseline leg of bench.py may import this package; the product never does."""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(_HERE, "liboracle.so")
MLAS_REF_SO = os.path.join(_HERE, "_ref", "libmlas_ref.so")

_vp, _i, _sz, _f, _d = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t, ctypes.c_float, ctypes.c_double
_lib = None
_ref = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(ORACLE_SO):
            raise RuntimeError(f"{ORACLE_SO} not built (make -C oracle)")
        L = ctypes.CDLL(ORACLE_SO)
        sig = {
            "oracle_max_threads": (_i, []),
            "oracle_f16_to_f32": (None, [_vp, _vp, _sz]),
            "oracle_f32_to_f16": (None, [_vp, _vp, _sz]),
            "oracle_dequantize_w4": (None, [_vp, _vp, _i, _i, _i, _i, _vp]),
            "oracle_dot_f32": (None, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i]),
            "oracle_dot_general": (None, [_vp, _vp, _i, _vp, _vp, _i, _i, _vp]),
            "oracle_gemm_nt_f64": (None, [_vp, _vp, _vp, _i, _i, _i]),
            "oracle_dequantize_wn": (None, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
            "oracle_wna16_gemm": (None, [_vp, _vp, _vp, _vp, _vp] + [_i] * 8),
            "oracle_w4a16_gemm_f32": (None, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i]),
            "oracle_w4a16_gemm": (None, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i]),
            "oracle_w8a8_acc": (None, [_vp, _vp, _vp, _i, _i, _i, _i]),
            "oracle_w8a8_acc_i64": (None, [_vp, _vp, _vp, _i, _i, _i]),
            "oracle_w8a8_epilogue": (None, [_vp, _vp, _vp, _vp, _i, _i]),
            "oracle_w8a8_gemm": (None, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i]),
            "oracle_sigmoid": (_f, [_f]),
            "oracle_rmsnorm_f16": (None, [_vp, _vp, _f, _vp, _i, _i]),
            "oracle_silu_mul_f16": (None, [_vp, _vp, _vp, _sz]),
            "oracle_add_f16": (None, [_vp, _vp, _vp, _sz]),
            "oracle_fused_mlp_w4a16": (None, [_vp, _vp, _f, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i]),
            "oracle_time_dot_f32": (_d, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp]),
            "oracle_time_w8a8_acc": (_d, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp]),
        }
        for name, (res, args) in sig.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def mlas_ref():
    """The reference's MLAS, or None when oracle/_ref has not been built."""
    global _ref
    if _ref is None and os.path.exists(MLAS_REF_SO):
        L = ctypes.CDLL(MLAS_REF_SO)
        L.mlas_ref_sgemm.restype = None
        L.mlas_ref_sgemm.argtypes = [_i, _i, _sz, _sz, _sz, _vp, _sz, _vp, _sz, _vp, _sz]
        L.mlas_ref_qgemm_u8s8.restype = None
        L.mlas_ref_qgemm_u8s8.argtypes = [_sz, _sz, _sz, _vp, _sz, ctypes.c_uint8, _vp, _sz, ctypes.c_int8, _vp, _sz]
        L.mlas_ref_time_sgemm_nt.restype = _d
        L.mlas_ref_time_sgemm_nt.argtypes = [_sz, _sz, _sz, _vp, _vp, _vp, _i, _i, _vp]
        _ref = L
    return _ref


def _c(a, dtype):
    a = np.ascontiguousarray(a)
    assert a.dtype == dtype, (a.dtype, dtype)
    return a


def _p(a):
    return a.ctypes.data


def f32_to_f16(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().oracle_f32_to_f16(_p(x), _p(out), x.size)
    return out.view(np.float16)


def f16_to_f32(x):
    x = _c(x.view(np.uint16), np.uint16)
    out = np.empty(x.shape, np.float32)
    lib().oracle_f16_to_f32(_p(x), _p(out), x.size)
    return out


def dequantize_w4(wq, scales, group=128, zp=8):
    wq = _c(wq, np.uint8)
    s = _c(scales.view(np.uint16), np.uint16)
    n, k = wq.shape[0], wq.shape[1] * 2
    out = np.empty((n, k), np.float32)
    lib().oracle_dequantize_w4(_p(wq), _p(s), n, k, group, zp, _p(out))
    return out


def dot_f32(a, b, trans_a=False, trans_b=False, threads=0):
    """2-D Dot as cpu::DotMlas: op(a) [M,K] . op(b) [K,N]."""
    a = _c(a, np.float32)
    b = _c(b, np.float32)
    m, k = (a.shape[1], a.shape[0]) if trans_a else a.shape
    n = b.shape[0] if trans_b else b.shape[1]
    assert (b.shape[1] if trans_b else b.shape[0]) == k
    out = np.empty((m, n), np.float32)
    lib().oracle_dot_f32(_p(a), _p(b), _p(out), m, n, k, int(trans_a), int(trans_b), threads)
    return out


def dot_general(a, b, reduction_axes):
    a = _c(a, np.float32)
    b = _c(b, np.float32)
    ad = np.array(a.shape, np.int64)
    bd = np.array(b.shape, np.int64)
    if a.ndim == 0 or b.ndim == 0:
        out_shape = b.shape if a.ndim == 0 else a.shape
    else:
        out_shape = a.shape[: a.ndim - reduction_axes] + b.shape[reduction_axes:]
    out = np.zeros(out_shape, np.float32)
    lib().oracle_dot_general(_p(a), _p(ad), a.ndim, _p(b), _p(bd), b.ndim, reduction_axes, _p(out))
    return out


def gemm_nt_f64(a, bt):
    a = _c(a, np.float32)
    bt = _c(bt, np.float32)
    out = np.empty((a.shape[0], bt.shape[0]), np.float64)
    lib().oracle_gemm_nt_f64(_p(a), _p(bt), _p(out), a.shape[0], bt.shape[0], a.shape[1])
    return out


def w4a16_gemm(a, wq, scales, group=128, zp=8, threads=0, f32_out=False):
    a16 = _c(a.view(np.uint16), np.uint16)
    wq = _c(wq, np.uint8)
    s = _c(scales.view(np.uint16), np.uint16)
    m, k = a16.shape
    n = wq.shape[0]
    if f32_out:
        out = np.empty((m, n), np.float32)
        lib().oracle_w4a16_gemm_f32(_p(a16), _p(wq), _p(s), _p(out), m, n, k, group, zp, threads)
        return out
    out = np.empty((m, n), np.uint16)
    lib().oracle_w4a16_gemm(_p(a16), _p(wq), _p(s), _p(out), m, n, k, group, zp, threads)
    return out.view(np.float16)


def dequantize_wn(wq, scales, bits, group, zp=8, zero_points=None):
    """fp32 [N, K] = (q - zero point) * scale for 4- or 8-bit weights, any group size that divides K, a scalar zero point
    or one per (row, group) (u8; bits = 4: packed two per byte along the groups, low nibble = even group)."""
    wq = _c(wq, np.uint8)
    s = _c(scales.view(np.uint16), np.uint16)
    n = wq.shape[0]
    k = wq.shape[1] * 8 // bits
    assert bits in (4, 8) and k % group == 0 and s.shape == (n, k // group)
    z = None if zero_points is None else _c(zero_points, np.uint8)
    assert z is None or z.shape == (n, (k // group * bits + 7) // 8)
    out = np.empty((n, k), np.float32)
    lib().oracle_dequantize_wn(_p(wq), _p(s), None if z is None else _p(z), n, k, bits, group, zp, _p(out))
    return out


def wna16_gemm(a, wq, scales, bits, group, zp=8, zero_points=None, threads=0, f32_out=False):
    """Y = A . dequantize_wn(W)^T, accumulated in fp32; fp32, or rounded to fp16 as the output tensor type asks."""
    a16 = _c(a.view(np.uint16), np.uint16)
    wq = _c(wq, np.uint8)
    s = _c(scales.view(np.uint16), np.uint16)
    m, k = a16.shape
    n = wq.shape[0]
    assert wq.shape[1] * 8 // bits == k and k % group == 0
    z = None if zero_points is None else _c(zero_points, np.uint8)
    out = np.empty((m, n), np.float32 if f32_out else np.uint16)
    lib().oracle_wna16_gemm(_p(a16), _p(wq), _p(s), None if z is None else _p(z), _p(out), m, n, k, bits, group, zp,
                            0 if f32_out else 1, threads)
    return out if f32_out else out.view(np.float16)


def w8a8_acc(a, w, threads=0):
    a = _c(a, np.int8)
    w = _c(w, np.int8)
    out = np.empty((a.shape[0], w.shape[0]), np.int32)
    lib().oracle_w8a8_acc(_p(a), _p(w), _p(out), a.shape[0], w.shape[0], a.shape[1], threads)
    return out


def w8a8_acc_i64(a, w):
    a = _c(a, np.int8)
    w = _c(w, np.int8)
    out = np.empty((a.shape[0], w.shape[0]), np.int64)
    lib().oracle_w8a8_acc_i64(_p(a), _p(w), _p(out), a.shape[0], w.shape[0], a.shape[1])
    return out


def w8a8_epilogue(acc, s_tok, s_ch):
    acc = _c(acc, np.int32)
    s_tok = _c(s_tok, np.float32)
    s_ch = _c(s_ch, np.float32)
    out = np.empty(acc.shape, np.uint16)
    lib().oracle_w8a8_epilogue(_p(acc), _p(s_tok), _p(s_ch), _p(out), acc.shape[0], acc.shape[1])
    return out.view(np.float16)


def w8a8_gemm(a, s_tok, w, s_ch, threads=0):
    return w8a8_epilogue(w8a8_acc(a, w, threads), s_tok, s_ch)


def rmsnorm_f16(x, gamma, eps=1e-6):
    x16 = _c(x.view(np.uint16), np.uint16)
    g16 = _c(gamma.view(np.uint16), np.uint16)
    out = np.empty(x16.shape, np.uint16)
    lib().oracle_rmsnorm_f16(_p(x16), _p(g16), eps, _p(out), x16.shape[0], x16.shape[1])
    return out.view(np.float16)


def silu_mul_f16(g, u):
    g16 = _c(g.view(np.uint16), np.uint16)
    u16 = _c(u.view(np.uint16), np.uint16)
    out = np.empty(g16.shape, np.uint16)
    lib().oracle_silu_mul_f16(_p(g16), _p(u16), _p(out), g16.size)
    return out.view(np.float16)


def add_f16(a, b):
    a16 = _c(a.view(np.uint16), np.uint16)
    b16 = _c(b.view(np.uint16), np.uint16)
    out = np.empty(a16.shape, np.uint16)
    lib().oracle_add_f16(_p(a16), _p(b16), _p(out), a16.size)
    return out.view(np.float16)


def fused_mlp_w4a16(x, gamma, wgu, sgu, wd, sd, eps=1e-6, group=128, zp=8, threads=0, return_h=False):
    x16 = _c(x.view(np.uint16), np.uint16)
    g16 = _c(gamma.view(np.uint16), np.uint16)
    wgu = _c(wgu, np.uint8)
    wd = _c(wd, np.uint8)
    sgu16 = _c(sgu.view(np.uint16), np.uint16)
    sd16 = _c(sd.view(np.uint16), np.uint16)
    m, h = x16.shape
    i = wgu.shape[0] // 2
    out = np.empty((m, h), np.uint16)
    hbuf = np.empty((m, i), np.uint16)
    lib().oracle_fused_mlp_w4a16(_p(x16), _p(g16), eps, _p(wgu), _p(sgu16), _p(wd), _p(sd16), _p(out), _p(hbuf),
                                 m, h, i, group, zp, threads)
    if return_h:
        return out.view(np.float16), hbuf.view(np.float16)
    return out.view(np.float16)


def time_dot_f32(a, bt, warmup=5, iters=100, threads=0):
    """(mean_ms, min_ms) of C = a . bt^T with the oracle's own GEMM."""
    a = _c(a, np.float32)
    bt = _c(bt, np.float32)
    c = np.empty((a.shape[0], bt.shape[0]), np.float32)
    mn = ctypes.c_double(0)
    mean = lib().oracle_time_dot_f32(_p(a), _p(bt), _p(c), a.shape[0], bt.shape[0], a.shape[1], warmup, iters,
                                     threads, ctypes.addressof(mn))
    return mean, mn.value


def mlas_sgemm(a, b, trans_a=False, trans_b=False):
    """MlasGemm exactly as cpu::DotMlas emits it; requires oracle/_ref."""
    L = mlas_ref()
    a = _c(a, np.float32)
    b = _c(b, np.float32)
    m, k = (a.shape[1], a.shape[0]) if trans_a else a.shape
    n = b.shape[0] if trans_b else b.shape[1]
    out = np.empty((m, n), np.float32)
    lda = m if trans_a else k
    ldb = k if trans_b else n
    L.mlas_ref_sgemm(int(trans_a), int(trans_b), m, n, k, _p(a), lda, _p(b), ldb, _p(out), n)
    return out


def mlas_time_sgemm_nt(a, bt, warmup=5, iters=100):
    L = mlas_ref()
    a = _c(a, np.float32)
    bt = _c(bt, np.float32)
    c = np.empty((a.shape[0], bt.shape[0]), np.float32)
    mn = ctypes.c_double(0)
    mean = L.mlas_ref_time_sgemm_nt(a.shape[0], bt.shape[0], a.shape[1], _p(a), _p(bt), _p(c), warmup, iters,
                                    ctypes.addressof(mn))
    return mean, mn.value


def mlas_qgemm_s8s8(a, w):
    """int8 x int8 -> int32 through MLAS's u8 x s8 routine: a is shifted by +128 with zero point 128."""
    L = mlas_ref()
    a = _c(a, np.int8)
    w = _c(w, np.int8)
    m, k = a.shape
    n = w.shape[0]
    au = (a.astype(np.int16) + 128).astype(np.uint8)
    b = np.ascontiguousarray(w.T)  # [K,N]
    out = np.empty((m, n), np.int32)
    L.mlas_ref_qgemm_u8s8(m, n, k, _p(au), k, 128, _p(b), n, 0, _p(out), n)
    return out
