"""Seeded synthetic tensors of the benchmark configurations (numpy views over the C++ generator).

Every tensor of a configuration has its own stream id so that changing one shape does not shift
the bytes of another.  Distributions: activations ~ N(0,1) fp16; int4 weights uniform 0..15 packed
two per byte along K; group scales uniform [0.005, 0.02) fp16; W8A8 int8 uniform [-127,127] with
fp32 scales uniform [0.001, 0.01); RMSNorm gamma ~ N(1, 0.1) fp16.
"""
import numpy as np

from . import _lib

# stream ids
S_ACT, S_WQ, S_SCALE, S_GAMMA, S_A8, S_W8, S_STOK, S_SCH, S_WQ2, S_SCALE2, S_BIAS, S_RES, S_ZP = range(1, 14)


def _ptr(a):
    return a.ctypes.data


def normal_f16(seed, stream, shape, mean=0.0, std=1.0):
    out = np.empty(shape, dtype=np.uint16)
    _lib.host().nnf_gen_normal_f16(seed, stream, mean, std, _ptr(out), out.size)
    return out.view(np.float16)


def uniform_f16(seed, stream, shape, lo, hi):
    out = np.empty(shape, dtype=np.uint16)
    _lib.host().nnf_gen_uniform_f16(seed, stream, lo, hi, _ptr(out), out.size)
    return out.view(np.float16)


def uniform_f32(seed, stream, shape, lo, hi):
    out = np.empty(shape, dtype=np.float32)
    _lib.host().nnf_gen_uniform_f32(seed, stream, lo, hi, _ptr(out), out.size)
    return out


def uniform_u4_packed(seed, stream, n, k):
    """u8 [n, k/2]; low nibble of byte b holds k = 2b, high nibble k = 2b+1."""
    assert k % 2 == 0
    out = np.empty((n, k // 2), dtype=np.uint8)
    _lib.host().nnf_gen_uniform_u4_packed(seed, stream, _ptr(out), n * k)
    return out


def uniform_i8(seed, stream, shape, lo=-127, hi=127):
    out = np.empty(shape, dtype=np.int8)
    _lib.host().nnf_gen_uniform_i8(seed, stream, lo, hi, _ptr(out), out.size)
    return out


def w4a16_case(seed, m, n, k, group=128):
    """(A fp16 [m,k], Wq u8 [n,k/2], scales fp16 [n,k/group]) of the fp16 x int4 configurations."""
    a = normal_f16(seed, S_ACT, (m, k))
    wq = uniform_u4_packed(seed, S_WQ, n, k)
    s = uniform_f16(seed, S_SCALE, (n, k // group), 0.005, 0.02)
    return a, wq, s


def wna16_case(seed, m, n, k, bits, group, zero_points=False):
    """(A fp16 [m,k], Wq u8 [n,k*bits/8], scales fp16 [n,k/group], zero points u8 [n, ceil(k/group*bits/8)] or None) with
    4- or 8-bit weights: weights and zero points uniform over their whole range, scales uniform [0.005, 0.02) / 2^(bits-4)
    (the same spread of dequantised values for either width)."""
    assert bits in (4, 8) and k % group == 0
    a = normal_f16(seed, S_ACT, (m, k))
    g = k // group
    if bits == 4:
        wq = uniform_u4_packed(seed, S_WQ, n, k)
        z = uniform_u4_packed(seed, S_ZP, n, g + (g & 1)) if zero_points else None
    else:
        wq = uniform_i8(seed, S_WQ, (n, k), -128, 127).view(np.uint8)
        z = uniform_i8(seed, S_ZP, (n, g), -128, 127).view(np.uint8) if zero_points else None
    s = uniform_f16(seed, S_SCALE, (n, g), 0.005 / (1 << (bits - 4)), 0.02 / (1 << (bits - 4)))
    return a, wq, s, z


def w8a8_case(seed, m, n, k):
    """(A i8 [m,k], s_tok f32 [m], W i8 [n,k], s_ch f32 [n]) of the W8A8 configuration."""
    a = uniform_i8(seed, S_A8, (m, k))
    w = uniform_i8(seed, S_W8, (n, k))
    s_tok = uniform_f32(seed, S_STOK, (m,), 0.001, 0.01)
    s_ch = uniform_f32(seed, S_SCH, (n,), 0.001, 0.01)
    return a, s_tok, w, s_ch


def mlp_case(seed, m, h, i, group=128):
    """(x, gamma, Wgu [2i,h/2], Sgu, Wd [h,i/2], Sd) of the fused Llama MLP configuration."""
    x = normal_f16(seed, S_ACT, (m, h))
    gamma = normal_f16(seed, S_GAMMA, (h,), 1.0, 0.1)
    wgu = uniform_u4_packed(seed, S_WQ, 2 * i, h)
    sgu = uniform_f16(seed, S_SCALE, (2 * i, h // group), 0.005, 0.02)
    wd = uniform_u4_packed(seed, S_WQ2, h, i)
    sd = uniform_f16(seed, S_SCALE2, (h, i // group), 0.005, 0.02)
    return x, gamma, wgu, sgu, wd, sd
