"""Pins the oracle's quantised arithmetic (no reference test covers it): closed forms, invariants, brute
force in int64 / fp64, and the reference's MLAS u8 x s8 GEMM where oracle/_ref is built."""
import numpy as np
import pytest

import oracle
from nnfusion_amd import datagen


def test_f16_conversions_exhaustive():
    bits = np.arange(65536, dtype=np.uint16)
    f = oracle.f16_to_f32(bits.view(np.float16))
    ref = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(ref)
    np.testing.assert_array_equal(f[~nan], ref[~nan])
    assert np.all(np.isnan(f[nan]))
    back = oracle.f32_to_f16(f).view(np.uint16)
    np.testing.assert_array_equal(back[~nan], bits[~nan])


def test_f32_to_f16_round_to_nearest_even_matches_numpy():
    rng = np.random.default_rng(0)
    x = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * 10.0,
        (rng.standard_normal(100000) * 1e-5).astype(np.float32),      # fp16 subnormals
        np.array([65504, 65519.99, 65520, 1e9, -1e9, 0.0, -0.0, 2.0 ** -24, 2.0 ** -25, 1.5 * 2.0 ** -25,
                  1 + 2.0 ** -11, 1 + 3 * 2.0 ** -11], np.float32),   # overflow edge, ties
    ])
    with np.errstate(over="ignore"):
        ref = x.astype(np.float16)
    np.testing.assert_array_equal(oracle.f32_to_f16(x).view(np.uint16), ref.view(np.uint16))
    # the generator's own converter (host library) agrees as well
    from nnfusion_amd import _lib

    h = _lib.host()
    for v in x[-12:]:
        assert h.nnf_f32_to_f16_bits(float(v)) == int(np.float32(v).astype(np.float16).view(np.uint16))


def _python_dequant(wq, s, group, zp):
    n, kb = wq.shape
    out = np.zeros((n, kb * 2), np.float32)
    for i in range(n):
        for b in range(kb):
            for nib in range(2):
                k = 2 * b + nib
                q = (int(wq[i, b]) >> (4 * nib)) & 0xF
                out[i, k] = np.float32(q - zp) * np.float32(s[i, k // group])
    return out


def test_dequantize_w4_brute_force_and_nibble_order():
    a, wq, s = datagen.w4a16_case(11, 1, 6, 256)
    out = oracle.dequantize_w4(wq, s)
    np.testing.assert_array_equal(out, _python_dequant(wq, s, 128, 8))
    # low nibble = even k: swapping the nibbles of every byte must swap neighbouring columns
    swapped = ((wq >> 4) | (wq << 4)).astype(np.uint8)
    out_sw = oracle.dequantize_w4(swapped, s)
    np.testing.assert_array_equal(out_sw[:, 0::2], out[:, 1::2])
    np.testing.assert_array_equal(out_sw[:, 1::2], out[:, 0::2])
    assert not np.array_equal(out_sw, out)
    # other zero points
    for zp in (0, 3, 15):
        np.testing.assert_array_equal(oracle.dequantize_w4(wq, s, zp=zp), _python_dequant(wq, s, 128, zp))


def test_w4a16_invariants():
    m, n, k = 3, 40, 384
    a, wq, s = datagen.w4a16_case(12, m, n, k)
    # all q == zp -> exactly zero
    z = np.full_like(wq, 0x88)
    assert np.all(oracle.w4a16_gemm(a, z, s, f32_out=True) == 0)
    # one-hot activation picks one dequantised weight
    wd = oracle.dequantize_w4(wq, s)
    for kk in (0, 1, 127, 128, 383):
        e = np.zeros((1, k), np.float16)
        e[0, kk] = 1
        np.testing.assert_array_equal(oracle.w4a16_gemm(e, wq, s, f32_out=True)[0], wd[:, kk])
    # scale 1, q = 9 -> Y[m, n] = sum_k a[m, k] (fp32 sum of fp16 values; compare with fp64)
    ones = np.ones_like(s)
    nine = np.full_like(wq, 0x99)
    y = oracle.w4a16_gemm(a, nine, ones, f32_out=True)
    ref = a.astype(np.float64).sum(axis=1, keepdims=True).repeat(n, axis=1)
    np.testing.assert_allclose(y, ref, rtol=0, atol=1e-3)
    # linear in the scales: doubling every scale doubles the fp32 result exactly
    np.testing.assert_array_equal(oracle.w4a16_gemm(a, wq, (s * 2).astype(np.float16), f32_out=True),
                                  2 * oracle.w4a16_gemm(a, wq, s, f32_out=True))
    # against fp64 end to end
    ref64 = a.astype(np.float64) @ wd.astype(np.float64).T
    yy = oracle.w4a16_gemm(a, wq, s, f32_out=True)
    assert np.abs(yy - ref64).max() <= 1e-4
    # fp16 output = RNE of the fp32 result
    np.testing.assert_array_equal(oracle.w4a16_gemm(a, wq, s).view(np.uint16), yy.astype(np.float16).view(np.uint16))


def test_w8a8_accumulators_against_int64_and_numpy():
    a, s_tok, w, s_ch = datagen.w8a8_case(13, 9, 70, 640)
    acc = oracle.w8a8_acc(a, w)
    np.testing.assert_array_equal(acc, oracle.w8a8_acc_i64(a, w))
    np.testing.assert_array_equal(acc, a.astype(np.int64) @ w.astype(np.int64).T)
    # extreme values at K = 8192 stay inside int32
    a2 = np.full((1, 8192), -127, np.int8)
    w2 = np.full((2, 8192), 127, np.int8)
    w2[1] = -127
    np.testing.assert_array_equal(oracle.w8a8_acc(a2, w2), [[-8192 * 127 * 127, 8192 * 127 * 127]])


@pytest.mark.skipif(oracle.mlas_ref() is None, reason="oracle/_ref (the reference's MLAS) is not built")
def test_w8a8_accumulators_against_reference_mlas_qgemm():
    """MlasGemm u8 x s8 -> s32 (thirdparty/mlas/inc/mlas.h:147-163) with A shifted by +128 and zero point 128."""
    a, _, w, _ = datagen.w8a8_case(14, 17, 96, 1024)
    np.testing.assert_array_equal(oracle.w8a8_acc(a, w), oracle.mlas_qgemm_s8s8(a, w))


def test_w8a8_epilogue_closed_form():
    acc = np.array([[132128768, -132128768, 1, 0, 95637]], np.int32)
    s_tok = np.array([0.009587127], np.float32)
    s_ch = np.array([0.0044499394, 0.001, 0.01, 0.5, 0.0044499394], np.float32)
    out = oracle.w8a8_epilogue(acc, s_tok, s_ch)
    ref = ((acc.astype(np.float32) * s_tok[:, None]).astype(np.float32) * s_ch[None, :]).astype(np.float32)
    with np.errstate(over="ignore"):
        np.testing.assert_array_equal(out.view(np.uint16), ref.astype(np.float16).view(np.uint16))
    # (float)acc rounds above 2^24: 132128768 is representable, 132128769 is not
    assert np.float32(132128769) == np.float32(132128768)


def test_rmsnorm_silu_add_closed_forms():
    m, k = 5, 512
    x = datagen.normal_f16(15, 1, (m, k))
    g = datagen.normal_f16(15, 2, (k,), 1.0, 0.1)
    out = oracle.rmsnorm_f16(x, g, 1e-6).astype(np.float64)
    x64, g64 = x.astype(np.float64), g.astype(np.float64)
    ref = x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + 1e-6) * g64
    assert np.abs(out - ref).max() <= 2.0 ** -10 * np.abs(ref).max()
    # a constant row c has RMS |c|: out = sign(c) * gamma
    xc = np.full((1, k), 3.0, np.float16)
    np.testing.assert_allclose(oracle.rmsnorm_f16(xc, g, 0.0).astype(np.float32), g.astype(np.float32)[None, :],
                               rtol=2.0 ** -10)
    gg = datagen.normal_f16(15, 3, (1000,), 0.0, 3.0)
    uu = datagen.normal_f16(15, 4, (1000,), 0.0, 3.0)
    h = oracle.silu_mul_f16(gg, uu).astype(np.float64)
    g64, u64 = gg.astype(np.float64), uu.astype(np.float64)
    refh = g64 / (1 + np.exp(-g64)) * u64
    assert np.all(np.abs(h - refh) <= 2.0 ** -10 * np.abs(refh) + 1e-7)
    assert oracle.lib().oracle_sigmoid(0.0) == 0.5
    np.testing.assert_array_equal(oracle.add_f16(gg, uu).view(np.uint16),
                                  (gg.astype(np.float32) + uu.astype(np.float32)).astype(np.float16).view(np.uint16))


def test_fused_mlp_is_the_composition_of_its_nodes():
    m, h, i = 4, 256, 384
    x, gamma, wgu, sgu, wd, sd = datagen.mlp_case(16, m, h, i)
    out, hbuf = oracle.fused_mlp_w4a16(x, gamma, wgu, sgu, wd, sd, return_h=True)
    xn = oracle.rmsnorm_f16(x, gamma, 1e-6)
    gu = oracle.w4a16_gemm(xn, wgu, sgu)
    hh = oracle.silu_mul_f16(np.ascontiguousarray(gu[:, :i]), np.ascontiguousarray(gu[:, i:]))
    np.testing.assert_array_equal(hbuf.view(np.uint16), hh.view(np.uint16))
    d = oracle.w4a16_gemm(hh, wd, sd)
    np.testing.assert_array_equal(out.view(np.uint16), oracle.add_f16(d, x).view(np.uint16))


# ---- the general form: 4 / 8 bits, groups of 32 / 64 / 128, scalar or per-(row, group) zero points ---------------------
def _rand_quant_case(seed, n, k, bits, group, zp_tensor):
    rng = np.random.default_rng(seed)
    wq = rng.integers(0, 256, (n, k * bits // 8), dtype=np.uint8)
    s = (rng.uniform(0.005, 0.02, (n, k // group))).astype(np.float16)
    g = k // group
    zps = rng.integers(0, 256, (n, (g * bits + 7) // 8), dtype=np.uint8) if zp_tensor else None
    return wq, s, zps


def _python_dequant_wn(wq, s, zps, bits, group, zp):
    """Element by element, from the definition: q and the zero point are unpacked with shifts, subtracted as integers,
    cast, multiplied by the scale of the block (cpu_reference_dequantize)."""
    n = wq.shape[0]
    k = wq.shape[1] * 8 // bits
    out = np.zeros((n, k), np.float32)
    for i in range(n):
        for kk in range(k):
            if bits == 4:
                q = (int(wq[i, kk // 2]) >> (4 * (kk % 2))) & 0xF
            else:
                q = int(wq[i, kk])
            g = kk // group
            if zps is None:
                z = zp
            elif bits == 4:
                z = (int(zps[i, g // 2]) >> (4 * (g % 2))) & 0xF
            else:
                z = int(zps[i, g])
            out[i, kk] = np.float32(q - z) * np.float32(s[i, g])
    return out


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("group", [32, 64, 128])
@pytest.mark.parametrize("zp_tensor", [False, True])
def test_dequantize_wn_brute_force(bits, group, zp_tensor):
    wq, s, zps = _rand_quant_case(bits * 1000 + group + zp_tensor, 5, 384, bits, group, zp_tensor)
    zp = 8 if bits == 4 else 128
    out = oracle.dequantize_wn(wq, s, bits, group, zp=zp, zero_points=zps)
    np.testing.assert_array_equal(out, _python_dequant_wn(wq, s, zps, bits, group, zp))


def test_dequantize_wn_reduces_to_the_w4_g128_form():
    _, wq, s = datagen.w4a16_case(12, 1, 9, 512)
    np.testing.assert_array_equal(oracle.dequantize_wn(wq, s, 4, 128, zp=8), oracle.dequantize_w4(wq, s))
    # ... and a zero-point tensor that holds the scalar everywhere changes nothing
    zps = np.full((9, 2), 0x88, np.uint8)
    np.testing.assert_array_equal(oracle.dequantize_wn(wq, s, 4, 128, zero_points=zps), oracle.dequantize_w4(wq, s))


def test_dequantize_wn_element_and_zero_point_order():
    """One weight / one zero point set at a time: pins byte and nibble order of both tensors and the block a scale and
    a zero point belong to."""
    n, k = 3, 256
    for bits, group in ((4, 32), (4, 64), (8, 32), (8, 128)):
        g = k // group
        s = (np.arange(n * g, dtype=np.float32).reshape(n, g) + 1).astype(np.float16)  # every block its own scale
        zero = np.zeros((n, k * bits // 8), np.uint8)
        zps0 = np.zeros((n, (g * bits + 7) // 8), np.uint8)
        for (row, kk) in ((0, 0), (1, 1), (2, 33), (1, 255), (0, 130)):
            wq = zero.copy()
            if bits == 4:
                wq[row, kk // 2] = 5 << (4 * (kk % 2))
            else:
                wq[row, kk] = 5
            out = oracle.dequantize_wn(wq, s, bits, group, zp=0, zero_points=zps0)
            want = np.zeros((n, k), np.float32)
            want[row, kk] = 5.0 * float(s[row, kk // group])
            np.testing.assert_array_equal(out, want)
        for (row, gg) in ((0, 0), (1, 1), (2, g - 1)):
            zps = zps0.copy()
            if bits == 4:
                zps[row, gg // 2] = 3 << (4 * (gg % 2))
            else:
                zps[row, gg] = 3
            out = oracle.dequantize_wn(zero, s, bits, group, zp=0, zero_points=zps)
            want = np.zeros((n, k), np.float32)
            want[row, gg * group:(gg + 1) * group] = -3.0 * float(s[row, gg])
            np.testing.assert_array_equal(out, want)


@pytest.mark.parametrize("bits,group,zp_tensor", [(4, 32, True), (4, 64, False), (8, 128, True), (8, 32, False), (4, 128, True)])
def test_wna16_gemm_against_fp64_and_one_hot(bits, group, zp_tensor):
    m, n, k = 7, 33, 512
    wq, s, zps = _rand_quant_case(77 + bits + group, n, k, bits, group, zp_tensor)
    zp = 8 if bits == 4 else 128
    a = datagen.normal_f16(5, datagen.S_ACT, (m, k))
    wd = _python_dequant_wn(wq, s, zps, bits, group, zp) if n * k <= 20000 else oracle.dequantize_wn(wq, s, bits, group, zp, zps)
    ref64 = a.astype(np.float64) @ wd.astype(np.float64).T
    y32 = oracle.wna16_gemm(a, wq, s, bits, group, zp=zp, zero_points=zps, f32_out=True)
    bound = 4 * k * 2.0 ** -24 * (np.abs(a.astype(np.float64)) @ np.abs(wd.astype(np.float64)).T) + 1e-30
    assert np.all(np.abs(y32 - ref64) <= bound)
    y16 = oracle.wna16_gemm(a, wq, s, bits, group, zp=zp, zero_points=zps)
    np.testing.assert_array_equal(y16.view(np.uint16), oracle.f32_to_f16(y32).view(np.uint16))
    # A = e_k picks column k of the dequantised weights, rounded to fp16
    for kk in (0, 1, 31, 32, 63, 64, 127, 128, 511):
        e = np.zeros((1, k), np.float16)
        e[0, kk] = 1.0
        y = oracle.wna16_gemm(e, wq, s, bits, group, zp=zp, zero_points=zps)
        np.testing.assert_array_equal(y[0], wd[:, kk].astype(np.float16))
