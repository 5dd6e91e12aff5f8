"""Pins the oracle's fp32 Dot against the vectors the reference's own tests hold, against the reference's
MLAS (oracle/_ref, when built) and against fp64 brute force."""
import json
import os

import numpy as np
import pytest

import oracle

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _cases():
    with open(os.path.join(GOLDEN, "dot_inventory.json")) as f:
        return json.load(f)["cases"]


@pytest.mark.parametrize("case", _cases(), ids=lambda c: f"inventory{c['case']}")
def test_dot_inventory_known_answers(case):
    """test/nnfusion/inventory/dot.cpp: default op::Dot contracts one axis (none if an argument is a scalar)."""
    a = np.array(case["a"], np.float32).reshape(case["shape_a"])
    b = np.array(case["b"], np.float32).reshape(case["shape_b"])
    r = 0 if (a.ndim == 0 or b.ndim == 0) else 1
    out = oracle.dot_general(a, b, r)
    expected = np.array(case["expected"], np.float32)
    assert out.size == expected.size
    np.testing.assert_array_equal(out.ravel(), expected)
    # 2-D cases also go through the MlasGemm-shaped entry point (and its transposed forms)
    if a.ndim == 2 and b.ndim == 2:
        np.testing.assert_array_equal(oracle.dot_f32(a, b).ravel(), expected)
        np.testing.assert_array_equal(oracle.dot_f32(a, np.ascontiguousarray(b.T), trans_b=True).ravel(), expected)
        np.testing.assert_array_equal(oracle.dot_f32(np.ascontiguousarray(a.T), b, trans_a=True).ravel(), expected)
    if a.ndim == 2 and b.ndim == 1:
        np.testing.assert_array_equal(oracle.dot_f32(a, b.reshape(-1, 1)).ravel(), expected)


def test_onnx_gemm_vector_with_both_transposes():
    """test/nnfusion/frontend/onnx_import.cpp gemm_op: alpha * a^T . b^T + beta * c (tolerance of the
    reference's all_close_f on values printed with 6 digits)."""
    with open(os.path.join(GOLDEN, "onnx_gemm_op.json")) as f:
        g = json.load(f)
    a = np.array(g["a"], np.float32).reshape(g["a_shape"])
    b = np.array(g["b"], np.float32).reshape(g["b_shape"])
    c = np.array(g["c"], np.float32).reshape(g["c_shape"])
    d = oracle.dot_f32(a, b, trans_a=True, trans_b=True)
    out = g["alpha"] * d + g["beta"] * c
    np.testing.assert_allclose(out.ravel(), np.array(g["expected"], np.float32), rtol=0, atol=2e-6)


def test_tensorflow_matmul_vector():
    """test/nnfusion/frontend/tensorflow_import.cpp:250-268 (matmul_op): A = 1..12 as (3,4), B = 13..24 as
    (4,3), expected {{190,200,210},{470,496,522},{750,792,834}}."""
    a = np.arange(1, 13, dtype=np.float32).reshape(3, 4)
    b = np.arange(13, 25, dtype=np.float32).reshape(4, 3)
    np.testing.assert_array_equal(oracle.dot_f32(a, b), np.array([[190, 200, 210], [470, 496, 522], [750, 792, 834]], np.float32))


@pytest.mark.parametrize("m,n,k", [(1, 64, 128), (7, 33, 200), (16, 100, 1024), (3, 5, 4096)])
@pytest.mark.parametrize("trans_a,trans_b", [(False, False), (False, True), (True, False), (True, True)])
def test_dot_matches_fp64_brute_force(m, n, k, trans_a, trans_b):
    rng = np.random.default_rng(m * 1000 + n + k)
    a = rng.standard_normal((k, m) if trans_a else (m, k)).astype(np.float32)
    b = rng.standard_normal((n, k) if trans_b else (k, n)).astype(np.float32)
    out = oracle.dot_f32(a, b, trans_a, trans_b)
    a64 = (a.T if trans_a else a).astype(np.float64)
    b64 = (b.T if trans_b else b).astype(np.float64)
    ref = a64 @ b64
    # fp32 accumulation error bound ~ K * eps * |a|.|b|
    bound = 4 * k * np.finfo(np.float32).eps * (np.abs(a64) @ np.abs(b64))
    assert np.all(np.abs(out - ref) <= bound + 1e-30)


@pytest.mark.skipif(oracle.mlas_ref() is None, reason="oracle/_ref (the reference's MLAS) is not built")
@pytest.mark.parametrize("m,n,k", [(1, 4096, 4096), (16, 512, 1024), (5, 77, 333), (128, 256, 512)])
def test_dot_matches_reference_mlas(m, n, k):
    """MlasGemm(NoTrans, Trans, ...) of the reference tree vs the oracle: same fp32 semantics, different
    summation order => agreement to fp32 accumulation accuracy."""
    rng = np.random.default_rng(k + n)
    a = rng.standard_normal((m, k)).astype(np.float32)
    bt = (rng.standard_normal((n, k)) * 0.1).astype(np.float32)
    ref = oracle.mlas_sgemm(a, bt, trans_b=True)
    out = oracle.dot_f32(a, bt, trans_b=True)
    scale = np.abs(a.astype(np.float64)) @ np.abs(bt.astype(np.float64)).T
    assert np.all(np.abs(out.astype(np.float64) - ref) <= 4 * k * np.finfo(np.float32).eps * scale)
    # non-transposed form too
    b = np.ascontiguousarray(bt.T)
    np.testing.assert_allclose(oracle.dot_f32(a, b), oracle.mlas_sgemm(a, b), rtol=0, atol=float(scale.max()) * 1e-5)


@pytest.mark.skipif(oracle.mlas_ref() is None, reason="oracle/_ref (the reference's MLAS) is not built")
def test_config0_w4a16_matches_dequant_plus_reference_mlas():
    """configs[0] (M=1, N=K=4096, seed 0): oracle vs  dequantize (reference formula) -> reference MlasGemm."""
    from nnfusion_amd import datagen

    a, wq, s = datagen.w4a16_case(0, 1, 4096, 4096)
    y = oracle.w4a16_gemm(a, wq, s, f32_out=True)
    ref = oracle.mlas_sgemm(a.astype(np.float32), oracle.dequantize_w4(wq, s), trans_b=True)
    rms = float(np.sqrt(np.mean(ref.astype(np.float64) ** 2)))
    assert 3.5 < rms < 4.3  # sqrt(K * E[(q-8)^2] * E[s^2]) = 3.9 for this configuration
    assert np.abs(y - ref).max() <= 1e-5 * rms
