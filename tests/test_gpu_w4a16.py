"""Parity of the fp16 x int4 GEMV/GEMM (HIP, through the C ABI) against the CPU oracle.

Tolerance (stated by the task): max|y - y_ref| <= 1e-2 * RMS(y_ref), y_ref = the fp32-accumulated
dequant-GEMM of the oracle (un-rounded fp32 output).
"""
import numpy as np
import pytest

import oracle
from nnfusion_amd import datagen

pytestmark = pytest.mark.gpu

TOL = 1e-2


@pytest.fixture(params=["auto", "valu_gemv", "mfma_skinny", "rows_gemv", "mfma_rows"])
def path(request):
    """Runs a test once per kernel family that can serve a few rows, through nnf_w4a16_gemm_variant; a family that does
    not take the shape skips the case (auto = the library's own choice;
    rows_gemv = the M = 1 row-streaming kernel; mfma_rows = the row-streaming MFMA kernel for M >= 2, in one launch
    or over ranges of K; mfma_skinny = the MFMA GEMV kernel, likewise)."""
    return request.param


_PATH_VARIANT = {"valu_gemv": "gemv_valu", "mfma_skinny": "gemv_mfma", "rows_gemv": "gemv_rows", "mfma_rows": "gemv_rows"}


def _run(gpu, a, wq, s, zp=8, path="auto"):
    import torch

    from nnfusion_amd import ops

    m, k = a.shape
    n = wq.shape[0]
    ta, tw, ts = torch.from_numpy(a).to(gpu), torch.from_numpy(wq).to(gpu), torch.from_numpy(s).to(gpu)
    variant = _PATH_VARIANT.get(path)
    if variant is None:
        y = ops.w4a16_gemm(ta, tw, ts, zp=zp)
    else:
        # a kernel that does not take the shape is not a case of its own: the library's choice has its own parameter
        if path == "rows_gemv" and m != 1 or path == "mfma_rows" and m == 1 or not ops.w4a16_variant_supported(m, n, k, variant):
            pytest.skip(f"{path} does not take M={m} N={n} K={k}")
        y = ops.w4a16_gemm_variant(ta, tw, ts, variant, zp=zp)
    torch.cuda.synchronize()
    return y.cpu().numpy()


def _check(y, ref):
    rms = float(np.sqrt(np.mean(ref.astype(np.float64) ** 2)))
    err = float(np.abs(y.astype(np.float32) - ref).max())
    assert err <= TOL * max(rms, 1e-6), (err, rms)
    return err, rms


@pytest.mark.parametrize("m,n,k", [
    (1, 4096, 4096),      # configs[0]
    (1, 12288, 4096), (1, 22016, 4096), (1, 4096, 11008),  # configs[1]
    (1, 7, 128), (1, 1, 256), (2, 33, 384), (3, 100, 2048), (4, 257, 2176),
    (5, 64, 4096), (7, 130, 1024), (8, 512, 8192), (16, 1024, 8192),
    (16, 256, 1024), (12, 96, 2048), (16, 48, 3072), (9, 400, 512),  # more rows than wavefronts in the workgroup
    (16, 1040, 8192), (8, 520, 8192), (13, 77, 4096), (16, 64, 16384),  # activations too large for LDS: K in ranges
    (8, 100, 11008), (16, 260, 11008), (12, 64, 13824), (16, 48, 8320), (9, 33, 5248),  # ... with a shorter last range
    (4, 300, 8192), (3, 200, 12288), (2, 96, 6144),  # two passes over K per tile
    # one activation row: rows shared by 1, 2, 4 wavefronts, ragged last K segment, fewer rows than wavefronts,
    # more rows per wavefront than one chunk of scales holds
    (1, 300, 1024), (1, 4096, 8192), (1, 1000, 2048), (1, 5000, 1280), (1, 513, 5120), (1, 2000, 14336),
    (1, 4100, 16384), (1, 151936, 1024), (1, 80000, 3072), (1, 40, 4096),
    # a handful of rows through the row-streaming MFMA kernel: every K it takes, ragged N, more tiles than CUs,
    # fewer tiles than CUs, a single tile
    (2, 4096, 1024), (3, 8200, 2048), (16, 4111, 4096), (9, 22016, 4096), (16, 12288, 8192), (6, 16, 8192), (11, 48, 2048),
    (16, 40000, 1024), (5, 4096, 3072), (16, 13824, 5120), (7, 1000, 6144), (16, 2050, 7168), (2, 640, 5120),
    # K a multiple of 256 but not of 1024 (and 5120 / 7168 above): the run-time-K form, wavefronts past the end of K
    (3, 77, 3584), (16, 520, 2560), (9, 16, 1280), (11, 333, 4352), (5, 1000, 7936), (16, 18944, 3584),
    # K above 8192: ranges of K on the run-time-K form, fp32 partial sums, reduction pass
    (16, 4111, 11008), (8, 1000, 14336), (16, 300, 28672), (7, 4096, 11008), (12, 333, 8448), (6, 16, 16384),
    # 17 .. 32 rows over ranges of K (K above 4096), and in one launch with a run-time K
    (32, 4111, 8192), (17, 1000, 11008), (24, 300, 14336), (32, 520, 5120), (20, 77, 3584), (31, 2000, 2560),
    # 33 .. 40 rows over ranges of K (four blocks of 16; 2048 < K <= 4096)
    (33, 4111, 4096), (40, 1000, 3072), (36, 300, 3584), (40, 77, 2560), (38, 22016, 4096),
    # 17 .. 32 rows (two blocks of 16), K <= 4096
    (17, 4096, 4096), (32, 22016, 4096), (24, 1000, 2048), (31, 77, 3072), (32, 300, 1024),
])
def test_gemv_matches_oracle(gpu, path, m, n, k):
    print(f"case M={m} N={n} K={k}", flush=True)
    a, wq, s = datagen.w4a16_case(0, m, n, k)
    y = _run(gpu, a, wq, s, path=path)
    ref = oracle.w4a16_gemm(a, wq, s, f32_out=True)
    _check(y, ref)


@pytest.mark.parametrize("log2_scale", [-12, -16])
@pytest.mark.parametrize("m,n,k", [(1, 4096, 4096), (1, 512, 11008), (4, 300, 2048), (16, 1040, 8192), (16, 520, 11008),
                                   (24, 300, 4096), (24, 300, 8192), (36, 300, 3584)])
def test_gemv_small_activations_lose_nothing(gpu, path, m, n, k, log2_scale):
    """Activations scaled down by 2^12 and 2^16 (into and below the fp16 subnormal range), on every kernel family
    and on the forms over ranges of K: no kernel may rescale them on the way (a 1/16 on the activations of the high
    nibbles would drop their low bits below 2^-10).  Same tolerance as everywhere, against the oracle on the same
    fp16 inputs."""
    a, wq, s = datagen.w4a16_case(9, m, n, k)
    a = (a.astype(np.float32) * np.float32(2.0 ** log2_scale)).astype(np.float16)
    y = _run(gpu, a, wq, s, path=path)
    ref = oracle.w4a16_gemm(a, wq, s, f32_out=True)
    _check(y, ref)


def test_gemv_very_large_n_parks_outputs_in_more_workgroups(gpu):
    """N so large that one workgroup per CU could not park its tiles' outputs in LDS: the launcher uses more,
    shorter workgroups.  Checked on sampled columns."""
    import torch

    from nnfusion_amd import ops

    m, n, k = 16, 500000, 128
    a, wq, s = datagen.w4a16_case(3, m, n, k)
    y = ops.w4a16_gemm(torch.from_numpy(a).to(gpu), torch.from_numpy(wq).to(gpu), torch.from_numpy(s).to(gpu))
    torch.cuda.synchronize()
    cols = np.sort(np.random.default_rng(5).choice(n, 4096, replace=False))
    cols[:32] = np.arange(32)
    cols[-32:] = np.arange(n - 32, n)
    ref = oracle.w4a16_gemm(a, wq[cols], s[cols], f32_out=True)
    _check(y.cpu().numpy()[:, cols], ref)


def test_gemv_all_zero_point_is_zero(gpu, path):
    # every q == zp  =>  Y == 0: exactly on the VALU path (it dequantises to the exact integer
    # q - zp); the MFMA path removes the 1024 + zp offset of its operand encoding from the fp32
    # group sum, which leaves fp32 rounding residue: bounded here at 2e-4 of the RMS a random
    # weight matrix of this K would give (50x below the parity tolerance).
    k = 512
    a, wq, s = datagen.w4a16_case(1, 2, 96, k)
    wq[:] = 0x88
    y = _run(gpu, a, wq, s, path=path)
    if path == "valu_gemv":
        assert np.all(y == 0)
    else:
        rms_typical = np.sqrt(k * 21.25 * 1.75e-4)
        assert np.abs(y.astype(np.float32)).max() <= 2e-4 * rms_typical


def test_gemv_one_hot_reads_single_weight(gpu, path):
    # A = e_k  =>  Y[n] = fp16((q[n,k]-8) * s[n,k/128]) : pins nibble order and scale indexing
    n, k = 64, 512
    _, wq, s = datagen.w4a16_case(2, 1, n, k)
    wd = oracle.dequantize_w4(wq, s)
    for kk in (0, 1, 2, 7, 8, 31, 32, 127, 128, 129, 255, 511):
        a = np.zeros((1, k), np.float16)
        a[0, kk] = 1.0
        y = _run(gpu, a, wq, s, path=path)
        np.testing.assert_array_equal(y[0], wd[:, kk].astype(np.float16))


@pytest.mark.parametrize("zp", [0, 7, 15])
def test_gemv_other_zero_points(gpu, path, zp):
    a, wq, s = datagen.w4a16_case(3, 2, 128, 1024)
    y = _run(gpu, a, wq, s, zp=zp, path=path)
    ref = oracle.w4a16_gemm(a, wq, s, zp=zp, f32_out=True)
    _check(y, ref)


@pytest.mark.parametrize("m,n,k", [(1, 512, 4096), (8, 300, 2048), (16, 128, 8192), (40, 256, 1024), (8, 300, 3072), (8, 300, 2176), (24, 300, 4096), (24, 300, 8192)])
def test_every_kernel_variant_that_accepts_a_shape_matches_the_oracle(gpu, m, n, k):
    """nnf_w4a16_gemm_variant: the entry point behind the per-variant emitters of profiling-based kernel selection.
    nnf_w4a16_variant_supported (host only) and the call itself agree on which variants serve a shape."""
    import torch

    from nnfusion_amd import _lib, ops

    a, wq, s = datagen.w4a16_case(0, m, n, k)
    ref = oracle.w4a16_gemm(a, wq, s, f32_out=True)
    ta, tw, ts = (torch.from_numpy(x).to(gpu) for x in (a, wq, s))
    served = []
    for name, v in ops.VARIANTS.items():
        ok = _lib.kernels().nnf_w4a16_variant_supported(m, n, k, 128, v)
        if ok:
            y = ops.w4a16_gemm_variant(ta, tw, ts, name)
            torch.cuda.synchronize()
            _check(y.cpu().numpy(), ref)
            served.append(name)
        else:
            with pytest.raises(ops.NnfError) as e:
                ops.w4a16_gemm_variant(ta, tw, ts, name)
            assert e.value.status == -2
    assert "auto" in served and "gemm_mfma" in served
    assert ("gemv_rows" in served) == (m == 1 or (m <= 32 and k % 256 == 0 and k >= 1024))
    assert ("gemv_valu" in served) == (m <= 16)
